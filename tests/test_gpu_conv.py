"""Parity of the quantized Conv2d forward (u8 x i8 -> i32 -> requantized i8) with the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


GEOMS = [
    # nb, c, h, w, oc, k, stride, pad, zp      (fast path: stride 1 and c % 32 == 0)
    (1, 128, 5, 5, 8, 3, (1, 1), (1, 1), 0),
    (3, 96, 10, 9, 40, 3, (1, 1), (1, 1), 77),     # three channel blocks: the tap walk wraps on a non-power of two
    (2, 32, 20, 20, 70, 5, (1, 1), (2, 2), 255),   # one channel block, 25 taps
    (1, 64, 33, 40, 8, 1, (1, 1), (0, 0), 1),      # 1x1: a plain matrix product over the pixels
    (1, 32, 70, 60, 33, 3, (1, 1), (1, 0), 128),   # padded rows of 60 pixels: the layout pass works in five bands
    (2, 160, 6, 5, 129, 2, (1, 1), (0, 1), 60),    # even kernel, k blocks padded up to a multiple of four
    (2, 128, 7, 6, 130, 3, (1, 1), (1, 1), 17),
    (1, 256, 6, 6, 64, 1, (1, 1), (0, 0), 3),
    (2, 128, 9, 8, 40, 5, (1, 1), (2, 2), 200),
    (1, 256, 14, 14, 32, 3, (1, 1), (0, 0), 128),
    # direct path
    (2, 3, 8, 8, 4, 3, (1, 1), (1, 1), 5),
    (1, 16, 9, 9, 6, 3, (2, 2), (1, 1), 0),
    (2, 128, 8, 8, 8, 3, (2, 1), (0, 1), 9),
    (1, 1, 3, 3, 1, 1, (1, 1), (0, 0), 0),
]


@pytest.mark.parametrize("nb,c,h,w,oc,k,stride,pad,zp", GEOMS)
def test_conv_accumulators_bit_exact(ctx, oracle, nb, c, h, w, oc, k, stride, pad, zp):
    rng = np.random.default_rng(nb * 7 + c + h * 3 + oc)
    x = rng.integers(0, 256, size=(nb, c, h, w), dtype=np.uint8)
    wq = rng.integers(-128, 128, size=(oc, c, k, k), dtype=np.int8)
    want = oracle.backend_conv2d_i32(x, zp, wq, stride, pad)
    got = host(ctx.conv2d_i32(dev(x), zp, dev(wq), stride, pad))
    np.testing.assert_array_equal(got, want)


def _quantized_conv_case(oracle, nb, c, h, w, oc, k, pad, seed):
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((nb, c, h, w)), 0).astype(np.float32)  # ReLU(N(0,1))
    wf = (rng.standard_normal((oc, c, k, k)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.01).astype(np.float32)
    mn, mx = oracle.find_min_max(x)
    s_in, zp_in = oracle.backend_params_asymmetric(mn, mx, 0, 255)
    xq = oracle.backend_quantize_f32(x, s_in, zp_in, 0, 255)
    wq, sw, _ = oracle.quantize_per_channel_auto(wf.reshape(oc, -1), 0, 0, oracle.PER_CHANNEL_SYMMETRIC)
    wq = wq.astype(np.int8).reshape(wf.shape)
    acc = oracle.backend_conv2d_i32(xq, zp_in, wq, (1, 1), (pad, pad))
    ho, wo = acc.shape[2:]
    acc2d = acc.reshape(nb * oc, ho * wo)
    out_f = (acc2d.astype(np.float32) * np.tile(np.float32(s_in) * sw, nb)[:, None]) + np.tile(bias, nb)[:, None]
    s_out, _ = oracle.calculate_symmetric_params(float(out_f.min()), float(out_f.max()), 0)
    return x, wf, bias, s_in, zp_in, xq, wq, sw, acc2d, s_out, out_f


@pytest.mark.parametrize("nb,c,h,w,oc,k,pad", [(2, 128, 14, 14, 64, 3, 1), (1, 256, 7, 7, 33, 3, 1), (3, 16, 10, 10, 8, 3, 1),
                                               (2, 96, 9, 11, 48, 3, 1)])
def test_quantized_conv2d_forward(ctx, hipq, oracle, nb, c, h, w, oc, k, pad):
    """The Conv2d configuration ([32,256,14,14], 3x3) at reduced size: asymmetric u8 activations, per-channel int8 filters, fused bias + requant."""
    x, wf, bias, s_in, zp_in, xq, wq, sw, acc2d, s_out, out_f = _quantized_conv_case(oracle, nb, c, h, w, oc, k, pad, c + oc)
    # activations quantized on the device: min/max -> asymmetric params -> u8
    dq, params = ctx.quantize_dynamic_per_tensor(dev(x), hipq.PARAMS_BACKEND_ASYMMETRIC, hipq.DTYPE_U8, hipq.FORM_DIV)
    p = ctx.read_qparams(params)
    assert (p.scale, p.zero_point) == (np.float32(s_in), zp_in)
    np.testing.assert_array_equal(host(dq), xq)
    # filters quantized per output channel on the device
    dwq, dsw, _, _ = ctx.quantize_per_row(dev(wf.reshape(oc, -1)))
    np.testing.assert_array_equal(host(dwq).reshape(wq.shape), wq)
    dwq = dwq.reshape(wq.shape)
    for mode, rm in ((hipq.ROUND_HALF_AWAY, 0), (hipq.ROUND_HALF_EVEN, 1)):
        oracle.set_round_mode(rm)
        try:
            want = oracle.requantize_epilogue(acc2d, s_in, sw, bias, s_out, -2, channel_axis_is_row=True, inner=oc)
        finally:
            oracle.set_round_mode(0)
        got = host(ctx.conv2d_i8(dq, zp_in, s_in, dwq, dsw, dev(bias), s_out, -2, (1, 1), (pad, pad), mode))
        np.testing.assert_array_equal(got.reshape(acc2d.shape), want)
        if c % 32 == 0:
            packed, sums = ctx.conv2d_pack_weights(dwq)
            got = host(ctx.conv2d_i8_packed(dq, zp_in, s_in, packed, sums, (k, k), dsw, dev(bias), s_out, -2, (pad, pad), mode))
            np.testing.assert_array_equal(got.reshape(acc2d.shape), want)
    # dequantize-with-bias epilogue: the same f32 expression in the same order -> identical bits
    got = host(ctx.conv2d_f32(dq, zp_in, s_in, dwq, dsw, dev(bias), (1, 1), (pad, pad)))
    np.testing.assert_array_equal(got.reshape(acc2d.shape), out_f)
    want = oracle.requantize_epilogue(acc2d, s_in, sw, None, s_out, 0, channel_axis_is_row=True, inner=oc)
    got = host(ctx.conv2d_i8(dq, zp_in, s_in, dwq, dsw, None, s_out, 0, (1, 1), (pad, pad)))
    np.testing.assert_array_equal(got.reshape(acc2d.shape), want)


def test_config4_full_size_against_direct_kernel_and_torch(ctx, hipq):
    """[32,256,14,14] (*) [256,256,3,3], stride 1, pad 1: the implicit-GEMM accumulators must equal an exact
    float64 convolution computed by torch (|acc| < 2^53), for a non-zero input zero point as well."""
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randint(0, 256, (32, 256, 14, 14), generator=g, device="cuda", dtype=torch.uint8)
    w = torch.randint(-128, 128, (256, 256, 3, 3), generator=g, device="cuda", dtype=torch.int8)
    for zp in (0, 37):
        acc = ctx.conv2d_i32(x, zp, w, (1, 1), (1, 1))
        ref = torch.nn.functional.conv2d(x.double() - zp, w.double(), padding=0)
        # zero padding of the real values: pad the shifted input with zeros
        ref = torch.nn.functional.conv2d(torch.nn.functional.pad(x.double() - zp, (1, 1, 1, 1)), w.double())
        torch.cuda.synchronize()
        assert torch.equal(acc, ref.to(torch.int32))


def test_config4_full_size_packed_requant_forward(ctx, hipq):
    """The Conv2d benchmark configuration at full size through the entry point the bench times (layout pass, packed filters,
    implicit GEMM, fused bias + requantize): every int8 output against the bytes re-derived, with torch's
    individually rounded f32 operations, from exact accumulators (float64 convolution, |acc| < 2^53); both
    roundings, a zero and a non-zero input zero point."""
    g = torch.Generator(device="cuda").manual_seed(9)
    nb, c, h, w_, oc = 32, 256, 14, 14, 256
    x = torch.randint(0, 256, (nb, c, h, w_), generator=g, device="cuda", dtype=torch.uint8)
    wq = torch.randint(-128, 128, (oc, c, 3, 3), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(oc, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(oc, generator=g, device="cuda") * 0.01
    packed, sums = ctx.conv2d_pack_weights(wq)
    s_in, s_out = 0.02, 0.37
    for zp_in, zp_out in ((0, 0), (37, -5)):
        acc = torch.nn.functional.conv2d(torch.nn.functional.pad(x.double() - zp_in, (1, 1, 1, 1)), wq.double())
        assert torch.equal(ctx.conv2d_i32(x, zp_in, wq, (1, 1), (1, 1)), acc.to(torch.int32))
        # acc as f32 * (s_in * s_w[oc]) + bias[oc], then round(v / s_out) + zp_out clamped: operations.rs:722-728
        s_comb = (torch.tensor(s_in, device="cuda", dtype=torch.float32) * sw)[None, :, None, None]
        v = acc.float() * s_comb + bias[None, :, None, None]
        t = v / torch.tensor(s_out, device="cuda", dtype=torch.float32)
        for mode, rounded in ((hipq.ROUND_HALF_AWAY, torch.trunc(t + torch.copysign(torch.full_like(t, 0.5), t))),
                              (hipq.ROUND_HALF_EVEN, torch.round(t))):
            if mode == hipq.ROUND_HALF_AWAY:  # trunc(t + 0.5) is f32::round except just below 0.5
                assert not bool(((t.abs() > 0.4999999) & (t.abs() < 0.5)).any())
            want = torch.clamp(rounded + zp_out, -128, 127).to(torch.int8)
            got = ctx.conv2d_i8_packed(x, zp_in, s_in, packed, sums, (3, 3), sw, bias, s_out, zp_out, (1, 1), mode)
            torch.cuda.synchronize()
            assert torch.equal(got, want)
            assert torch.equal(ctx.conv2d_i8(x, zp_in, s_in, wq, sw, bias, s_out, zp_out, (1, 1), (1, 1), mode), want)


PATCH_GEOMS = [
    # nb, c, h, w, oc, k, pad, zp: 128 or 256 channels, planes of a multiple of 4 bytes, raw rows within 128 bytes
    (3, 128, 14, 14, 40, 3, 1, 77),    # three images: patches that run from one image into the next
    (2, 256, 14, 14, 256, 3, 1, 0),
    (1, 256, 14, 14, 130, 3, 0, 128),  # no padding; a last filter block of two
    (5, 128, 8, 8, 64, 3, 1, 255),     # small planes: most patches span two images
    (2, 256, 10, 10, 33, 1, 0, 9),     # 1 x 1
    (2, 128, 12, 12, 70, 5, 2, 60),    # 25 taps
    (1, 128, 16, 12, 32, 2, 1, 3),     # even kernel, taps x channel blocks not a multiple of the loop's trip
]


@pytest.mark.parametrize("nb,c,h,w,oc,k,pad,zp", PATCH_GEOMS)
def test_conv_one_launch_patch_form(ctx, hipq, oracle, nb, c, h, w, oc, k, pad, zp):
    """The measured alternative behind test hook 14 (the workgroups gather their own patches of the image; no
    layout pass): int32 accumulators against the oracle, and the int8 / fp32 forwards bit for bit against the
    default two-launch form."""
    rng = np.random.default_rng(nb + c + h * 5 + oc + k)
    x = rng.integers(0, 256, size=(nb, c, h, w), dtype=np.uint8)
    wq = rng.integers(-128, 128, size=(oc, c, k, k), dtype=np.int8)
    sw = rng.uniform(1e-4, 1e-3, oc).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.01).astype(np.float32)
    want = oracle.backend_conv2d_i32(x, zp, wq, (1, 1), (pad, pad))
    xd, wd, swd, bd = dev(x), dev(wq), dev(sw), dev(bias)
    packed, sums = ctx.conv2d_pack_weights(wd)
    outs = {}
    try:
        for variant in (0, 14):
            ctx.set_gemm_kernel_variant(variant)
            outs[variant] = (
                host(ctx.conv2d_i32(xd, zp, wd, (1, 1), (pad, pad))),
                host(ctx.conv2d_i8_packed(xd, zp, 0.02, packed, sums, (k, k), swd, bd, 0.3, -4, (pad, pad))),
                host(ctx.conv2d_i8_packed(xd, zp, 0.02, packed, sums, (k, k), swd, bd, 0.3, -4, (pad, pad),
                                          hipq.ROUND_HALF_EVEN)),
                host(ctx.conv2d_f32(xd, zp, 0.02, wd, swd, bd, (1, 1), (pad, pad))),
            )
    finally:
        ctx.set_gemm_kernel_variant(0)
    np.testing.assert_array_equal(outs[14][0], want)
    for a, b in zip(outs[14], outs[0]):
        np.testing.assert_array_equal(a.view(np.uint8) if a.dtype == np.int8 else a.view(np.int32),
                                      b.view(np.uint8) if b.dtype == np.int8 else b.view(np.int32))


def test_conv_error_cases(ctx, hipq):
    x = torch.zeros((1, 4, 5, 5), dtype=torch.uint8, device="cuda")
    w = torch.zeros((2, 3, 3, 3), dtype=torch.int8, device="cuda")
    with pytest.raises(hipq.HipqError) as e:
        ctx.conv2d_i32(x, 0, w)
    assert e.value.code == hipq.DIMENSION_MISMATCH
    w = torch.zeros((2, 4, 7, 7), dtype=torch.int8, device="cuda")
    with pytest.raises(hipq.HipqError) as e:
        ctx.conv2d_i32(x, 0, w)
    assert e.value.code == hipq.SHAPE_ERROR
    w = torch.zeros((2, 4, 3, 3), dtype=torch.int8, device="cuda")
    sw = torch.ones(2, device="cuda")
    with pytest.raises(hipq.HipqError):
        ctx.conv2d_i8(x, 0, -1.0, w, sw, None, 1.0, 0)
    with pytest.raises(hipq.HipqError):
        ctx.conv2d_i8(x, 300, 1.0, w, sw, None, 1.0, 0)


@pytest.mark.parametrize("nb,c,h,w,oc,k,pad", [
    (2, 32, 5, 5, 16, (3, 3), (1, 1)), (1, 64, 7, 9, 40, (3, 2), (1, 0)), (3, 96, 12, 10, 33, (1, 1), (0, 0)),
    (32, 256, 14, 14, 256, (3, 3), (1, 1)),   # configs[3] at full size, as specified: fp32 in, int8 out
    (64, 128, 30, 30, 32, (3, 3), (1, 1)),    # image pass too large to be resident at once: quantized in a pass of its own
])
def test_conv2d_forward_from_fp32_equals_quantize_then_conv(ctx, hipq, nb, c, h, w, oc, k, pad):
    """hipq_conv2d_dynamic_f32_i8_packed (dynamic per-tensor uint8 quantize of the fp32 input fused into the image
    pass, parameters kept on the device) must give the parameters and the output bytes of
    hipq_quantize_dynamic_per_tensor_f32 followed by hipq_conv2d_u8i8_i8_packed with those parameters passed by
    value - the composition the oracle tests above pin - for both quantize forms and roundings."""
    g = torch.Generator(device="cuda").manual_seed(nb * 131 + c + h)
    x = torch.relu(torch.randn(nb, c, h, w, generator=g, device="cuda")) * 1.7
    wq = torch.randint(-128, 128, (oc, c) + k, generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(oc, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(oc, generator=g, device="cuda") * 0.05
    packed, sums = ctx.conv2d_pack_weights(wq)
    for qmode in (0, hipq.FORM_DIV, hipq.ROUND_HALF_EVEN | hipq.FORM_DIV):
        q, params = ctx.quantize_dynamic_per_tensor(x, hipq.PARAMS_BACKEND_ASYMMETRIC, hipq.DTYPE_U8, qmode)
        p = ctx.read_qparams(params)
        want = ctx.conv2d_i8_packed(q, p.zero_point, p.scale, packed, sums, k, sw, bias, 0.05, 3, pad,
                                    mode=hipq.ROUND_HALF_EVEN)
        got, gparams = ctx.conv2d_dynamic_packed(x, packed, sums, k, sw, bias, 0.05, 3, pad, quant_mode=qmode,
                                                 mode=hipq.ROUND_HALF_EVEN)
        torch.cuda.synchronize()
        gp = ctx.read_qparams(gparams)
        assert (gp.scale, gp.zero_point, gp.min_val, gp.max_val, gp.status) == (p.scale, p.zero_point, p.min_val,
                                                                                p.max_val, p.status)
        assert torch.equal(got, want), qmode
        ctx.set_gemm_kernel_variant(11)  # the same without the filter lines touched while the quantizer's grid waits
        try:
            off, _ = ctx.conv2d_dynamic_packed(x, packed, sums, k, sw, bias, 0.05, 3, pad, quant_mode=qmode,
                                               mode=hipq.ROUND_HALF_EVEN)
            torch.cuda.synchronize()
        finally:
            ctx.set_gemm_kernel_variant(0)
        assert torch.equal(off, want), qmode


def test_conv2d_forward_from_fp32_reports_a_bad_range(ctx, hipq):
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn(2, 32, 6, 6, generator=g, device="cuda")
    x[1, 3, 2, 2] = float("inf")
    wq = torch.randint(-128, 128, (8, 32, 3, 3), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(8, generator=g, device="cuda") * 1e-3 + 1e-4
    packed, sums = ctx.conv2d_pack_weights(wq)
    out, params = ctx.conv2d_dynamic_packed(x, packed, sums, (3, 3), sw, None, 0.05, 0, (1, 1))
    torch.cuda.synchronize()
    p = ctx.read_qparams(params)
    assert p.status == hipq.INVALID_ARGUMENT and p.scale != p.scale
    with pytest.raises(hipq.HipqError):
        ctx.conv2d_dynamic_packed(x[:, :31].contiguous(), packed, sums, (3, 3), sw, None, 0.05, 0, (1, 1))
