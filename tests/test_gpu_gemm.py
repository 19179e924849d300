"""Parity of the int8 MFMA GEMM and the quantized Linear forward with the CPU oracle.

int32 accumulators and int8 outputs are bit-exact; fp32 outputs are held to 1e-5
relative (and are in practice bit-exact, since the epilogue is the same sequence of
individually rounded f32 operations).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def rand_i8(rng, shape):
    return rng.integers(-128, 128, size=shape, dtype=np.int8)


SHAPES = [
    (1, 1, 16), (1, 16, 64), (16, 16, 64), (17, 33, 128), (64, 64, 256), (128, 64, 128), (130, 70, 144),
    (127, 129, 4096), (512, 256, 1024), (5, 300, 48), (256, 512, 16), (33, 1000, 2048),
]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_i32_bit_exact(ctx, oracle, m, n, k):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    got = host(ctx.gemm_i8_i32(dev(a), dev(w)))
    np.testing.assert_array_equal(got, oracle.gemm_i8_nk(a, w))


@pytest.mark.parametrize("m,n,k", [(3, 5, 7), (16, 16, 20), (9, 40, 1001), (1, 1, 1)])
def test_gemm_generic_path_for_odd_k(ctx, oracle, m, n, k):
    rng = np.random.default_rng(k)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    np.testing.assert_array_equal(host(ctx.gemm_i8_i32(dev(a), dev(w))), oracle.gemm_i8_nk(a, w))


def test_gemm_matches_reference_kn_layout(ctx, oracle):
    """The reference's B operand is [K,N]; the kernel takes its transpose and must give the same integers."""
    rng = np.random.default_rng(77)
    a, b_kn = rand_i8(rng, (20, 64)), rand_i8(rng, (64, 24))
    acc, _ = oracle.backend_matmul_i32(a, b_kn)
    got = host(ctx.gemm_i8_i32(dev(a), dev(np.ascontiguousarray(b_kn.T))))
    np.testing.assert_array_equal(got, acc)


def test_gemm_extreme_values_and_identity(ctx):
    a = np.full((32, 4096), -128, np.int8)
    got = host(ctx.gemm_i8_i32(dev(a), dev(a)))
    np.testing.assert_array_equal(got, np.full((32, 32), 4096 * 16384, np.int32))
    eye = np.eye(64, dtype=np.int8)
    rng = np.random.default_rng(1)
    x = rand_i8(rng, (48, 64))
    np.testing.assert_array_equal(host(ctx.gemm_i8_i32(dev(x), dev(eye))), x.astype(np.int32))


def test_gemm_linearity_full_size(ctx):
    """M=512, K=N=4096: (a1 + a2) W^T == a1 W^T + a2 W^T, checked against torch's int64 matmul on a slice."""
    g = torch.Generator(device="cuda").manual_seed(2)
    a1 = torch.randint(-60, 60, (512, 4096), generator=g, device="cuda", dtype=torch.int8)
    a2 = torch.randint(-60, 60, (512, 4096), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (4096, 4096), generator=g, device="cuda", dtype=torch.int8)
    c1, c2, c12 = ctx.gemm_i8_i32(a1, w), ctx.gemm_i8_i32(a2, w), ctx.gemm_i8_i32(a1 + a2, w)
    torch.cuda.synchronize()
    assert torch.equal(c12, c1 + c2)
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 511], device="cuda")
    ref = (a1[rows].double() @ w.double().T).to(torch.int32)  # exact: |acc| < 2^53
    assert torch.equal(c1[rows], ref)


def _quantized_linear_case(oracle, m, n, k, per_token, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float32)
    wf = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    wq, sw, _ = oracle.quantize_per_channel_auto(wf, 0, 0, oracle.PER_CHANNEL_SYMMETRIC)
    if per_token:
        aq, sa, _ = oracle.quantize_per_channel_auto(x, 0, 0, oracle.PER_CHANNEL_SYMMETRIC)
    else:
        aq, s, _ = oracle.quantize_tensor_auto(x, 0, oracle.PER_TENSOR_SYMMETRIC)
        sa = np.array([s], np.float32)
    acc = oracle.gemm_i8_nk(aq.astype(np.int8), wq.astype(np.int8))
    out = oracle.linear_dequant_epilogue(acc, sa, sw, bias)
    return x, wf, bias, wq.astype(np.int8), sw, aq.astype(np.int8), sa, acc, out


@pytest.mark.parametrize("m,n,k", [(4, 8, 16), (64, 128, 256), (100, 200, 304), (512, 512, 512), (33, 65, 1040)])
@pytest.mark.parametrize("per_token", [False, True])
def test_quantized_linear_forward(ctx, hipq, oracle, m, n, k, per_token):
    x, wf, bias, wq, sw, aq, sa, acc, want = _quantized_linear_case(oracle, m, n, k, per_token, m + n + k)
    # weights quantized on the device (offline step), bit-exact with the oracle
    dwq, dsw, _, _ = ctx.quantize_per_row(dev(wf))
    np.testing.assert_array_equal(host(dwq), wq)
    np.testing.assert_array_equal(host(dsw), sw)
    # separate steps
    got = host(ctx.linear_i8_f32(dev(aq), dev(sa), dwq, dsw, dev(bias)))
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=0)
    np.testing.assert_array_equal(got, want)
    # whole forward from fp32 activations
    got = host(ctx.linear_dynamic(dev(x), dwq, dsw, dev(bias), per_token=per_token,
                                  mode=hipq.FORM_MUL_INV if x.size > 64 else hipq.FORM_DIV))
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=0)
    np.testing.assert_array_equal(got, want)
    # no bias
    got = host(ctx.linear_i8_f32(dev(aq), dev(sa), dwq, dsw, None))
    np.testing.assert_array_equal(got, oracle.linear_dequant_epilogue(acc, sa, sw, None))


# K % 128 == 0 reaches the pipelined kernel, whose int8 epilogue stores dwords when N % 4 == 0 (ragged M and N tiles
# included) and bytes otherwise; the other shapes reach the register-staged and the generic kernels.
@pytest.mark.parametrize("m,n,k", [(7, 24, 64), (128, 96, 512), (50, 130, 272), (50, 100, 256), (130, 132, 384),
                                   (67, 130, 256), (300, 260, 128), (512, 1024, 1024)])
def test_quantized_linear_requant_epilogue(ctx, hipq, oracle, m, n, k):
    x, wf, bias, wq, sw, aq, sa, acc, out = _quantized_linear_case(oracle, m, n, k, False, 5 * m + k)
    s_out, _ = oracle.calculate_symmetric_params(*oracle.find_min_max(out), 0)
    for mode, rm in ((hipq.ROUND_HALF_AWAY, 0), (hipq.ROUND_HALF_EVEN, 1)):
        oracle.set_round_mode(rm)
        try:
            want = oracle.requantize_epilogue(acc, sa, sw, bias, s_out, 2)
        finally:
            oracle.set_round_mode(0)
        got = host(ctx.linear_i8_i8(dev(aq), dev(sa), dev(wq), dev(sw), dev(bias), s_out, 2, mode))
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("m,n,k", [(4096, 1024, 512), (4100, 1000, 256), (8192, 768, 768), (2048, 2304, 256),
                                   (2000, 2300, 384)])
def test_many_tile_shapes_persistent_kernel(ctx, hipq, oracle, m, n, k):
    """Shapes with at least two 128x64 tiles per compute unit run on the persistent kernel: accumulators, the
    dequantize epilogue with per-token scales, the residual add and the requantize epilogue against the oracle.
    The shapes cover its tile forms (N = 768 and 2304 take 128x192 tiles, the ragged ones the bounds-checked
    epilogues)."""
    rng = np.random.default_rng(m + n + k)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    acc = oracle.gemm_i8_nk(a, w)
    np.testing.assert_array_equal(host(ctx.gemm_i8_i32(dev(a), dev(w))), acc)
    sa = (rng.random(m) * 0.05 + 0.001).astype(np.float32)
    sw = (rng.random(n) * 0.002 + 0.0001).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    want = oracle.linear_dequant_epilogue(acc, sa, sw, bias)
    np.testing.assert_array_equal(host(ctx.linear_i8_f32(dev(a), dev(sa), dev(w), dev(sw), dev(bias))), want)
    s1 = np.array([0.021], np.float32)
    want1 = oracle.linear_dequant_epilogue(acc, s1, sw, None)
    np.testing.assert_array_equal(host(ctx.linear_i8_f32(dev(a), dev(s1), dev(w), dev(sw), None)), want1)
    res = rng.standard_normal((m, n)).astype(np.float32)
    got = host(ctx.linear_i8_f32_residual(dev(a), dev(sa), dev(w), dev(sw), dev(bias), dev(res)))
    np.testing.assert_array_equal(got, want + res)
    s_out, _ = oracle.calculate_symmetric_params(*oracle.find_min_max(want), 0)
    for mode, rm in ((hipq.ROUND_HALF_AWAY, 0), (hipq.ROUND_HALF_EVEN, 1)):
        oracle.set_round_mode(rm)
        try:
            wantq = oracle.requantize_epilogue(acc, sa, sw, bias, s_out, -5)
        finally:
            oracle.set_round_mode(0)
        np.testing.assert_array_equal(host(ctx.linear_i8_i8(dev(a), dev(sa), dev(w), dev(sw), dev(bias), s_out, -5, mode)), wantq)


@pytest.mark.parametrize("m", [1, 4, 16])
def test_decode_shapes_small_n(ctx, hipq, oracle, m):
    """Config-3 shaped (per-token activations, K=4096) at an N the oracle finishes quickly."""
    x, wf, bias, wq, sw, aq, sa, acc, want = _quantized_linear_case(oracle, m, 344, 4096, True, 40 + m)
    got = host(ctx.linear_dynamic(dev(x), dev(wq), dev(sw), dev(bias), per_token=True))
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(host(ctx.gemm_i8_i32(dev(aq), dev(wq))), acc)


def test_gemm_error_cases(ctx, hipq):
    a = torch.zeros((4, 16), dtype=torch.int8, device="cuda")
    w = torch.zeros((4, 32), dtype=torch.int8, device="cuda")
    with pytest.raises(hipq.HipqError) as e:
        ctx.gemm_i8_i32(a, w)
    assert e.value.code == hipq.DIMENSION_MISMATCH
    with pytest.raises(hipq.HipqError):
        ctx.call("hipq_gemm_i8_i32", a.data_ptr(), None, 4, 4, 16, a.data_ptr())
    # empty M or N is a no-op
    ctx.call("hipq_gemm_i8_i32", a.data_ptr(), w.data_ptr(), 0, 4, 16, None)


@pytest.mark.parametrize("m", [1, 4, 16, 17, 40, 64])
def test_config3_full_size_weight_streaming(ctx, hipq, m):
    """Llama-7B up-proj shape N=11008, K=4096: int32 accumulators against an exact
    float64 product computed by torch, and the fused per-token epilogue against the same f32 expression."""
    g = torch.Generator(device="cuda").manual_seed(5 + m)
    n, k = 11008, 4096
    a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    acc = ctx.gemm_i8_i32(a, w)
    ref = (a.double() @ w.double().T).to(torch.int32)  # exact: |acc| < 2^53
    torch.cuda.synchronize()
    assert torch.equal(acc, ref)
    sa = torch.rand(m, generator=g, device="cuda") * 0.05 + 0.01
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(n, generator=g, device="cuda") * 0.01
    out = ctx.linear_i8_f32(a, sa, w, sw, bias)
    want = ref.float() * (sa[:, None] * sw[None, :]) + bias[None, :]  # same individually rounded f32 ops
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    # The kernels the benchmark times at this shape run on prepared (fragment-packed) operands: the one-row-block
    # kernel and both forms of the weight-streaming kernel, at 344 weight row blocks x 128 k blocks, against the
    # same exact product and the same f32 expression.
    pa, pw = ctx.pack_rows(a), ctx.pack_rows(w)
    assert torch.equal(ctx.gemm_packed_i8_i32(pa, pw, m, n, k), ref)
    assert torch.equal(ctx.linear_packed_i8_f32(pa, sa, pw, sw, bias, m, n, k), want)
    assert torch.equal(ctx.linear_packed_i8_f32(pa, sa[:1], pw, sw, None, m, n, k),
                       ref.float() * (sa[0] * sw[None, :]))  # one scale for the tensor, no bias


@pytest.mark.parametrize("m", [1, 2, 4, 16])
def test_config3_full_size_forward_from_fp32_against_the_oracle(ctx, hipq, oracle, m):
    """configs[2] as specified, at its own size (N=11008, K=4096): fp32 activations, per-token dynamic int8, prepared
    per-channel weights, fp32 out.  One or two rows take the one-launch kernel in which every workgroup quantizes
    the rows itself, more rows the per-row quantizer and the product; both against the oracle's per-channel
    quantize (axis 0) + int32 GEMM + dequantize epilogue, bit for bit."""
    rng = np.random.default_rng(500 + m)
    n, k = 11008, 4096
    x = rng.standard_normal((m, k)).astype(np.float32)
    wq = rand_i8(rng, (n, k))
    sw = (rng.random(n) * 0.002 + 0.0001).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    aq, sa, _ = oracle.quantize_per_channel_auto(x, 0, oracle.DTYPE_I8, oracle.PER_CHANNEL_SYMMETRIC)
    acc = oracle.gemm_i8_nk(aq.astype(np.int8), wq)
    want = oracle.linear_dequant_epilogue(acc, sa, sw, bias)
    pw = ctx.pack_rows(dev(wq))
    got = host(ctx.linear_dynamic_packed(dev(x), pw, dev(sw), dev(bias), per_token=True))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)
    np.testing.assert_array_equal(got, want)
    want_nb = oracle.linear_dequant_epilogue(acc, sa, sw, None)
    np.testing.assert_array_equal(host(ctx.linear_dynamic_packed(dev(x), pw, dev(sw), None, per_token=True)), want_nb)


@pytest.mark.parametrize("n,k", [(2304, 768), (768, 768), (3072, 768), (768, 3072)])
def test_config5_full_size_projection_shapes(ctx, hipq, n, k):
    """The projection stack's GEMMs at their real size (8192 tokens, d = 768, d_ff = 3072), which run on the
    persistent kernel's large tile forms: every accumulator against an exact float64 product computed by torch in
    row chunks, the per-token dequantize epilogue and the residual form against the same f32 expression, and the
    requantize epilogue's bytes re-derived from the f32 output with numpy's IEEE division."""
    m = 8192
    g = torch.Generator(device="cuda").manual_seed(n + k)
    a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    acc = ctx.gemm_i8_i32(a, w)
    ref = torch.empty((m, n), dtype=torch.int32, device="cuda")
    wd = w.double().T.contiguous()
    for r0 in range(0, m, 1024):
        ref[r0:r0 + 1024] = (a[r0:r0 + 1024].double() @ wd).to(torch.int32)  # exact: |acc| < 2^53
    torch.cuda.synchronize()
    assert torch.equal(acc, ref)
    sa = torch.rand(m, generator=g, device="cuda") * 0.05 + 0.01
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(n, generator=g, device="cuda") * 0.01
    want = ref.float() * (sa[:, None] * sw[None, :]) + bias[None, :]  # same individually rounded f32 ops
    assert torch.equal(ctx.linear_i8_f32(a, sa, w, sw, bias), want)
    res = torch.randn((m, n), generator=g, device="cuda")
    assert torch.equal(ctx.linear_i8_f32_residual(a, sa, w, sw, bias, res), want + res)
    x = res.clone()  # in place, as the stack uses it
    ctx.linear_i8_f32_residual(a, sa, w, sw, bias, x, out=x)
    assert torch.equal(x, want + res)
    s_out = np.float32(float(want.abs().max()) / 127.0)
    q = ctx.linear_i8_i8(a, sa, w, sw, bias, float(s_out), 3)
    torch.cuda.synchronize()
    t = want.cpu().numpy() / s_out  # IEEE f32 division
    r = np.trunc(t + np.copysign(np.float32(0.49999997), t))  # f32::round (tests/host/round_away_check.c)
    assert r.dtype == np.float32
    wantq = np.clip(r + np.float32(3), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(q.cpu().numpy(), wantq)


@pytest.mark.parametrize("m,n,k", [(48, 80, 256), (512, 512, 512), (2048, 768, 256), (5, 24, 48)])
def test_linear_with_static_activation_scale(ctx, hipq, oracle, m, n, k):
    """Static quantization: the activation scale comes from calibration (an observer), not from the input.  The
    fused call equals the oracle's per-tensor quantize (both forms) -> int32 GEMM -> dequantize epilogue, and the
    publishing quantize records the parameters it was given."""
    rng = np.random.default_rng(m * 3 + n)
    x = rng.standard_normal((m, k)).astype(np.float32)
    wq = rand_i8(rng, (n, k))
    sw = (rng.random(n) * 0.002 + 0.0001).astype(np.float32)
    bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
    s_a = np.float32(4.0 / 127.0)  # clips the tail of N(0,1): saturation is part of the case
    for mode, quantize in ((hipq.FORM_MUL_INV, oracle.quantize_to_int8_simd), (hipq.FORM_DIV, oracle.quantize_per_tensor_affine_i8)):
        aq = quantize(x.ravel(), s_a, 0).reshape(m, k).astype(np.int8)
        want = oracle.linear_dequant_epilogue(oracle.gemm_i8_nk(aq, wq), np.array([s_a], np.float32), sw, bias)
        got = host(ctx.linear_static(dev(x), float(s_a), dev(wq), dev(sw), dev(bias), mode=mode))
        np.testing.assert_array_equal(got, want)
        q, params = ctx.quantize_static_per_tensor(dev(x), float(s_a), 0, mode)
        np.testing.assert_array_equal(host(q), aq)
        rec = ctx.read_qparams(params)
        assert rec.scale == s_a and rec.zero_point == 0 and rec.status == hipq.SUCCESS
    with pytest.raises(hipq.HipqError) as e:
        ctx.linear_static(dev(x), 0.0, dev(wq), dev(sw), dev(bias))
    assert e.value.code == hipq.INVALID_ARGUMENT and "Scale must be positive" in str(e.value)


@pytest.mark.parametrize("variant", [1, 2, 3, 5, 6, 7, 8, 10])
def test_every_gemm_kernel_form_gives_the_same_bits(ctx, hipq, oracle, variant):
    """The kernel form is a performance choice only: each form, forced on shapes it would not be picked for, gives
    the oracle's accumulators and epilogue outputs bit for bit (interior and ragged tiles, all four epilogues)."""
    try:
        ctx.set_gemm_kernel_variant(variant)
        for (m, n, k) in ((300, 200, 256), (1024, 768, 512), (130, 2304, 256)):
            rng = np.random.default_rng(variant * 1000 + m)
            a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
            acc = oracle.gemm_i8_nk(a, w)
            np.testing.assert_array_equal(host(ctx.gemm_i8_i32(dev(a), dev(w))), acc)
            sa = (rng.random(m) * 0.05 + 0.001).astype(np.float32)
            sw = (rng.random(n) * 0.002 + 0.0001).astype(np.float32)
            bias = (rng.standard_normal(n) * 0.01).astype(np.float32)
            want = oracle.linear_dequant_epilogue(acc, sa, sw, bias)
            np.testing.assert_array_equal(host(ctx.linear_i8_f32(dev(a), dev(sa), dev(w), dev(sw), dev(bias))), want)
            res = rng.standard_normal((m, n)).astype(np.float32)
            got = host(ctx.linear_i8_f32_residual(dev(a), dev(sa), dev(w), dev(sw), dev(bias), dev(res)))
            np.testing.assert_array_equal(got, want + res)
            s_out, _ = oracle.calculate_symmetric_params(*oracle.find_min_max(want), 0)
            wantq = oracle.requantize_epilogue(acc, sa, sw, bias, s_out, -5)
            np.testing.assert_array_equal(host(ctx.linear_i8_i8(dev(a), dev(sa), dev(w), dev(sw), dev(bias), s_out, -5)), wantq)
    finally:
        ctx.set_gemm_kernel_variant(0)
    with pytest.raises(hipq.HipqError):
        ctx.set_gemm_kernel_variant(99)


def test_a_wait_that_gives_up_is_reported_not_swallowed(hipq, oracle):
    """The persistent kernel bounds every wait so that its grid always drains.  With the spin limit forced to 0
    the consumer waves do not wait for the first K-tile (a wait that is certain to be needed: the fills need a
    memory round trip), run on and finish normally with a wrong product; the context must then report
    HIPQ_DEVICE_ERROR at the next synchronize, once, and work normally again afterwards."""
    c = hipq.Context(0)
    try:
        rng = np.random.default_rng(5)
        a, w = rand_i8(rng, (1024, 512)), rand_i8(rng, (768, 512))
        da, dw = dev(a), dev(w)
        c.set_gemm_kernel_variant(7)  # a persistent form
        c.set_wait_spin_limit(0)
        c.gemm_i8_i32(da, dw)
        with pytest.raises(hipq.HipqError) as e:
            c.synchronize()
        assert e.value.code == hipq.DEVICE_ERROR and "gave up" in str(e.value)
        c.synchronize()  # reported once, then cleared
        c.set_wait_spin_limit(-1)
        got = c.gemm_i8_i32(da, dw)
        c.synchronize()
        np.testing.assert_array_equal(got.cpu().numpy(), oracle.gemm_i8_nk(a, w))
    finally:
        c.close()


def test_output_larger_than_four_gib(ctx, hipq, oracle):
    """[32768, 128] x [32768, 128]^T: the fp32 / int32 output is 4 GiB, so byte offsets into it pass 2^32.  Both
    operands are a 512-row block repeated 64 times; every 512 x 512 block of the output must equal the oracle's
    product of the two blocks (and its dequantize epilogue with the per-row and per-channel scales repeated)."""
    blk, reps, k = 512, 64, 128
    rng = np.random.default_rng(77)
    a0, w0 = rand_i8(rng, (blk, k)), rand_i8(rng, (blk, k))
    sa0 = (rng.random(blk) * 0.05 + 0.01).astype(np.float32)
    sw0 = (rng.random(blk) * 0.002 + 0.0001).astype(np.float32)
    b0 = (rng.standard_normal(blk) * 0.01).astype(np.float32)
    acc0 = oracle.gemm_i8_nk(a0, w0)
    out0 = oracle.linear_dequant_epilogue(acc0, sa0, sw0, b0)
    a, w = dev(a0).repeat(reps, 1), dev(w0).repeat(reps, 1)
    acc = ctx.gemm_i8_i32(a, w)
    torch.cuda.synchronize()
    assert acc.numel() * 4 == 1 << 32
    assert bool((acc.view(reps, blk, reps, blk) == dev(acc0)[None, :, None, :]).all())
    del acc
    out = ctx.linear_i8_f32(a, dev(sa0).repeat(reps), w, dev(sw0).repeat(reps), dev(b0).repeat(reps))
    torch.cuda.synchronize()
    assert bool((out.view(reps, blk, reps, blk) == dev(out0)[None, :, None, :]).all())
