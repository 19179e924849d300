"""Parity of the row-panel Linear forwards (a workgroup owns 32 whole rows of the output - or two workgroups of one
XCD share 64 rows, half of the columns each - and applies the row operation that follows the Linear - per-token
quantizer, GELU, skip connection, LayerNorm - to its accumulators) and of the projection stack built from them.

What is bit-exact and what is not:
  * the fp32 product, the skip connection and GELU + per-token int8 perform, per element, the f32 operations of
    the separate entry points in their order: outputs are compared bit for bit with those entry points, which
    the other test files hold against the CPU oracle;
  * a LayerNorm folds its row sums in another order than the row kernel (any two orders differ in the last bits
    of mean and variance), so its per-token scales are held to 1e-6 relative and its codes to one step, on at most
    1e-5 of the elements; the oracle's LayerNorm of the device's own x gives a second, independent bound.
"""
import numpy as np
import pytest
import torch

from test_gpu_packed import dev, host, pack_reference, rand_i8

pytestmark = pytest.mark.gpu


def unpack_reference(p: np.ndarray, rows: int, k: int) -> np.ndarray:
    """Inverse of pack_reference: packed bytes -> int8 [rows, k]."""
    rb, kb = (rows + 31) // 32, ((k + 31) // 32 + 3) // 4 * 4
    t = p.reshape(rb, kb, 2, 32, 16).transpose(0, 3, 1, 2, 4).reshape(rb * 32, kb * 32)
    return np.ascontiguousarray(t[:rows, :k])


def operands(rng, m, n, k, per_row=True, bias=True):
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    sa = (rng.uniform(0.001, 0.02, m if per_row else 1)).astype(np.float32)
    sw = rng.uniform(1e-4, 2e-3, n).astype(np.float32)
    b = rng.standard_normal(n).astype(np.float32) if bias else None
    return a, w, sa, sw, b


def bits(t):
    return host(t).view(np.int32)


# m ragged and whole; n: every instantiation (<= 768, <= 1536, <= 2304, <= 3072) and widths that leave waves
# without columns; k ragged, one stage of the activation panel (768), several (1600, 3072)
F32_SHAPES = [(1, 32, 16), (100, 256, 96), (33, 96, 70), (64, 160, 768), (257, 768, 800), (40, 1536, 1600),
              (130, 2304, 768), (96, 3072, 768), (65, 800, 3072), (32, 2080, 64)]


@pytest.mark.parametrize("m,n,k", F32_SHAPES)
@pytest.mark.parametrize("per_row,bias", [(True, True), (False, False)])
def test_linear_rows_f32_equals_the_tiled_form(ctx, oracle, m, n, k, per_row, bias):
    rng = np.random.default_rng(m * 31 + n * 7 + k)
    a, w, sa, sw, b = operands(rng, m, n, k, per_row, bias)
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    bd = dev(b) if bias else None
    got = ctx.linear_rows_packed_i8_f32(pa, dev(sa), pw, dev(sw), bd, m, n, k)
    want = ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), bd, m, n, k)
    np.testing.assert_array_equal(bits(got), bits(want))
    if m * n * k <= 1 << 24:  # and the oracle itself where it is quick
        acc = oracle.gemm_i8_nk(a, w)
        ref = oracle.linear_dequant_epilogue(acc, np.broadcast_to(sa, (m,)).copy(), sw, b)
        np.testing.assert_array_equal(host(got), ref)


Q_SHAPES = [(1, 128, 32), (100, 256, 96), (33, 128, 70), (257, 768, 800), (40, 1536, 1600), (130, 2304, 768),
            (96, 3072, 768), (65, 768, 3072), (70, 1024, 200)]


@pytest.mark.parametrize("m,n,k", Q_SHAPES)
@pytest.mark.parametrize("mode", [0, 1])
def test_linear_gelu_quantize_equals_its_parts(ctx, hipq, m, n, k, mode):
    rng = np.random.default_rng(m * 13 + n * 5 + k + mode)
    a, w, sa, sw, b = operands(rng, m, n, k)
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    rmode = hipq.ROUND_HALF_EVEN if mode else 0
    f = ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    q, s = ctx.gelu_tanh_quantize(f, mode=rmode)
    got_q, got_s = ctx.linear_gelu_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), m, n, k, mode=rmode)
    np.testing.assert_array_equal(bits(got_s), bits(s))
    np.testing.assert_array_equal(host(got_q), pack_reference(host(q)))  # (padding rows and k blocks: zeros)


@pytest.mark.parametrize("m,n,k", [(40, 256, 64), (72, 1536, 64)])
def test_linear_gelu_quantize_rows_that_are_not_finite(ctx, m, n, k):
    """A row whose GELU output holds an infinity gets a NaN scale and zero codes, a NaN element is code 0 and does
    not enter the row's maximum: as the row kernel has it (in a panel of one workgroup and in one of a pair)."""
    rng = np.random.default_rng(5)
    a, w, sa, sw, b = operands(rng, m, n, k)
    b[3] = np.inf
    sa[7] = np.nan  # a whole row of NaN
    sw[9] = np.nan  # one NaN per row
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    f = ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    q, s = ctx.gelu_tanh_quantize(f)
    got_q, got_s = ctx.linear_gelu_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    assert np.isnan(host(got_s)).sum() >= m - 1  # (column 3 is +inf in every row; row 7 is NaN throughout)
    np.testing.assert_array_equal(np.isnan(host(got_s)), np.isnan(host(s)))
    np.testing.assert_array_equal(host(got_q), pack_reference(host(q)))
    b[3] = 0.5
    f = ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    q, s = ctx.gelu_tanh_quantize(f)
    got_q, got_s = ctx.linear_gelu_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    np.testing.assert_array_equal(bits(got_s), bits(s))
    np.testing.assert_array_equal(host(got_q), pack_reference(host(q)))


LN_SHAPES = [(1, 128, 32), (100, 256, 96), (257, 768, 800), (65, 768, 3072), (40, 1536, 160), (48, 3072, 64),
             (97, 3072, 768), (70, 1536, 1600)]  # (the last two: panels of 64 rows shared by two compute units)


@pytest.mark.parametrize("m,n,k", LN_SHAPES)
@pytest.mark.parametrize("affine", [True, False])
def test_linear_residual_layer_norm_quantize(ctx, oracle, m, n, k, affine):
    rng = np.random.default_rng(m * 3 + n + k)
    a, w, sa, sw, b = operands(rng, m, n, k)
    x0 = rng.standard_normal((m, n)).astype(np.float32)
    gamma = rng.uniform(0.5, 1.5, n).astype(np.float32) if affine else None
    beta = (rng.standard_normal(n) * 0.1).astype(np.float32) if affine else None
    gd, bd = (dev(gamma), dev(beta)) if affine else (None, None)
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    # the separate entry points
    f = ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    x_parts = dev(x0)
    q, s = ctx.add_layer_norm_quantize(x_parts, f, gd, bd)
    # one kernel
    x_one = dev(x0)
    got_q, got_s = ctx.linear_residual_layer_norm_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), m, n, k, x_one, gd, bd)
    np.testing.assert_array_equal(bits(x_one), bits(x_parts))  # the stream: bit for bit
    np.testing.assert_allclose(host(got_s), host(s), rtol=1e-6, atol=0)
    codes = unpack_reference(host(got_q), m, n).astype(np.int16)
    diff = np.abs(codes - host(q).astype(np.int16))
    assert diff.max() <= 1
    assert (diff != 0).mean() <= 1e-5 + 2.0 / diff.size
    # against the oracle's LayerNorm of the device's own stream (f32 sums in yet another order): every code
    # within one step of the oracle's quantization of its own LayerNorm output
    h = oracle.layer_norm(host(x_one), gamma, beta, 1e-5)
    oq, osc, _ = oracle.quantize_per_channel_auto(h, 0, 0, oracle.PER_CHANNEL_SYMMETRIC)
    np.testing.assert_allclose(host(got_s), osc, rtol=2e-6, atol=0)
    assert np.abs(codes - oq.astype(np.int16)).max() <= 1
    # padding of the packed output is zero
    full = host(got_q)
    np.testing.assert_array_equal(full, pack_reference(codes.astype(np.int8)))
    # without the LayerNorm: only the skip connection
    x_res = dev(x0)
    ctx.linear_residual_layer_norm_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), m, n, k, x_res, normalize=False)
    np.testing.assert_array_equal(bits(x_res), bits(x_parts))


@pytest.mark.parametrize("m,n,k", [(65, 768, 3072), (97, 3072, 768)])
def test_linear_residual_layer_norm_quantize_half_even(ctx, hipq, m, n, k):
    """The same comparison with codes rounded half to even (single panels and pairs)."""
    rng = np.random.default_rng(m + n + k)
    a, w, sa, sw, b = operands(rng, m, n, k)
    x0 = rng.standard_normal((m, n)).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, n).astype(np.float32), (rng.standard_normal(n) * 0.1).astype(np.float32)
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    f = ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), m, n, k)
    x_parts, x_one = dev(x0), dev(x0)
    q, s = ctx.add_layer_norm_quantize(x_parts, f, dev(gamma), dev(beta), mode=hipq.ROUND_HALF_EVEN)
    got_q, got_s = ctx.linear_residual_layer_norm_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), m, n, k, x_one,
                                                                  dev(gamma), dev(beta), mode=hipq.ROUND_HALF_EVEN)
    np.testing.assert_array_equal(bits(x_one), bits(x_parts))
    np.testing.assert_allclose(host(got_s), host(s), rtol=1e-6, atol=0)
    diff = np.abs(unpack_reference(host(got_q), m, n).astype(np.int16) - host(q).astype(np.int16))
    assert diff.max() <= 1 and (diff != 0).mean() <= 1e-5 + 2.0 / diff.size


def test_row_panel_shapes_that_are_refused(ctx, hipq):
    rng = np.random.default_rng(1)
    a, w, sa, sw, b = operands(rng, 8, 3104, 32)
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    with pytest.raises(hipq.HipqError) as e:  # wider than a workgroup's registers hold
        ctx.linear_rows_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), 8, 3104, 32)
    assert e.value.code == hipq.SHAPE_ERROR
    a, w, sa, sw, b = operands(rng, 8, 96, 32)
    pa, pw = ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w))
    with pytest.raises(hipq.HipqError) as e:  # a packed int8 output is the K of the next product: whole groups of 4 k blocks
        ctx.linear_gelu_quantize_packed(pa, dev(sa), pw, dev(sw), dev(b), 8, 96, 32)
    assert e.value.code == hipq.SHAPE_ERROR
    with pytest.raises(hipq.HipqError) as e:
        ctx.linear_rows_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), 8, 90, 32)
    assert e.value.code == hipq.SHAPE_ERROR
    # nothing to do
    ctx.linear_rows_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(b), 0, 96, 32, out=torch.empty((0, 96), device="cuda"))


def test_buffer_accesses_past_the_extent_are_checked_with_the_scalar_offset(ctx):
    """The row-panel kernels give their buffer descriptors exact extents and rely on the hardware for what lies past
    them (column blocks past N, k blocks past K, rows past M), with the distance in the SCALAR offset of the access:
    such loads must give zeros and such stores must be dropped, lane by lane.  The probe keeps every address it could
    reach inside one allocation, so it is safe on hardware that checked less."""
    mem = torch.empty(1 << 18, dtype=torch.int32, device="cuda")
    loaded = torch.empty(64, dtype=torch.int32, device="cuda")
    for soff, inside in ((0, 64), (3968, 32), (4096, 0), (8192, 0), (65536, 0), ((1 << 20) - 256, 0)):
        mem.fill_(0x11111111)
        ctx.call("hipq_probe_buffer_range_check", mem.data_ptr(), mem.numel() * 4, 4096, soff, loaded.data_ptr())
        ctx.synchronize()
        got = host(loaded)
        assert (got[:inside] == 0x11111111).all() and (got[inside:] == 0).all(), (soff, got)
        window = host(mem[soff // 4:soff // 4 + 64])
        assert (window[:inside] == 0x7777).all() and (window[inside:] == 0x11111111).all(), (soff, window)
    with pytest.raises(Exception):  # an access the allocation would not cover is refused by the host
        ctx.call("hipq_probe_buffer_range_check", mem.data_ptr(), mem.numel() * 4, 4096, 1 << 20, loaded.data_ptr())


# ---- the same forward from fp32 rows: the per-token quantizer inside the kernel -------------------------------

FROM_F32_SHAPES = [(8192, 768, 768, 2304), (100, 256, 96, 96), (33, 128, 1536, 1600), (257, 1536, 800, 2400),
                   (40, 1024, 64, 64), (1, 128, 4, 8)]  # m, n, k, row pitch of the activations


@pytest.mark.parametrize("m,n,k,lda", FROM_F32_SHAPES)
@pytest.mark.parametrize("mode", [0, 1])
def test_linear_from_f32_rows_equals_the_quantizer_then_the_linear(ctx, hipq, m, n, k, lda, mode):
    """hipq_linear_from_f32_residual_layer_norm_quantize_packed_i8 (every workgroup quantizes its own 32 fp32 rows per
    token and keeps the codes on chip) against hipq_quantize_per_row_packed_f32_i8 on a dense copy of the rows and
    the forward on packed activations: the stream, the codes and the scales bit for bit, with and without the
    LayerNorm.  Rows that are a slice of a wider matrix; a NaN element; a row holding an infinity (NaN scale, zero
    codes: its outputs are NaN in both)."""
    g = torch.Generator(device="cuda").manual_seed(m * 7 + n + k + mode)
    rmode = hipq.ROUND_HALF_EVEN if mode else 0
    a_full = torch.randn(m, lda, generator=g, device="cuda") * 1.7
    a = a_full[:, lda - k:]
    a[m // 2, k // 3] = float("nan")
    if m > 8:
        a[5, k - 1] = float("inf")
    w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(n, generator=g, device="cuda") * 2e-3 + 1e-4
    b = torch.randn(n, generator=g, device="cuda")
    gamma = torch.rand(n, generator=g, device="cuda") + 0.5
    beta = torch.randn(n, generator=g, device="cuda") * 0.1
    x0 = torch.randn(m, n, generator=g, device="cuda")
    pw = ctx.pack_rows(w)
    try:
        ctx.set_gemm_kernel_variant(15)  # (the packed-activation forward on single panels, like the kernel under test)
        qa, sa = ctx.quantize_per_row_packed(a.contiguous(), mode=rmode)
        x_parts, x_res_parts = x0.clone(), x0.clone()
        want_q, want_s = ctx.linear_residual_layer_norm_quantize_packed(qa, sa, pw, sw, b, m, n, k, x_parts, gamma, beta,
                                                                        mode=rmode)
        ctx.linear_residual_layer_norm_quantize_packed(qa, sa, pw, sw, b, m, n, k, x_res_parts, normalize=False)
    finally:
        ctx.set_gemm_kernel_variant(0)
    x_one, x_res = x0.clone(), x0.clone()
    got_q, got_s = ctx.linear_from_f32_residual_layer_norm_quantize_packed(a, pw, sw, b, n, x_one, gamma, beta,
                                                                           mode=rmode)
    ctx.linear_from_f32_residual_layer_norm_quantize_packed(a, pw, sw, b, n, x_res, mode=rmode, normalize=False)
    np.testing.assert_array_equal(bits(x_one), bits(x_parts))
    np.testing.assert_array_equal(bits(x_res), bits(x_res_parts))
    np.testing.assert_array_equal(bits(got_s), bits(want_s))
    np.testing.assert_array_equal(host(got_q), host(want_q))


def test_linear_from_f32_rows_shapes_that_are_refused(ctx, hipq):
    g = torch.Generator(device="cuda").manual_seed(4)
    def call(m, n, k, lda, off=0):
        a = torch.randn(m * lda + 8, generator=g, device="cuda")[off:off + m * lda].view(m, lda)[:, :k]
        w = ctx.pack_rows(torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8))
        sw = torch.rand(n, generator=g, device="cuda")
        x = torch.zeros(m, n, device="cuda")
        return ctx.linear_from_f32_residual_layer_norm_quantize_packed(a, w, sw, None, n, x)
    for args in ((8, 128, 1540, 1540), (8, 1664, 64, 64), (8, 128, 62, 64), (8, 128, 64, 66), (8, 128, 64, 64, 1),
                 (8, 96, 64, 64)):
        with pytest.raises(hipq.HipqError) as e:
            call(*args)
        assert e.value.code == hipq.SHAPE_ERROR, args
    call(8, 128, 64, 64)
    ctx.synchronize()


# ---- panels of 64 rows shared by a pair of compute units ------------------------------------------------------

PAIR_SHAPES = [(8192, 3072, 768), (97, 3072, 768), (70, 1536, 1600), (40, 2048, 1056), (200, 2304, 1024), (33, 1664, 96)]


# shapes whose quantizing forms keep single panels by default (narrow outputs: waves without columns), with the
# pair form forced (test hook 16)
FORCED_PAIR_SHAPES = [(100, 256, 96), (257, 768, 800), (65, 768, 3072), (130, 1280, 64), (8192, 768, 768)]


@pytest.mark.parametrize("m,n,k,pairs", [s + (0,) for s in PAIR_SHAPES] + [s + (16,) for s in FORCED_PAIR_SHAPES])
def test_pair_panels_equal_single_panels(hipq, m, n, k, pairs):
    """The row-panel kernels in their pair form (two workgroups of one XCD share 64 rows and take half of the columns
    each; row maxima and sums cross through the XCD's L2) against the single-workgroup panels (test hook 15): the fp32
    product, the skip connection, GELU + per-token int8 bit for bit, the LayerNorm form within the bound that holds
    between any two orders of its sums.  Twice in a row: the exchange flags must be back at zero."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(m + n + k)
        a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
        w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
        sa = torch.rand(m, generator=g, device="cuda") * 0.02 + 0.001
        sw = torch.rand(n, generator=g, device="cuda") * 2e-3 + 1e-4
        b = torch.randn(n, generator=g, device="cuda")
        gamma = torch.rand(n, generator=g, device="cuda") + 0.5
        beta = torch.randn(n, generator=g, device="cuda") * 0.1
        x0 = torch.randn(m, n, generator=g, device="cuda")
        pa, pw = c.pack_rows(a), c.pack_rows(w)

        def forms():
            f = c.linear_rows_packed_i8_f32(pa, sa, pw, sw, b, m, n, k)
            gq, gs = c.linear_gelu_quantize_packed(pa, sa, pw, sw, b, m, n, k)
            x_ln, x_res = x0.clone(), x0.clone()
            lq, ls = c.linear_residual_layer_norm_quantize_packed(pa, sa, pw, sw, b, m, n, k, x_ln, gamma, beta)
            c.linear_residual_layer_norm_quantize_packed(pa, sa, pw, sw, b, m, n, k, x_res, normalize=False)
            c.synchronize()  # (would report an exchange that gave up)
            return f, gq, gs, x_ln, lq, ls, x_res

        c.set_gemm_kernel_variant(15)
        single = forms()
        c.set_gemm_kernel_variant(pairs)
        for _ in range(2):
            pair = forms()
            for i in (0, 1, 2, 3, 6):
                assert torch.equal(pair[i].view(torch.int32) if pair[i].dtype == torch.float32 else pair[i],
                                   single[i].view(torch.int32) if single[i].dtype == torch.float32 else single[i]), i
            np.testing.assert_allclose(host(pair[5]), host(single[5]), rtol=1e-6, atol=0)
            diff = (pair[4].to(torch.int16) - single[4].to(torch.int16)).abs()
            assert int(diff.max()) <= 1
            assert float((diff != 0).float().mean()) <= 1e-5 + 2.0 / diff.numel()
    finally:
        c.close()


def test_pair_panels_give_up_cleanly(hipq):
    """With the spin limit forced to 0 a workgroup looks for its partner's row maxima exactly once, which is too early
    for some of the 128 pairs: the kernel must drain all the same, the context reports HIPQ_DEVICE_ERROR at the next
    synchronize, once, and the same call is right again afterwards (flags that a given-up exchange left set have
    been cleared).  The single-workgroup panels wait for nothing."""
    m, n, k = 8192, 3072, 768
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(2)
        a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
        w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
        sa = torch.rand(m, generator=g, device="cuda") * 0.02 + 0.001
        sw = torch.rand(n, generator=g, device="cuda") * 2e-3 + 1e-4
        b = torch.randn(n, generator=g, device="cuda")
        pa, pw = c.pack_rows(a), c.pack_rows(w)
        want_q, want_s = c.linear_gelu_quantize_packed(pa, sa, pw, sw, b, m, n, k)
        c.synchronize()
        c.set_wait_spin_limit(0)
        c.linear_gelu_quantize_packed(pa, sa, pw, sw, b, m, n, k)
        with pytest.raises(hipq.HipqError) as e:
            c.synchronize()
        assert e.value.code == hipq.DEVICE_ERROR and "gave up" in str(e.value)
        c.synchronize()  # reported once
        c.set_gemm_kernel_variant(15)
        q, s_ = c.linear_gelu_quantize_packed(pa, sa, pw, sw, b, m, n, k)
        c.synchronize()
        assert torch.equal(q, want_q) and torch.equal(s_, want_s)
        c.set_gemm_kernel_variant(0)
        c.set_wait_spin_limit(-1)
        for _ in range(2):
            q, s_ = c.linear_gelu_quantize_packed(pa, sa, pw, sw, b, m, n, k)
            c.synchronize()
            assert torch.equal(q, want_q) and torch.equal(s_, want_s)
    finally:
        c.close()


def test_captured_pair_panels_replay(hipq):
    """The exchange between the two workgroups of a panel keeps no host state per launch and leaves its flags at
    zero, so a captured MLP (fc1 + GELU + quantizer, fc2 + skip + LayerNorm + quantizer, both as pairs) can be
    replayed: every replay, with new inputs in the captured buffers and eager work on the same context in between,
    equals the eager forwards of the same inputs."""
    m, d, dff = 200, 256, 1024
    g = torch.Generator(device="cuda").manual_seed(21)
    w1 = torch.randint(-128, 128, (dff, d), generator=g, device="cuda", dtype=torch.int8)
    w2 = torch.randint(-128, 128, (d, dff), generator=g, device="cuda", dtype=torch.int8)
    s1 = torch.rand(dff, generator=g, device="cuda") * 2e-3 + 1e-4
    s2 = torch.rand(d, generator=g, device="cuda") * 2e-3 + 1e-4
    b1 = torch.randn(dff, generator=g, device="cuda")
    b2 = torch.randn(d, generator=g, device="cuda")
    gamma = torch.rand(d, generator=g, device="cuda") + 0.5
    beta = torch.randn(d, generator=g, device="cuda") * 0.1
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        c = hipq.Context(0)
        try:
            c.set_gemm_kernel_variant(16)
            p1, p2 = c.pack_rows(w1), c.pack_rows(w2)
            a = torch.randint(-128, 128, (m, d), generator=g, device="cuda", dtype=torch.int8)
            pa = c.pack_rows(a)
            sa = torch.rand(m, generator=g, device="cuda") * 0.02 + 0.001
            x = torch.randn(m, d, generator=g, device="cuda")

            def mlp(pa_, sa_, x_, hq=None, hs=None, oq=None, os_=None):
                hq, hs = c.linear_gelu_quantize_packed(pa_, sa_, p1, s1, b1, m, dff, d, out=hq, scales=hs)
                return (hq, hs) + tuple(c.linear_residual_layer_norm_quantize_packed(
                    hq, hs, p2, s2, b2, m, d, dff, x_, gamma, beta, out=oq, scales=os_))

            bufs = mlp(pa, sa, x.clone())  # allocates the exchange area outside the capture
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                mlp(pa, sa, x, *bufs)
            for rep in range(6):
                an = torch.randint(-128, 128, (m, d), generator=g, device="cuda", dtype=torch.int8)
                xn = torch.randn(m, d, generator=g, device="cuda") * (rep + 1)
                pa.copy_(c.pack_rows(an))
                x.copy_(xn)
                side.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                got = [t.clone() for t in bufs] + [x.clone()]
                xe = xn.clone()
                eager = list(mlp(c.pack_rows(an), sa, xe)) + [xe]
                side.synchronize()
                for i, (u, v) in enumerate(zip(got, eager)):
                    assert torch.equal(u.view(torch.int32) if u.dtype == torch.float32 else u,
                                       v.view(torch.int32) if v.dtype == torch.float32 else v), (rep, i)
            c.synchronize()  # no exchange gave up
        finally:
            torch.cuda.synchronize()
            c.close()


def test_pair_panels_on_two_contexts_that_share_the_device(hipq):
    """Two contexts that were told about each other (hipq_ctx_set_resident_share(ctx, 2)) size the shared panels for
    half of the device each: 4096 rows take the pair form on both at once (both grids are resident together, so no
    exchange waits for a workgroup that cannot start), 8192 rows no longer fit a context's share and take single
    panels.  Same bits as one context alone; no wait gives up."""
    m, n, k = 4096, 3072, 768
    g = torch.Generator(device="cuda").manual_seed(31)
    a = torch.randint(-128, 128, (2 * m, k), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sa = torch.rand(2 * m, generator=g, device="cuda") * 0.02 + 0.001
    sw = torch.rand(n, generator=g, device="cuda") * 2e-3 + 1e-4
    b = torch.randn(n, generator=g, device="cuda")
    alone = hipq.Context(0)
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ctxs = []
    try:
        pw = alone.pack_rows(w)
        pas = [alone.pack_rows(a[i * m:(i + 1) * m]) for i in range(2)]
        want = [alone.linear_gelu_quantize_packed(pas[i], sa[i * m:(i + 1) * m], pw, sw, b, m, n, k) for i in range(2)]
        pa_all = alone.pack_rows(a)
        want_all = alone.linear_gelu_quantize_packed(pa_all, sa, pw, sw, b, 2 * m, n, k)
        alone.synchronize()
        torch.cuda.synchronize()
        for s_ in streams:
            with torch.cuda.stream(s_):
                c = hipq.Context(0)
                c.call("hipq_ctx_set_resident_share", 2)
                ctxs.append(c)
        for rep in range(5):
            got = []
            for i, (c, s_) in enumerate(zip(ctxs, streams)):
                with torch.cuda.stream(s_):
                    got.append(c.linear_gelu_quantize_packed(pas[i], sa[i * m:(i + 1) * m], pw, sw, b, m, n, k))
            for c in ctxs:
                c.synchronize()  # (would report an exchange that gave up)
            for i in range(2):
                assert torch.equal(got[i][0], want[i][0]) and torch.equal(got[i][1], want[i][1]), (rep, i)
        with torch.cuda.stream(streams[0]):
            big = ctxs[0].linear_gelu_quantize_packed(pa_all, sa, pw, sw, b, 2 * m, n, k)
        ctxs[0].synchronize()
        assert torch.equal(big[0], want_all[0]) and torch.equal(big[1], want_all[1])
    finally:
        torch.cuda.synchronize()
        for c in ctxs:
            c.close()
        alone.close()


# ---- the projection stack on prepared weights ---------------------------------------------------------------

from test_gpu_stack import _make_blocks, _oracle_stack  # noqa: E402


@pytest.mark.parametrize("tokens,d,dff,layers", [(48, 128, 512, 2), (130, 256, 1024, 3)])
def test_prepared_stack_small_against_the_oracle(ctx, oracle, tokens, d, dff, layers):
    rng = np.random.default_rng(tokens + d)
    blocks_h = _make_blocks(rng, layers, d, dff, oracle)
    for blk in blocks_h:
        for ln in ("ln1", "ln2"):
            blk[ln + "_gamma"] = rng.uniform(0.5, 1.5, d).astype(np.float32)
            blk[ln + "_beta"] = (rng.standard_normal(d) * 0.1).astype(np.float32)
    x = rng.standard_normal((tokens, d)).astype(np.float32)
    want = _oracle_stack(oracle, blocks_h, x, d)
    blocks_d = [{k: dev(v) for k, v in blk.items()} for blk in blocks_h]
    prepared = ctx.stack_prepare(blocks_d)
    got = host(ctx.stack_forward(prepared, dev(x), dff, ctx.stack_workspace_prepared(tokens, d, dff), prepared=True))
    plain = host(ctx.stack_forward(blocks_d, dev(x), dff, ctx.stack_workspace(tokens, d, dff)))
    # fp32 LayerNorm / GELU rounding feeds re-quantization (an occasional code flips by one level); the same loose
    # bound as for the unprepared stack, and the two device forms as close to each other as to the oracle
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    rel_plain = np.linalg.norm(got - plain) / np.linalg.norm(plain)
    print(f"prepared stack tokens={tokens} d={d} layers={layers}: rel L2 vs oracle {rel:.3e}, vs the plain stack {rel_plain:.3e}")
    assert rel < 2e-3
    assert rel_plain < 2e-3


def test_prepared_stack_full_size_equals_its_parts(ctx, hipq):
    """Config 5 at its real size (8192 tokens, d = 768, d_ff = 3072; 3 layers keep the test short): the one call is
    bit-identical to the same layers composed from the entry points tested above, and stays within the drift bound
    of the stack on row-major weights."""
    tokens, d, dff, layers = 8192, 768, 3072, 3
    g = torch.Generator(device="cuda").manual_seed(11)
    blocks = []
    for _ in range(layers):
        blk = {}
        for name, (o, i) in {"qkv": (3 * d, d), "out": (d, d), "fc1": (dff, d), "fc2": (d, dff)}.items():
            wf = torch.randn(o, i, generator=g, device="cuda") * 0.02
            q, sc, _, _ = ctx.quantize_per_row(wf)
            blk["w_" + name], blk["s_" + name] = q, sc
            blk["b_" + name] = torch.randn(o, generator=g, device="cuda") * 0.01
        for ln in ("ln1", "ln2"):
            blk[ln + "_gamma"] = torch.rand(d, generator=g, device="cuda") + 0.5
            blk[ln + "_beta"] = torch.randn(d, generator=g, device="cuda") * 0.1
        blocks.append(blk)
    prepared = ctx.stack_prepare(blocks)
    x0 = torch.randn(tokens, d, generator=g, device="cuda")
    got = ctx.stack_forward(prepared, x0.clone(), dff, ctx.stack_workspace_prepared(tokens, d, dff), prepared=True)
    x = x0.clone()
    q, s = ctx.layer_norm_quantize(x, blocks[0]["ln1_gamma"], blocks[0]["ln1_beta"], 1e-5)
    qa = ctx.pack_rows(q)
    for i, blk in enumerate(prepared):
        qkv = ctx.linear_packed_i8_f32(qa, s, blk["w_qkv"], blk["s_qkv"], blk["b_qkv"], tokens, 3 * d, d)
        q, s = ctx.quantize_per_row_strided(qkv, tokens, d, 3 * d, elem_offset=2 * d)
        qa, s = ctx.linear_residual_layer_norm_quantize_packed(ctx.pack_rows(q), s, blk["w_out"], blk["s_out"], blk["b_out"],
                                                               tokens, d, d, x, blk["ln2_gamma"], blk["ln2_beta"])
        qb, sb = ctx.linear_gelu_quantize_packed(qa, s, blk["w_fc1"], blk["s_fc1"], blk["b_fc1"], tokens, dff, d)
        last = i + 1 == layers
        nxt = None if last else prepared[i + 1]
        qa, s = ctx.linear_residual_layer_norm_quantize_packed(
            qb, sb, blk["w_fc2"], blk["s_fc2"], blk["b_fc2"], tokens, d, dff, x,
            None if last else nxt["ln1_gamma"], None if last else nxt["ln1_beta"], normalize=not last)
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    assert torch.equal(got, x)
    plain = ctx.stack_forward(blocks, x0.clone(), dff, ctx.stack_workspace(tokens, d, dff))
    rel = float((got - plain).norm() / plain.norm())
    print(f"prepared vs plain stack at full size, {layers} layers: rel L2 {rel:.3e}")
    assert rel < 2e-3


def test_prepared_stack_arguments(ctx, hipq):
    x = torch.zeros((8, 128), device="cuda")
    with pytest.raises(hipq.HipqError) as e:
        ctx.stack_forward([{}], x, 512, torch.empty(1024, dtype=torch.uint8, device="cuda"), prepared=True)
    assert e.value.code == hipq.INVALID_ARGUMENT
    with pytest.raises(hipq.HipqError) as e:  # d_ff beyond what a workgroup's registers hold
        ctx.stack_forward([{}], x, 4096, ctx.stack_workspace_prepared(8, 128, 4096), prepared=True)
    assert e.value.code == hipq.SHAPE_ERROR
    with pytest.raises(hipq.HipqError) as e:
        ctx.stack_forward([{}], torch.zeros((8, 96), device="cuda"), 512, ctx.stack_workspace_prepared(8, 96, 512),
                          prepared=True)
    assert e.value.code == hipq.SHAPE_ERROR
