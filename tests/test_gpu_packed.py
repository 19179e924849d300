"""Parity of the fragment-packed GEMM / Linear forward (the fast path of the headline shape).

Packed operands hold the same integers as the row-major ones, so every result is compared bit for bit with
the CPU oracle (int32 accumulators, int8 outputs, and in practice the fp32 outputs too, which are also held
to the stated 1e-5 relative bar), and with the row-major entry points of the library.
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


def pack_reference(q: np.ndarray) -> np.ndarray:
    """The packed layout written out in numpy: [rows/32][k blocks, padded to 4][64 slots of 16 bytes],
    slot l = row l % 32, bytes 16 * (l // 32) .. + 15 of the 32-byte k block."""
    rows, k = q.shape
    rb, kb = (rows + 31) // 32, ((k + 31) // 32 + 3) // 4 * 4
    padded = np.zeros((rb * 32, kb * 32), np.int8)
    padded[:rows, :k] = q
    # [rb, 32 rows, kb, 2 halves, 16 bytes] -> [rb, kb, half, row, 16]
    t = padded.reshape(rb, 32, kb, 2, 16).transpose(0, 2, 3, 1, 4)
    return np.ascontiguousarray(t).reshape(-1)


@pytest.mark.parametrize("rows,k", [(1, 1), (32, 32), (33, 31), (64, 128), (100, 304), (5, 1001), (130, 4096)])
def test_pack_rows_layout(ctx, rows, k):
    rng = np.random.default_rng(rows * 7919 + k)
    q = rand_i8(rng, (rows, k))
    assert ctx.packed_size(rows, k) == pack_reference(q).size
    np.testing.assert_array_equal(host(ctx.pack_rows(dev(q))), pack_reference(q))


SHAPES = [
    (1, 1, 16), (1, 16, 64), (16, 16, 64), (17, 33, 128), (64, 64, 256), (128, 64, 128), (130, 70, 144),
    (127, 129, 4096), (512, 256, 1024), (5, 300, 48), (256, 512, 16), (33, 1000, 2048), (9, 40, 1001), (3, 5, 7),
    (129, 65, 512), (200, 96, 768), (256, 128, 2304), (96, 200, 11008),
    (2100, 1100, 512), (4100, 600, 272),  # more tiles than compute units: two workgroups per compute unit
    (65, 4096, 4096), (50, 300, 1040), (100, 7000, 512), (128, 96, 80),  # 33..128 rows: the skinny kernel's 2..4 row blocks
    (17, 9700, 96), (40, 10000, 272), (64, 9632, 1040), (1, 10016, 64),  # >= 300 weight row blocks: two per workgroup (odd counts too)
]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_packed_bit_exact(ctx, oracle, m, n, k):
    rng = np.random.default_rng(m * 1000003 + n * 1009 + k)
    a, w = rand_i8(rng, (m, k)), rand_i8(rng, (n, k))
    got = host(ctx.gemm_packed_i8_i32(ctx.pack_rows(dev(a)), ctx.pack_rows(dev(w)), m, n, k))
    np.testing.assert_array_equal(got, oracle.gemm_i8_nk(a, w))


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (512, 4096, 512), (1024, 2048, 1024), (256, 8192, 1536), (128, 16384, 512)])
def test_gemm_one_tile_per_pair_of_compute_units(hipq, oracle, m, n, k):
    """Test hook 12: one 128 x 128 tile per pair of compute units, K halved between the two workgroups, which exchange
    partial sums through the L2 of the XCD they share (shapes of whole tiles that fill the device once).  int32
    accumulators against an exact float64 product (and the oracle where it finishes in a second), the fp32
    epilogue with per-tensor and per-row activation scales against the same individually rounded f32 expression,
    and the same bits as the default form; twice in a row, since the exchange flags must be back at zero."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(m + n + k)
        a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
        w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
        ref = torch.empty((m, n), dtype=torch.int32, device="cuda")
        wd = w.double().T.contiguous()
        for r0 in range(0, m, 128):
            ref[r0:r0 + 128] = (a[r0:r0 + 128].double() @ wd).to(torch.int32)  # exact: |acc| < 2^53
        if m * n * k <= 512 * 4096 * 512:
            np.testing.assert_array_equal(host(ref), oracle.gemm_i8_nk(host(a), host(w)))
        pa, pw = c.pack_rows(a), c.pack_rows(w)
        sa = torch.rand(m, generator=g, device="cuda") * 0.05 + 0.01
        sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
        bias = torch.randn(n, generator=g, device="cuda") * 0.01
        default = c.linear_packed_i8_f32(pa, sa, pw, sw, bias, m, n, k)
        c.set_gemm_kernel_variant(12)
        for _ in range(2):
            assert torch.equal(c.gemm_packed_i8_i32(pa, pw, m, n, k), ref)
            got = c.linear_packed_i8_f32(pa, sa, pw, sw, bias, m, n, k)
            assert torch.equal(got, ref.float() * (sa[:, None] * sw[None, :]) + bias[None, :])
            assert torch.equal(got, default)
            got = c.linear_packed_i8_f32(pa, sa[:1], pw, sw, None, m, n, k)
            assert torch.equal(got, ref.float() * (sa[0] * sw[None, :]))
        c.synchronize()  # no wait of the exchange gave up
    finally:
        c.close()


def test_gemm_packed_extreme_values(ctx):
    a = np.full((32, 4096), -128, np.int8)
    pa = ctx.pack_rows(dev(a))
    got = host(ctx.gemm_packed_i8_i32(pa, pa, 32, 32, 4096))
    np.testing.assert_array_equal(got, np.full((32, 32), 4096 * 16384, np.int32))


def _linear_case(oracle, m, n, k, per_token, seed):
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
    return x, bias, wq.astype(np.int8), sw, aq.astype(np.int8), sa, acc, out


@pytest.mark.parametrize("m,n,k", [(4, 8, 16), (64, 128, 256), (100, 200, 304), (512, 512, 512), (33, 65, 1040),
                                   (130, 72, 768)])
@pytest.mark.parametrize("per_token", [False, True])
def test_linear_packed_forward(ctx, hipq, oracle, m, n, k, per_token):
    x, bias, wq, sw, aq, sa, acc, want = _linear_case(oracle, m, n, k, per_token, m + n + k)
    pw = ctx.pack_rows(dev(wq))
    # separate steps: packed int8 activations given by the caller
    got = host(ctx.linear_packed_i8_f32(ctx.pack_rows(dev(aq)), dev(sa), pw, dev(sw), dev(bias), m, n, k))
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=0)
    np.testing.assert_array_equal(got, want)
    # whole forward from fp32 activations (the reference's branch for the size: x * (1/scale) above 64 elements)
    mode = hipq.FORM_MUL_INV if x.size > 64 else hipq.FORM_DIV
    got = host(ctx.linear_dynamic_packed(dev(x), pw, dev(sw), dev(bias), per_token=per_token, mode=mode))
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=0)
    np.testing.assert_array_equal(got, want)
    # the row-major entry point gives the same bits
    np.testing.assert_array_equal(
        got, host(ctx.linear_dynamic(dev(x), dev(wq), dev(sw), dev(bias), per_token=per_token, mode=mode)))
    # no bias
    got = host(ctx.linear_packed_i8_f32(ctx.pack_rows(dev(aq)), dev(sa), pw, dev(sw), None, m, n, k))
    np.testing.assert_array_equal(got, oracle.linear_dequant_epilogue(acc, sa, sw, None))


@pytest.mark.parametrize("m,n,k", [(7, 24, 64), (128, 96, 512), (50, 130, 272), (130, 132, 384), (67, 131, 256)])
def test_linear_packed_requant_epilogue(ctx, hipq, oracle, m, n, k):
    x, bias, wq, sw, aq, sa, acc, out = _linear_case(oracle, m, n, k, False, 5 * m + k)
    s_out, _ = oracle.calculate_symmetric_params(*oracle.find_min_max(out), 0)
    pa, pw = ctx.pack_rows(dev(aq)), ctx.pack_rows(dev(wq))
    for mode, rm in ((hipq.ROUND_HALF_AWAY, 0), (hipq.ROUND_HALF_EVEN, 1)):
        oracle.set_round_mode(rm)
        try:
            wantq = oracle.requantize_epilogue(acc, sa, sw, bias, s_out, -5)
        finally:
            oracle.set_round_mode(0)
        got = host(ctx.linear_packed_i8_i8(pa, dev(sa), pw, dev(sw), dev(bias), m, n, k, s_out, -5, mode))
        np.testing.assert_array_equal(got, wantq)


@pytest.mark.parametrize("rows,cols", [(1, 8), (3, 70), (64, 256), (100, 304), (33, 1001), (512, 4096)])
def test_quantize_per_tensor_packed_matches_row_major(ctx, hipq, rows, cols):
    """Codes and parameters of the packed quantizer = those of the row-major dynamic quantizer (itself bit-exact
    with the oracle, tests/test_gpu_elementwise.py), then packed; both quantize forms and roundings; static scale."""
    g = torch.Generator(device="cuda").manual_seed(rows * 31 + cols)
    x = torch.randn(rows, cols, generator=g, device="cuda")
    x[0, 0] = 2.5 * x.abs().max()  # makes x / scale land on ties here and there
    for mode in (hipq.FORM_MUL_INV, hipq.FORM_DIV, hipq.FORM_DIV | hipq.ROUND_HALF_EVEN, hipq.ROUND_HALF_EVEN):
        q, params = ctx.quantize_dynamic_per_tensor(x, mode=mode)
        pq, pparams = ctx.quantize_per_tensor_packed(x, dynamic=True, mode=mode)
        torch.cuda.synchronize()
        assert torch.equal(pq, ctx.pack_rows(q))
        a, b = ctx.read_qparams(params), ctx.read_qparams(pparams)
        assert (a.scale, a.zero_point, a.min_val, a.max_val, a.status) == (b.scale, b.zero_point, b.min_val, b.max_val,
                                                                        b.status)
        qs = ctx.quantize_per_tensor_i8(x, 0.037, 0, mode)
        pqs, sp = ctx.quantize_per_tensor_packed(x, dynamic=False, scale=0.037, mode=mode)
        torch.cuda.synchronize()
        assert torch.equal(pqs, ctx.pack_rows(qs))
        assert ctx.read_qparams(sp).scale == np.float32(0.037)


@pytest.mark.parametrize("rows,cols", [(1, 8), (3, 70), (64, 256), (100, 304), (33, 1001), (40, 1500), (512, 4096)])
def test_quantize_per_row_packed_matches_row_major(ctx, hipq, rows, cols):
    """Codes and scales of the packed per-row quantizer = those of the row-major one (bit-exact with the oracle,
    tests/test_gpu_elementwise.py), then packed; the padding of the packed buffer is written as zeros even when
    the buffer held something else before."""
    g = torch.Generator(device="cuda").manual_seed(rows * 131 + cols)
    x = torch.randn(rows, cols, generator=g, device="cuda")
    x[rows // 2] *= 40.0
    for mode in (0, hipq.ROUND_HALF_EVEN):
        q, s, _, _ = ctx.quantize_per_row(x, mode=mode)
        dirty = torch.full((ctx.packed_size(rows, cols),), 77, dtype=torch.int8, device="cuda")
        pq, ps = ctx.quantize_per_row_packed(x, mode=mode, out=dirty)
        torch.cuda.synchronize()
        assert torch.equal(pq, ctx.pack_rows(q))
        assert torch.equal(ps, s)


@pytest.mark.parametrize("m,n,k", [(8192, 768, 768), (4100, 1100, 272)])
def test_linear_packed_many_tiles_matches_row_major(ctx, hipq, m, n, k):
    """More tiles than compute units (the packed kernel then runs two workgroups per compute unit and sums its K
    split one column block at a time), fp32 epilogue with per-row activation scales and bias: the same bits as
    the row-major entry point, which the oracle tests of tests/test_gpu_gemm.py pin."""
    g = torch.Generator(device="cuda").manual_seed(m + n + k)
    a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
    w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sa = torch.rand(m, generator=g, device="cuda") * 1e-2 + 1e-3
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(n, generator=g, device="cuda")
    want = ctx.linear_i8_f32(a, sa, w, sw, bias)
    got = ctx.linear_packed_i8_f32(ctx.pack_rows(a), sa, ctx.pack_rows(w), sw, bias, m, n, k)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("m,n,k", [(65, 4096, 4096), (128, 2048, 8192), (96, 1000, 4096), (33, 11008, 512), (64, 300, 11008),
                                   (40, 64, 48), (160, 1024, 512), (256, 4096, 256), (384, 2304, 768), (130, 100, 1040)])
def test_weight_streaming_kernel_matches_tiled(hipq, m, n, k):
    """From 33 activation rows up to as many as make one round of 64 x 64 tiles over the compute units, prepared
    operands take the weight-streaming kernel (one or two 32-row blocks of weights per workgroup against two
    activation row blocks, the row-block pair picked by the grid's second dimension); variant 9 keeps the 128 x 64
    tiles.  Same bits for the fp32 epilogue (per-row scales, bias), the requantizing one (both roundings) and the raw
    accumulators."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(m * 3 + n + k)
        a = torch.randint(-128, 128, (m, k), generator=g, device="cuda", dtype=torch.int8)
        w = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
        pa, pw = c.pack_rows(a), c.pack_rows(w)
        sa = torch.rand(m, generator=g, device="cuda") * 1e-2 + 1e-3
        sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
        bias = torch.randn(n, generator=g, device="cuda")
        got = {}
        for variant in (0, 9):
            c.set_gemm_kernel_variant(variant)
            got[variant] = (c.linear_packed_i8_f32(pa, sa, pw, sw, bias, m, n, k),
                            c.linear_packed_i8_i8(pa, sa, pw, sw, bias, m, n, k, 0.31, -3),
                            c.linear_packed_i8_i8(pa, sa[:1], pw, sw, None, m, n, k, 0.05, 7, mode=hipq.ROUND_HALF_EVEN),
                            c.gemm_packed_i8_i32(pa, pw, m, n, k))
            c.synchronize()
        for x, y in zip(got[0], got[9]):
            assert torch.equal(x, y)
        want = a.double() @ w.double().T  # exact: |acc| < 2^53
        assert torch.equal(got[0][3], want.to(torch.int32))
    finally:
        c.close()


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (256, 4096, 1024), (128, 2048, 4096), (384, 1024, 8192),
                                   (500, 4096, 4096), (512, 4032, 4096), (512, 4096, 4000), (64, 512, 1024)])
def test_dynamic_forward_with_and_without_weight_line_touching(hipq, m, n, k):
    """The dynamic per-tensor forward on prepared weights lets its activation quantizer touch weight lines for the
    GEMM while the grid waits for the range (shapes whose tiles make one round over the compute units and split into
    one rectangle per die; the last four shapes here do not qualify or are ragged).  Values read that way are not
    used: outputs and parameters are the same bits with the touching switched off (variant 11), call after call on
    rotating weights."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(m + n + k)
        sets = []
        for _ in range(3):
            wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
            sets.append((c.pack_rows(wq), torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4,
                         torch.randn(n, generator=g, device="cuda")))
        xs = [torch.randn(m, k, generator=g, device="cuda") * (i + 1) for i in range(6)]
        got = {}
        for variant in (0, 11):
            c.set_gemm_kernel_variant(variant)
            got[variant] = [c.linear_dynamic_packed(x, *sets[i % 3]).clone() for i, x in enumerate(xs)]
            c.synchronize()
        for a, b in zip(got[0], got[11]):
            assert torch.equal(a, b)
        # and against the separate calls: quantize into the packed layout, then the product
        pw, sw, bias = sets[0]
        pa, params = c.quantize_per_tensor_packed(xs[0])
        want = c.linear_packed_i8_f32(pa, params.view(torch.float32)[:1], pw, sw, bias, m, n, k)  # scale: first field
        c.synchronize()
        assert torch.equal(got[0][0], want)
    finally:
        c.close()


@pytest.mark.parametrize("m,n,k", [(1, 64, 16), (1, 11008, 4096), (4, 11008, 4096), (16, 11008, 4096), (32, 1024, 1040),
                                   (7, 300, 11008), (3, 96, 16384), (5, 4096, 272),
                                   # up to four rows in one launch (every workgroup quantizes the rows itself):
                                   (2, 512, 8192), (1, 768, 16384), (3, 1000, 4608), (1, 4096, 11008), (2, 100, 2048),
                                   (4, 33, 256), (2, 4096, 4096), (1, 64, 1024)])
def test_decode_forward_per_token(hipq, m, n, k):
    """Per-token dynamic forward with M <= 32 rows (the decode shapes of configs[2] among them), from fp32
    activations: same bits as the per-row quantizer followed by the product on its output (both pinned to the oracle
    elsewhere), for both roundings; a row with an infinite value gives a NaN row and leaves the others."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(m * 7 + n + k)
        wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
        pw = c.pack_rows(wq)
        sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
        bias = torch.randn(n, generator=g, device="cuda")
        for it in range(20):
            x = torch.randn(m, k, generator=g, device="cuda") * (it + 1)
            x[m // 2, k // 3] *= 30.0
            mode = hipq.ROUND_HALF_EVEN if it % 2 else 0
            got = c.linear_dynamic_packed(x, pw, sw, bias, per_token=True, mode=mode)
            pq, ps = c.quantize_per_row_packed(x, mode=mode)
            want = c.linear_packed_i8_f32(pq, ps, pw, sw, bias, m, n, k)
            c.synchronize()
            assert torch.equal(got, want), it
            if it == 0:  # and without a bias
                got = c.linear_dynamic_packed(x, pw, sw, None, per_token=True, mode=mode)
                want = c.linear_packed_i8_f32(pq, ps, pw, sw, None, m, n, k)
                c.synchronize()
                assert torch.equal(got, want)
        xb = x.clone()
        xb[m - 1, 5] = float("inf")
        got = c.linear_dynamic_packed(xb, pw, sw, bias, per_token=True)
        good = c.linear_dynamic_packed(x, pw, sw, bias, per_token=True)
        c.synchronize()
        assert torch.isnan(got[m - 1]).all()
        if m > 1:
            assert torch.equal(got[: m - 1], good[: m - 1])
    finally:
        c.close()


@pytest.mark.parametrize("m,n,k", [(1, 11008, 4096), (4, 11008, 4096), (3, 1000, 4096), (2, 512, 8192), (1, 300, 16384),
                                   (4, 96, 512), (2, 4096, 11008), (4, 64, 8192)])
def test_decode_forward_with_a_static_scale(hipq, m, n, k):
    """hipq_linear_static_packed_f32 with up to four rows runs as one launch where the rows fit a thread's registers
    (the last two shapes do not): same bits as the two launches (variant 6) for both quantize forms and roundings,
    with values that saturate, a NaN and an infinity among them."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(m * 11 + n + k)
        wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
        pw = c.pack_rows(wq)
        sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
        bias = torch.randn(n, generator=g, device="cuda")
        x = torch.randn(m, k, generator=g, device="cuda") * 2.0
        x[0, 3] = 1e6
        x[m - 1, 7] = float("nan")
        x[m // 2, 11] = float("-inf")
        for mode in (hipq.FORM_MUL_INV, hipq.FORM_DIV, hipq.FORM_DIV | hipq.ROUND_HALF_EVEN, hipq.ROUND_HALF_EVEN):
            for b in (bias, None):
                c.set_gemm_kernel_variant(0)
                got = c.linear_static_packed(x, 0.037, pw, sw, b, mode=mode)
                c.set_gemm_kernel_variant(6)
                want = c.linear_static_packed(x, 0.037, pw, sw, b, mode=mode)
                c.synchronize()
                assert torch.equal(got, want), mode
        c.set_gemm_kernel_variant(0)
        with pytest.raises(hipq.HipqError):
            c.linear_static_packed(x, 0.0, pw, sw, bias)
    finally:
        c.close()


def test_linear_static_packed(ctx, hipq):
    g = torch.Generator(device="cuda").manual_seed(3)
    m, n, k = 96, 160, 512
    x = torch.randn(m, k, generator=g, device="cuda")
    wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(n, generator=g, device="cuda") * 0.01
    want = ctx.linear_static(x, 0.031, wq, sw, bias, mode=hipq.FORM_MUL_INV)
    got = ctx.linear_static_packed(x, 0.031, ctx.pack_rows(wq), sw, bias, mode=hipq.FORM_MUL_INV)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("per_token", [False, True])
@pytest.mark.parametrize("bad", [float("nan"), float("inf"), float("-inf")])
def test_non_finite_activations_give_nan_outputs_not_stale_scratch(ctx, hipq, packed, per_token, bad):
    """The reference refuses a range that is not finite (algorithms.rs:403-407: an Inf among the activations).
    An asynchronous call cannot fail after the fact; it must not multiply whatever an earlier call left in the
    scratch either: the outputs that depend on the bad range are NaN (all of them per tensor, the row per token),
    the rest exact.  A NaN is different: f32::min / f32::max skip it (simd_ops.rs:95-108), the range stays finite
    and the element quantizes to 0 (`NaN as i8`), i.e. the result is that of the input with a 0.0 in its place."""
    g = torch.Generator(device="cuda").manual_seed(17)
    m, n, k = 40, 72, 256
    x = torch.randn(m, k, generator=g, device="cuda")
    wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(n, generator=g, device="cuda") * 0.01
    w_arg = ctx.pack_rows(wq) if packed else wq
    run = ctx.linear_dynamic_packed if packed else ctx.linear_dynamic
    good = run(x, w_arg, sw, bias, per_token=per_token, mode=hipq.FORM_MUL_INV)  # fills the scratch with real codes
    xb = x.clone()
    xb[7, 100] = bad
    got = run(xb, w_arg, sw, bias, per_token=per_token, mode=hipq.FORM_MUL_INV)
    torch.cuda.synchronize()
    if bad != bad:
        xz = x.clone()
        xz[7, 100] = 0.0
        want = run(xz, w_arg, sw, bias, per_token=per_token, mode=hipq.FORM_MUL_INV)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    elif per_token:
        assert torch.isnan(got[7]).all()
        keep = [i for i in range(m) if i != 7]
        assert torch.equal(got[keep], good[keep])
    else:
        assert torch.isnan(got).all()


def test_config2_full_size_packed_forward(ctx, hipq):
    """The headline Linear benchmark configuration at full size through the packed forward the bench times: M=512, K=N=4096.  int8
    activations against torch's formulation of clamp(round_half_away(x * (1/s))), accumulators against an exact
    float64 product, fp32 output against the same individually rounded f32 expression (1e-5 relative stated;
    equal in practice), and the row-major entry point against the packed one."""
    g = torch.Generator(device="cuda").manual_seed(2)
    m, n, k = 512, 4096, 4096
    x = torch.randn(m, k, generator=g, device="cuda")
    wf = torch.randn(n, k, generator=g, device="cuda") * 0.02
    bias = torch.randn(n, generator=g, device="cuda") * 0.01
    wq, sw, _, _ = ctx.quantize_per_row(wf)
    pw = ctx.pack_rows(wq)
    out = ctx.linear_dynamic_packed(x, pw, sw, bias, per_token=False, mode=hipq.FORM_MUL_INV)
    # activations: a2 + a5 (len > 64 branch), restated with torch ops
    absmax = x.abs().max()
    s = absmax / 127.0
    inv = 1.0 / s
    t = x * inv
    # f32::round = trunc(t + copysign(0.5, t)), exact except where t + 0.5 rounds up across an integer, which
    # happens only for |t| = 0.49999997: make sure no element sits there, then the simple form is the definition
    assert not bool(((t.abs() > 0.4999999) & (t.abs() < 0.5)).any())
    qa = torch.clamp(torch.trunc(t + torch.copysign(torch.full_like(t, 0.5), t)), -128, 127)
    pq, params = ctx.quantize_per_tensor_packed(x, dynamic=True, mode=hipq.FORM_MUL_INV)
    torch.cuda.synchronize()
    assert ctx.read_qparams(params).scale == float(s)
    assert torch.equal(pq, ctx.pack_rows(qa.to(torch.int8)))
    acc = (qa.double() @ wq.double().T)  # exact: |acc| < 2^53
    assert torch.equal(ctx.gemm_packed_i8_i32(pq, pw, m, n, k), acc.to(torch.int32))
    want = acc.float() * (s * sw[None, :]) + bias[None, :]  # same individually rounded f32 operations
    torch.cuda.synchronize()
    torch.testing.assert_close(out, want, rtol=RTOL, atol=0)
    assert torch.equal(out, want)
    assert torch.equal(out, ctx.linear_dynamic(x, wq, sw, bias, per_token=False, mode=hipq.FORM_MUL_INV))


def test_packed_argument_errors(ctx, hipq):
    a = torch.zeros(1024, dtype=torch.int8, device="cuda")
    out = torch.zeros((4, 4), dtype=torch.int32, device="cuda")
    with pytest.raises(hipq.HipqError) as e:
        ctx.call("hipq_gemm_packed_i8_i32", a.data_ptr(), None, 4, 4, 16, out.data_ptr())
    assert e.value.code == hipq.INVALID_ARGUMENT
    with pytest.raises(hipq.HipqError) as e:
        ctx.call("hipq_gemm_packed_i8_i32", a.data_ptr(), a.data_ptr(), 4, 4, 1 << 17, out.data_ptr())
    assert e.value.code == hipq.SHAPE_ERROR
    with pytest.raises(hipq.HipqError) as e:  # packed operand of 2 GiB or more
        ctx.call("hipq_gemm_packed_i8_i32", a.data_ptr(), a.data_ptr(), 1 << 20, 4, 4096, out.data_ptr())
    assert e.value.code == hipq.SHAPE_ERROR
    ctx.call("hipq_gemm_packed_i8_i32", a.data_ptr(), a.data_ptr(), 0, 4, 16, None)  # empty M: no-op


def test_phase_stamps_do_not_change_the_product(ctx, hipq, oracle):
    """hipq_ctx_set_trace_buffer: the stamped form of the kernel gives the same bits, every wave of the grid
    writes its record (six increasing shader-clock values, then the 100 MHz counter at the first and the last of
    them), and a buffer that is too small leaves the ordinary kernel in place."""
    m, n, k = 256, 192, 1024
    x, bias, wq, sw, aq, sa, acc, want = _linear_case(oracle, m, n, k, False, 77)
    pa, pw = ctx.pack_rows(dev(aq)), ctx.pack_rows(dev(wq))
    plain = host(ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(bias), m, n, k))
    waves = ((m + 127) // 128) * ((n + 63) // 64) * 4
    trace = torch.zeros(waves, 8, dtype=torch.int64, device="cuda")
    ctx.set_trace_buffer(trace)
    try:
        stamped = host(ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(bias), m, n, k))
        ctx.set_trace_buffer(trace[:1])  # too small: ignored
        small = host(ctx.linear_packed_i8_f32(pa, dev(sa), pw, dev(sw), dev(bias), m, n, k))
    finally:
        ctx.set_trace_buffer(None)
    np.testing.assert_array_equal(stamped, plain)
    np.testing.assert_array_equal(small, plain)
    t = trace.cpu().numpy()
    assert (t[:, :6] > 0).all()
    assert (np.diff(t[:, :6], axis=1) >= 0).all()
    assert (t[:, 7] >= t[:, 6]).all()


def test_one_launch_dynamic_quantize_over_many_launches(hipq):
    """The dynamic per-tensor packed quantizer of matrices of up to 16 Mi elements is one kernel (one or four
    fragments per wave, at most four workgroups per compute unit) whose workgroups meet through device words of the
    context, numbered by a counter in device memory that starts
    a few launches before its wrap.  A fresh context therefore crosses the wrap here; grids of different sizes
    follow one another (a small one after a large one leaves the large one's words behind), inputs change between
    launches, and every launch must give the codes and parameters of the row-major dynamic quantizer (bit-exact
    with the oracle, tests/test_gpu_elementwise.py), as must the two-launch form (variant 6) it replaces."""
    c = hipq.Context(0)
    try:
        shapes = [(512, 4096), (1, 16), (1000, 1008), (33, 48), (64, 256), (1024, 4096), (100, 304), (31, 4096),
                  (2048, 4096), (5000, 1008)]  # the last two: four fragments per wave
        g = torch.Generator(device="cuda").manual_seed(99)
        for it in range(48):
            rows, cols = shapes[it % len(shapes)]
            x = torch.randn(rows, cols, generator=g, device="cuda") * (1.0 + it)
            mode = (0, hipq.FORM_DIV, hipq.ROUND_HALF_EVEN, hipq.FORM_DIV | hipq.ROUND_HALF_EVEN)[it % 4]
            q, params = c.quantize_dynamic_per_tensor(x, mode=mode)
            pq, pparams = c.quantize_per_tensor_packed(x, dynamic=True, mode=mode)
            c.set_gemm_kernel_variant(6)
            pq2, pparams2 = c.quantize_per_tensor_packed(x, dynamic=True, mode=mode)
            c.set_gemm_kernel_variant(0)
            c.synchronize()
            want = c.pack_rows(q)
            assert torch.equal(pq, want) and torch.equal(pq2, want), (it, rows, cols)
            a, b, b2 = c.read_qparams(params), c.read_qparams(pparams), c.read_qparams(pparams2)
            for p in (b, b2):
                assert (a.scale, a.zero_point, a.min_val, a.max_val, a.status) == (p.scale, p.zero_point, p.min_val,
                                                                                p.max_val, p.status), (it, rows, cols)
    finally:
        c.close()


def test_flat_one_launch_dynamic_quantize_over_many_launches(hipq):
    """The same one-launch quantizer with a row-major output, behind hipq_linear_dynamic_f32 (activations of up to
    4 Mi elements, a multiple of 4): over a fresh context's first 48 launches (across the wrap of the meeting
    number, grids of changing size, all four modes) the forward equals the one whose quantizer runs as two
    launches (variant 6), which tests/test_gpu_gemm.py pins to the oracle."""
    c = hipq.Context(0)
    try:
        shapes = [(512, 4096), (1, 4), (1000, 1008), (33, 48), (64, 256), (1024, 4096), (100, 304), (3, 20), (7, 9)]
        g = torch.Generator(device="cuda").manual_seed(123)
        n = 40
        for it in range(48):
            m, k = shapes[it % len(shapes)]
            x = torch.randn(m, k, generator=g, device="cuda") * (1.0 + it)
            wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
            sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
            bias = torch.randn(n, generator=g, device="cuda")
            mode = (0, hipq.FORM_DIV, hipq.ROUND_HALF_EVEN, hipq.FORM_DIV | hipq.ROUND_HALF_EVEN)[it % 4]
            got = c.linear_dynamic(x, wq, sw, bias, mode=mode)
            c.set_gemm_kernel_variant(6)
            want = c.linear_dynamic(x, wq, sw, bias, mode=mode)
            c.set_gemm_kernel_variant(0)
            c.synchronize()
            assert torch.equal(got, want), (it, m, k, mode)
    finally:
        c.close()


def test_resident_share_changes_the_path_not_the_result(hipq):
    """hipq_ctx_set_resident_share(ctx, n) tells a context that n contexts launch concurrently: the one-launch
    quantizers then size their grids for 1 / n of the device and what does not fit takes two launches.  The codes
    and parameters are the same whatever the share; out-of-range shares are refused."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(21)
        for rows, cols in ((512, 4096), (2048, 4096), (4096, 4096)):
            x = torch.randn(rows, cols, generator=g, device="cuda")
            want = None
            for share in (1, 2, 4, 8, 64):
                c.set_resident_share(share)
                pq, pparams = c.quantize_per_tensor_packed(x, dynamic=True)
                q, params = c.quantize_dynamic_per_tensor(x.reshape(-1))
                c.synchronize()
                got = (pq.clone(), q.clone(), c.read_qparams(pparams).scale, c.read_qparams(params).scale)
                if want is None:
                    want = got
                assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]) and got[2:] == want[2:], (rows, share)
        for bad in (0, -1, 65):
            with pytest.raises(hipq.HipqError):
                c.set_resident_share(bad)
    finally:
        c.close()


def test_two_contexts_meet_side_by_side(hipq):
    """Two contexts on two streams, each told that two contexts launch concurrently (hipq_ctx_set_resident_share),
    run their one-launch quantizers and Linear steps at the same time for a few hundred launches: each has its own
    meeting words, the grids of both fit the device together, and every result equals the one the same context
    computes alone afterwards."""
    a, b = hipq.Context(0, own_stream=True), hipq.Context(0, own_stream=True)
    try:
        a.set_resident_share(2)
        b.set_resident_share(2)
        g = torch.Generator(device="cuda").manual_seed(77)
        m, n, k = 512, 1024, 4096
        pw = a.pack_rows(torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8))
        sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
        xs = [torch.randn(m, k, generator=g, device="cuda") * (i + 1) for i in range(6)]
        big = [torch.randn(2048 * 4096, generator=g, device="cuda") * (i + 1) for i in range(2)]
        a.synchronize()
        torch.cuda.synchronize()  # the inputs were made on torch's stream, the contexts have their own
        outs = {}
        for it in range(240):
            c = a if it % 2 == 0 else b
            if it % 8 < 6:
                outs[it] = c.linear_dynamic_packed(xs[it % 6], pw, sw, None)
            else:
                outs[it] = c.quantize_dynamic_per_tensor(big[it % 2])[0]
        a.synchronize()
        b.synchronize()
        for it in range(0, 240, 7):
            if it % 8 < 6:
                want = a.linear_dynamic_packed(xs[it % 6], pw, sw, None)
            else:
                want = a.quantize_dynamic_per_tensor(big[it % 2])[0]
            a.synchronize()
            assert torch.equal(outs[it], want), it
    finally:
        a.close()
        b.close()


def test_one_launch_forms_beside_unrelated_work_on_the_device(hipq):
    """Co-tenancy: a plain torch stream that knows nothing of the library keeps the device busy (long elementwise
    kernels over a 256 MiB tensor, back to back, on a side stream) while a context runs the forms whose workgroups
    wait for each other - the dynamic Linear forward on prepared weights, the 16 Mi-element dynamic quantize (four
    workgroups per compute unit, all of which must be resident), the convolution from fp32 - a few hundred times.
    Every result must equal the quiet-device result and no wait may give up (hipq_ctx_synchronize would say so).
    The other tenant's workgroups finish on their own, so every wait ends normally; nothing is made to hang."""
    c = hipq.Context(0)
    side = torch.cuda.Stream()
    try:
        g = torch.Generator(device="cuda").manual_seed(77)
        m, n, k = 512, 1024, 4096
        xs = [torch.randn(m, k, generator=g, device="cuda") * (i + 1) for i in range(4)]
        pw = c.pack_rows(torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8))
        sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
        bias = torch.randn(n, generator=g, device="cuda")
        big = torch.randn(4096 * 4096, generator=g, device="cuda")
        want_lin = [c.linear_dynamic_packed(x, pw, sw, bias) for x in xs]
        want_q, want_p = c.quantize_dynamic_per_tensor(big)
        c.synchronize()
        want_scale = c.read_qparams(want_p).scale
        noise_a = torch.randn(64 << 20, device="cuda")
        noise_b = torch.empty_like(noise_a)
        torch.cuda.synchronize()
        outs, qs = [], []
        for it in range(240):
            with torch.cuda.stream(side):  # the other tenant: enqueued ahead, so that it is running throughout
                for _ in range(2):
                    torch.mul(noise_a, 1.0001, out=noise_b)
                    torch.add(noise_b, 0.5, out=noise_a)
            outs.append(c.linear_dynamic_packed(xs[it % 4], pw, sw, bias))
            if it % 8 == 0:
                qs.append(c.quantize_dynamic_per_tensor(big))
        c.synchronize()  # raises if a bounded wait gave up
        side.synchronize()
        for it, o in enumerate(outs):
            assert torch.equal(o, want_lin[it % 4]), it
        for q, p in qs:
            assert torch.equal(q, want_q) and c.read_qparams(p).scale == want_scale
            assert c.read_qparams(p).status == hipq.SUCCESS
    finally:
        torch.cuda.synchronize()
        c.close()


def test_one_launch_dynamic_quantize_gives_up_cleanly(hipq):
    """With the spin limit forced to 0 every workgroup looks at the other workgroups' range words exactly once,
    which with hundreds of workgroups is certain to come too early for some of them: the kernel must still drain, a
    workgroup that gave up must leave zero codes (never codes made with a partial range), the others the right
    codes, and the context must report HIPQ_DEVICE_ERROR at the next synchronize, once, and work normally again
    afterwards."""
    c = hipq.Context(0)
    try:
        g = torch.Generator(device="cuda").manual_seed(5)
        x = torch.randn(512, 4096, generator=g, device="cuda")
        q, params = c.quantize_dynamic_per_tensor(x)
        want = c.pack_rows(q)
        c.synchronize()
        c.set_wait_spin_limit(0)
        pq, pparams = c.quantize_per_tensor_packed(x, dynamic=True)
        with pytest.raises(hipq.HipqError) as e:
            c.synchronize()
        assert e.value.code == hipq.DEVICE_ERROR and "gave up" in str(e.value)
        p = c.read_qparams(pparams)
        # The record normally carries the error too (workgroup 0 writes it when it gave up itself, then with a NaN
        # scale, or sees the context marked; a workgroup that stopped waiting for workgroup 0 writes it as well),
        # but those two writers are not ordered: the synchronize above is the report that cannot be missed.
        assert p.status in (hipq.SUCCESS, hipq.DEVICE_ERROR)
        assert p.scale != p.scale or p.scale == c.read_qparams(params).scale
        assert bool(((pq == 0) | (pq == want)).all())  # never codes made with part of the range
        c.synchronize()  # reported once, then cleared
        c.set_wait_spin_limit(-1)
        for _ in range(3):
            pq, pparams = c.quantize_per_tensor_packed(x, dynamic=True)
            c.synchronize()
            assert torch.equal(pq, want)
            assert c.read_qparams(pparams).scale == c.read_qparams(params).scale
    finally:
        c.close()


def test_captured_dynamic_linear_replays(hipq):
    """The one-launch quantizer keeps no host state per launch (its meeting number lives in device memory), so a
    captured dynamic Linear forward can be replayed: every replay, with new activations in the captured input
    buffer and eager work on the same context in between, equals the eager forward of the same activations."""
    m, n, k = 512, 1024, 1024
    g = torch.Generator(device="cuda").manual_seed(8)
    wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    bias = torch.randn(n, generator=g, device="cuda")
    x = torch.randn(m, k, generator=g, device="cuda")
    out = torch.empty(m, n, device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        c = hipq.Context(0)
        try:
            pw = c.pack_rows(wq)
            c.linear_dynamic_packed(x, pw, sw, bias, out=out)  # grows the scratch outside the capture
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                c.linear_dynamic_packed(x, pw, sw, bias, out=out)
            for rep in range(24):
                xn = torch.randn(m, k, generator=g, device="cuda") * (rep + 1)
                x.copy_(xn)
                side.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                got = out.clone()
                eager = c.linear_dynamic_packed(xn, pw, sw, bias)
                side.synchronize()
                assert torch.equal(got, eager), rep
            # The captured kernels hold pointers into the context scratch of the time of the capture.  An eager
            # call that outgrows it must not free that block: the graph is replayed again afterwards.
            mb, kb = 4096, 4096  # 16 MiB of packed activations: more than the scratch of a new context
            xb = torch.randn(mb, kb, generator=g, device="cuda")
            wb = c.pack_rows(torch.randint(-128, 128, (64, kb), generator=g, device="cuda", dtype=torch.int8))
            big = c.linear_dynamic_packed(xb, wb, sw[:64], None)
            side.synchronize()
            for rep in range(3):
                xn = torch.randn(m, k, generator=g, device="cuda") * (rep + 2)
                x.copy_(xn)
                side.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                got = out.clone()
                eager = c.linear_dynamic_packed(xn, pw, sw, bias)
                side.synchronize()
                assert torch.equal(got, eager), rep
            assert torch.equal(big, c.linear_dynamic_packed(xb, wb, sw[:64], None))
        finally:
            torch.cuda.synchronize()
            c.close()


def test_scratch_growth_under_capture_is_refused_not_attempted(hipq):
    """A call that would have to allocate context scratch while its stream is capturing returns
    HIPQ_ALLOCATION_ERROR (memory cannot be allocated under capture) and records nothing; the same call outside a
    capture then works, and so does a capture of it afterwards."""
    m, n, k = 4096, 64, 4096  # needs 16 MiB of scratch, a new context holds 8
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(m, k, generator=g, device="cuda")
    wq = torch.randint(-128, 128, (n, k), generator=g, device="cuda", dtype=torch.int8)
    sw = torch.rand(n, generator=g, device="cuda") * 1e-3 + 1e-4
    out = torch.empty(m, n, device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        c = hipq.Context(0)
        try:
            pw = c.pack_rows(wq)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            refused = None
            with torch.cuda.graph(graph, stream=side):
                try:
                    c.linear_dynamic_packed(x, pw, sw, None, out=out)
                except hipq.HipqError as e:
                    refused = e
            assert refused is not None and refused.code == hipq.ALLOCATION_ERROR and "capturing" in str(refused)
            del graph
            want = c.linear_dynamic_packed(x, pw, sw, None)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                c.linear_dynamic_packed(x, pw, sw, None, out=out)
            for _ in range(2):
                out.zero_()
                side.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(out, want)
        finally:
            torch.cuda.synchronize()
            c.close()
