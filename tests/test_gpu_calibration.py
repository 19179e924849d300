"""Parity of the calibration / metrics kernels (through the C-ABI) with the CPU oracle.

Integer results (histogram counts, non-finite counts, zero-error counts) and order-independent
float results (min, max, max error, the fake-quantized image) are bit-exact.  Sums are compared
with a stated tolerance: the reference adds f32 terms in element order, the kernels carry f64, so
against the oracle's f64-sum variant the tolerance is 1e-6 relative, and against the faithful f32
sequential sums it is 1e-5 on inputs short enough (<= 4096 elements) that the sequential f32 sum
itself is that accurate.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXACT_FIELDS = ("max_error", "zero_error_percentage", "compression_ratio")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def normal(seed, shape, std=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * std).astype(np.float32)


@pytest.fixture(scope="module")
def cal():
    with open(os.path.join(ROOT, "tests", "golden", "calibration_vectors.json")) as f:
        return json.load(f)


def check_metrics(got, want32, want64, rel32=None):
    for k in EXACT_FIELDS:
        assert np.float32(got[k]) == np.float32(want64[k]), (k, got[k], want64[k])
    for k in ("mse", "psnr", "snr", "mae", "cosine_similarity"):
        g, w = float(got[k]), float(want64[k])
        if math.isinf(w):
            assert g == w, (k, g, w)
        else:
            assert g == pytest.approx(w, rel=1e-6, abs=1e-7), (k, g, w)
        if rel32 is not None and not math.isinf(float(want32[k])):
            assert g == pytest.approx(float(want32[k]), rel=rel32, abs=1e-7), (k, g, want32[k])


def test_metrics_golden_vectors(ctx, oracle, cal):
    for case in cal["metrics"]:
        a, b = np.float32(case["original"]), np.float32(case["quantized"])
        got = ctx.read_metrics(ctx.quantization_metrics(dev(a), dev(b), case["original_bits"], case["quantized_bits"]))
        want32 = oracle.calculate_quantization_metrics(a, b, case["original_bits"], case["quantized_bits"])
        want64 = oracle.calculate_quantization_metrics_f64(a, b, case["original_bits"], case["quantized_bits"])
        check_metrics(got, want32, want64, rel32=1e-5)
        assert got["compression_ratio"] == case["assert"]["compression_ratio"]
    empty = torch.empty(0, dtype=torch.float32, device="cuda")
    got = ctx.read_metrics(ctx.quantization_metrics(empty, empty))
    assert got == dict(mse=0, psnr=0, snr=0, mae=0, max_error=0, zero_error_percentage=100, cosine_similarity=1,
                       compression_ratio=1)


@pytest.mark.parametrize("n", [1, 3, 64, 1000, 4096, 4099, 65536 + 7, 1 << 20])
def test_metrics_two_tensors(ctx, oracle, n):
    a = normal(n, n)
    b = (a + normal(n + 1, n, 0.02)).astype(np.float32)
    b[:: 7] = a[:: 7]                                  # some exact matches
    got = ctx.read_metrics(ctx.quantization_metrics(dev(a), dev(b), 32, 8))
    check_metrics(got, oracle.calculate_quantization_metrics(a, b), oracle.calculate_quantization_metrics_f64(a, b),
                  rel32=1e-5 if n <= 4096 else None)


def test_metrics_unaligned_views(ctx, oracle):
    a = normal(21, 10000)
    b = (a * np.float32(1.01)).astype(np.float32)
    da, db = dev(a), dev(b)
    for off in (1, 2, 3):
        got = ctx.read_metrics(ctx.quantization_metrics(da[off:], db[off:]))
        check_metrics(got, None, oracle.calculate_quantization_metrics_f64(a[off:], b[off:]))


def test_metrics_closed_forms_on_device(ctx):
    n = 1 << 16
    got = ctx.read_metrics(ctx.quantization_metrics(dev(np.full(n, 4.0, np.float32)), dev(np.full(n, 4.5, np.float32)), 32, 4))
    assert got["mse"] == 0.25 and got["mae"] == 0.5 and got["max_error"] == 0.5 and got["zero_error_percentage"] == 0
    assert got["psnr"] == pytest.approx(20 * math.log10(8.0), rel=1e-6)
    assert got["snr"] == pytest.approx(10 * math.log10(64.0), rel=1e-6)
    assert got["cosine_similarity"] == pytest.approx(1.0, abs=1e-6) and got["compression_ratio"] == 8.0
    got = ctx.read_metrics(ctx.quantization_metrics(dev(np.float32([2.0, 0.0])), dev(np.float32([0.0, 4.0]))))
    assert got["mse"] == 10.0 and got["mae"] == 3.0 and got["cosine_similarity"] == 0.0
    assert got["psnr"] == pytest.approx(20 * math.log10(2.0 / math.sqrt(10.0)), rel=1e-6)
    assert got["snr"] == pytest.approx(10 * math.log10(0.2), rel=1e-6)


@pytest.mark.parametrize("form", ["mul_inv", "div"])
@pytest.mark.parametrize("n", [5, 4096, 100003, 1 << 20])
def test_fused_fake_quantize_metrics_equal_the_three_step_path(ctx, hipq, oracle, n, form):
    # compare_quantization_configs: quantize (x * 1/scale form for len > 64) -> dequantize -> metrics.
    x = normal(100 + n, n, 2.0)
    mn, mx = oracle.find_min_max(x)
    scale, zp = oracle.calculate_affine_params(mn, mx, oracle.DTYPE_I8)
    mode = hipq.FORM_DIV if form == "div" else hipq.FORM_MUL_INV
    if form == "div":
        y = oracle.model_fake_quantize(x, scale, zp)
    else:
        y = oracle.dequantize_per_tensor_affine(oracle.quantize_per_tensor_affine_simd(x, scale, zp), scale, zp)
    got = ctx.read_metrics(ctx.fake_quantize_metrics(dev(x), scale, zp, -128, 127, mode))
    check_metrics(got, oracle.calculate_quantization_metrics(x, y), oracle.calculate_quantization_metrics_f64(x, y),
                  rel32=1e-5 if n <= 4096 else None)
    # and the image itself, bit for bit
    img = host(ctx.fake_quantize(dev(x), scale, zp, -128, 127, mode | (hipq.FAKE_INT_CAST if form == "div" else 0)))
    np.testing.assert_array_equal(img, y)
    # two-tensor kernel on the materialised image gives the same record as the fused kernel
    two = ctx.read_metrics(ctx.quantization_metrics(dev(x), dev(y)))
    for k in two:
        assert two[k] == pytest.approx(got[k], rel=1e-6, abs=1e-9) or (math.isinf(two[k]) and two[k] == got[k])


def test_fake_quantize_metrics_with_device_params(ctx, hipq, oracle):
    x = normal(77, 50000)
    q, params = ctx.quantize_dynamic_per_tensor(dev(x), hipq.PARAMS_AFFINE)
    p = ctx.read_qparams(params)
    got = ctx.read_metrics(ctx.fake_quantize_metrics(dev(x), 0.0, 0, -128, 127, 0, params=params))
    want = ctx.read_metrics(ctx.fake_quantize_metrics(dev(x), p.scale, p.zero_point, -128, 127, 0))
    assert got == want


def test_fake_quantize_nan_semantics_and_errors(ctx, hipq, oracle):
    x = np.float32([float("nan"), 1.2, float("inf"), -float("inf"), 1.25, -1.25])
    want = oracle.model_fake_quantize(x, 0.5, 3)
    got = host(ctx.fake_quantize(dev(x), 0.5, 3, -128, 127, hipq.FORM_DIV | hipq.FAKE_INT_CAST))
    np.testing.assert_array_equal(got, want)
    carrier = host(ctx.fake_quantize(dev(x), 0.5, 3, -128, 127, hipq.FORM_DIV))
    assert np.isnan(carrier[0])
    np.testing.assert_array_equal(carrier[1:], want[1:])
    with pytest.raises(hipq.HipqError) as e:
        ctx.fake_quantize(dev(x), 0.0, 0)
    assert e.value.code == hipq.INVALID_ARGUMENT and "Scale must be positive" in e.value.message
    with pytest.raises(hipq.HipqError):
        ctx.fake_quantize_metrics(dev(x), 1.0, 0, 5, -5)
    with pytest.raises(hipq.HipqError):
        ctx.fake_quantize(dev(x), 1.0, 0, mode=64)


@pytest.mark.parametrize("n", [1, 7, 4096, 4099, (1 << 20) + 3])
@pytest.mark.parametrize("qrange", [(-128, 127), (0, 255)])
def test_qat_fake_quantize_matches_reference_formula(ctx, hipq, oracle, n, qrange):
    """fake_quantize_per_tensor_affine of the QAT module: division form, clamp by max-then-min (a NaN becomes qmin),
    scale * (q - zp).  Bit-exact against the oracle, ties, saturation and non-finite inputs included."""
    qmin, qmax = qrange
    x = normal(300 + n, n, 2.0)
    special = np.float32([np.nan, np.inf, -np.inf, 0.25, -0.25, 0.75, 1e9, -1e9])
    x[: min(n, special.size)] = special[: min(n, special.size)]
    scale, zp = 0.5 if n % 2 else 0.0173, 3
    mode = hipq.FORM_DIV | hipq.FAKE_NAN_TO_QMIN
    want = oracle.fake_quantize_per_tensor_affine(x, scale, zp, qmin, qmax)
    got = host(ctx.fake_quantize(dev(x), scale, zp, qmin, qmax, mode))
    np.testing.assert_array_equal(got, want)
    assert not np.isnan(got).any()
    # the fused form measures exactly that image
    finite = np.where(np.isfinite(x), x, np.float32(0.0)).astype(np.float32)
    want_m = oracle.calculate_quantization_metrics_f64(finite, oracle.fake_quantize_per_tensor_affine(finite, scale, zp, qmin, qmax))
    got_m = ctx.read_metrics(ctx.fake_quantize_metrics(dev(finite), scale, zp, qmin, qmax, mode))
    for key in ("mse", "mae", "max_error", "cosine_similarity"):
        assert got_m[key] == pytest.approx(want_m[key], rel=1e-6, abs=1e-12), key
    with pytest.raises(hipq.HipqError):
        ctx.fake_quantize(dev(x), scale, zp, qmin, qmax, hipq.FAKE_INT_CAST | hipq.FAKE_NAN_TO_QMIN)


# ---- observers -------------------------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 63, 4096, 4097, 1 << 20, (1 << 22) + 5])
def test_observe_range_and_nonfinite_count(ctx, oracle, n):
    x = normal(n + 9, n, 3.0)
    st = ctx.read_observe(ctx.observe(dev(x)))
    mn, mx = oracle.min_max_fold(x)
    assert (st.min_val, st.max_val, st.nonfinite) == (mn, mx, 0)
    if n >= 63:
        x[5], x[n // 2], x[n - 1] = np.nan, np.inf, -np.inf
        st = ctx.read_observe(ctx.observe(dev(x)))
        assert st.nonfinite == 3


def test_observe_empty(ctx):
    st = ctx.read_observe(ctx.observe(torch.empty(0, dtype=torch.float32, device="cuda")))
    assert st.min_val == float("inf") and st.max_val == -float("inf") and st.nonfinite == 0


@pytest.mark.parametrize("bins", [1, 10, 256, 1000, 2048, 5000, 16384])
def test_histogram_counts_are_exact(ctx, oracle, bins):
    n = 300000
    x = normal(bins, n, 1.5)
    lo, hi = oracle.min_max_fold(x)
    got = host(ctx.histogram(dev(x), lo, hi, bins)).astype(np.uint64)
    want = oracle.histogram_accumulate(x, lo, hi, bins)
    np.testing.assert_array_equal(got, want)
    assert int(got.sum()) == n


def test_histogram_edges_clamping_and_accumulation(ctx, oracle):
    x = np.float32([-5.0, 0.0, 0.999, 1.0, 9.999, 10.0, 11.0, 1e30, float("nan"), float("inf"), -float("inf")])
    counts = ctx.histogram(dev(x), 0.0, 10.0, 10)
    want = oracle.histogram_accumulate(x, 0.0, 10.0, 10)
    np.testing.assert_array_equal(host(counts).astype(np.uint64), want)
    # second batch adds into the same counters; a narrower range than the data clamps to the end bins
    y = normal(4, 70001, 4.0)
    counts = ctx.histogram(dev(y), -1.0, 1.0, 10, counts=counts)
    want = oracle.histogram_accumulate(y, -1.0, 1.0, 10, counts=want)
    np.testing.assert_array_equal(host(counts).astype(np.uint64), want)
    # degenerate ranges: everything in bin 0
    for lo, hi in ((3.0, 3.0), (4.0, 3.0)):
        got = host(ctx.histogram(dev(y), lo, hi, 16))
        assert got[0] == y.size and got[1:].sum() == 0


def test_histogram_awkward_ranges_bit_exact(ctx, oracle):
    # Ranges whose width is not a power of two and values sitting on bin edges: the bin index depends on the
    # correctly rounded quotient, so this fails if the division is replaced by a multiplication.
    rng = np.random.default_rng(8)
    for lo, hi, bins in ((-0.7, 2.9, 256), (1e-3, 3e-3, 100), (-1e6, 3.3e6, 777), (0.1, 0.7, 6)):
        edges = (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * (np.arange(bins + 1, dtype=np.float32) / np.float32(bins)))
        x = np.concatenate([edges, np.nextafter(edges, np.float32(-np.inf)), np.nextafter(edges, np.float32(np.inf)),
                            rng.uniform(lo, hi, 50000).astype(np.float32)]).astype(np.float32)
        got = host(ctx.histogram(dev(x), lo, hi, bins)).astype(np.uint64)
        np.testing.assert_array_equal(got, oracle.histogram_accumulate(x, lo, hi, bins), err_msg=str((lo, hi, bins)))


def test_histogram_unaligned_and_errors(ctx, hipq, oracle):
    x = normal(31, 100001)
    dx = dev(x)
    for off in (1, 2, 3):
        got = host(ctx.histogram(dx[off:], -4.0, 4.0, 64)).astype(np.uint64)
        np.testing.assert_array_equal(got, oracle.histogram_accumulate(x[off:], -4.0, 4.0, 64))
    with pytest.raises(hipq.HipqError):
        ctx.histogram(dx, 0.0, 1.0, 0, counts=torch.zeros(1, dtype=torch.int64, device="cuda"))
    with pytest.raises(hipq.HipqError) as e:
        ctx.histogram(dx, 0.0, 1.0, hipq.HISTOGRAM_MAX_BINS + 1)
    assert "exceeds" in e.value.message


def test_histogram_observer_sequence_matches_the_oracle(ctx, oracle):
    # The observer's own update order: range first (grown by the batch), then the batch is binned over it.
    ob = oracle.Observer(oracle.OBS_HISTOGRAM)
    counts = torch.zeros(256, dtype=torch.int64, device="cuda")
    hmin, hmax = np.float32(np.inf), np.float32(-np.inf)
    for i, std in enumerate((1.0, 0.5, 3.0, 2.0)):
        x = normal(500 + i, 123457, std)
        ob.update(x)
        st = ctx.read_observe(ctx.observe(dev(x)))
        assert st.nonfinite == 0
        hmin, hmax = min(hmin, np.float32(st.min_val)), max(hmax, np.float32(st.max_val))
        ctx.histogram(dev(x), hmin, hmax, 256, counts=counts)
        np.testing.assert_array_equal(host(counts).astype(np.uint64), ob.histogram())
    assert ob.get_hist_range() == (hmin, hmax)


def test_full_size_properties(ctx, hipq, oracle):
    # 4096 x 4096 (the streaming configuration): size-independent properties.
    n = 4096 * 4096
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(n, dtype=torch.float32, device="cuda", generator=g)
    mm = host(ctx.minmax(x))
    st = ctx.read_observe(ctx.observe(x))
    assert (st.min_val, st.max_val, st.nonfinite) == (mm[0], mm[1], 0)
    counts = host(ctx.histogram(x, mm[0], mm[1], 256))
    assert counts.sum() == n and counts.min() >= 0
    # histogram of a concatenation = sum of histograms
    c2 = ctx.histogram(x[: n // 2], mm[0], mm[1], 256)
    c2 = host(ctx.histogram(x[n // 2:], mm[0], mm[1], 256, counts=c2))
    np.testing.assert_array_equal(c2, counts)
    # torch.histc bins by the same rule up to rounding of the quotient: totals per coarse region agree
    absmax = max(abs(mm[0]), abs(mm[1]))
    scale = float(np.float32(absmax) / np.float32(127.0))
    fused = ctx.read_metrics(ctx.fake_quantize_metrics(x, scale, 0))
    y = ctx.dequantize(ctx.quantize_per_tensor_i8(x, scale, 0), scale, 0)
    two = ctx.read_metrics(ctx.quantization_metrics(x, y))
    for k in fused:
        assert fused[k] == pytest.approx(two[k], rel=1e-6), k
    # uniform-quantizer noise model: mse ~ scale^2 / 12 for a fine grid, and SNR = 10 log10(var / mse)
    assert fused["mse"] == pytest.approx(scale * scale / 12.0, rel=0.02)
    assert fused["snr"] == pytest.approx(10 * math.log10(1.0 / fused["mse"]), abs=0.05)
    assert fused["max_error"] <= scale / 2 * (1 + 1e-6)
    # a tensor against itself
    same = ctx.read_metrics(ctx.quantization_metrics(x, x))
    assert same["mse"] == 0 and same["zero_error_percentage"] == 100 and math.isinf(same["psnr"])
    assert same["cosine_similarity"] == pytest.approx(1.0, abs=1e-6)


def test_more_than_two_to_the_32_elements(ctx, hipq, oracle):
    """(2^20 + 7) x 4097 elements, one seeded block repeated: counts, sums and images of the repeated tensor
    follow from the oracle's on the block.  What lies beyond element 2^32 (a NaN, an infinity, the range's ends,
    the largest error) is only seen with 64-bit indices, and every count must add up to all the elements."""
    period, reps = (1 << 20) + 7, 4097
    n = period * reps
    assert n > 1 << 32
    base = normal(21, (period,), 1.5)
    scale, zp = np.float32(0.04), 3
    x = dev(base).repeat(reps)
    # observe: range ends and two non-finite values past 2^32
    x[n - 3], x[(1 << 32) + 9] = 50.0, -60.0
    bad = x[(1 << 32) + 100:(1 << 32) + 102].clone()
    x[(1 << 32) + 100], x[(1 << 32) + 101] = float("nan"), float("inf")
    st = ctx.read_observe(ctx.observe(x))
    assert (st.min_val, st.max_val, st.nonfinite) == (-60.0, float("inf"), 2)  # NaN ignored, +inf is the maximum
    x[(1 << 32) + 100:(1 << 32) + 102] = bad
    st = ctx.read_observe(ctx.observe(x))
    assert (st.min_val, st.max_val, st.nonfinite) == (-60.0, 50.0, 0)
    # tensor statistics: range from beyond 2^32, moments = the block's plus the two planted values
    b64 = base.astype(np.float64)
    pos = [(n - 3) % period, ((1 << 32) + 9) % period]
    total = b64.sum() * reps - b64[pos].sum() + (50.0 - 60.0)
    total_sq = (b64 * b64).sum() * reps - (b64[pos] ** 2).sum() + (50.0 ** 2 + 60.0 ** 2)
    mean = total / n
    for one_pass in (False, True):
        ts = ctx.tensor_stats(x, one_pass=one_pass)
        assert (ts.min_val, ts.max_val) == (-60.0, 50.0)
        assert ts.mean == pytest.approx(mean, rel=1e-5, abs=1e-7)
        assert ts.variance == pytest.approx(total_sq / n - mean * mean, rel=1e-5)
    # adaptive ternary: the codes must follow the threshold the search chose, everywhere
    qa, params = ctx.quantize_ternary_adaptive(x)
    p = ctx.read_qparams(params)
    assert p.max_val == 60.0 and 0 < p.min_val <= 60.0
    want_codes = torch.where(x.abs() <= p.min_val, torch.zeros_like(x), torch.sign(x)).to(torch.int8)
    torch.cuda.synchronize()
    assert torch.equal(qa, want_codes)
    kept = x.abs() > p.min_val
    kept_sum = torch.where(kept, x.abs(), torch.zeros_like(x)).sum(dtype=torch.float64)
    assert p.scale == pytest.approx(float(kept_sum) / int(kept.sum()), rel=1e-6)
    del qa, want_codes, kept
    # histogram: block counts x repetitions; the two planted values move from their old bins to the end bins
    lo, hi, bins = -6.0, 6.0, 256
    block_counts = oracle.histogram_accumulate(base, lo, hi, bins).astype(np.int64)
    want = block_counts * reps
    for pos in ((n - 3) % period, ((1 << 32) + 9) % period):
        want[oracle.value_to_bin_index(base[pos], lo, hi, bins)] -= 1
    want[bins - 1] += 1
    want[0] += 1
    counts = host(ctx.histogram(x, lo, hi, bins))
    np.testing.assert_array_equal(counts, want)
    assert host(ctx.histogram(x, lo, hi, 1))[0] == n  # one counter beyond 2^32
    # fake quantize: the block's image repeated
    img_block = oracle.model_fake_quantize(base, scale, zp)
    img = ctx.fake_quantize(x, scale, zp, -128, 127, hipq.FORM_DIV | hipq.FAKE_INT_CAST)
    want_img = dev(img_block).repeat(reps)
    ends = oracle.model_fake_quantize(np.array([50.0, -60.0], np.float32), scale, zp)
    want_img[n - 3], want_img[(1 << 32) + 9] = float(ends[0]), float(ends[1])
    torch.cuda.synchronize()
    assert torch.equal(img, want_img)
    del want_img
    # metrics: means over the repeated tensor = the block's, plus the two saturated values' errors
    e = (np.array([50.0, -60.0], np.float64) - ends.astype(np.float64))
    blk = oracle.calculate_quantization_metrics_f64(base, img_block)
    for got in (ctx.read_metrics(ctx.quantization_metrics(x, img)),
                ctx.read_metrics(ctx.fake_quantize_metrics(x, scale, zp, -128, 127, hipq.FORM_DIV | hipq.FAKE_INT_CAST))):
        assert got["max_error"] == np.float32(np.abs(e).max())
        assert got["mse"] == pytest.approx(blk["mse"] + float((e * e).sum()) / n, rel=1e-5)
        assert got["mae"] == pytest.approx(blk["mae"] + float(np.abs(e).sum()) / n, rel=1e-5)
        assert got["zero_error_percentage"] == pytest.approx(blk["zero_error_percentage"], rel=1e-5, abs=1e-6)


@pytest.mark.parametrize("n", [1, 5, 63, 4096, 4099, (1 << 20) + 3, 1 << 24])
def test_tensor_stats_both_forms(ctx, oracle, n):
    """calculate_tensor_stats_simd (two passes, centered) and calculate_tensor_stats_cache_optimized (raw moments):
    range exact; mean, variance and standard deviation to 1e-6 of the oracle's f64 sums (the order of f64
    additions differs), the raw-moment variance to the cancellation it carries."""
    x = normal(500 + (n % 1000), n, 2.0) + np.float32(3.0)
    d = dev(x)
    st = ctx.tensor_stats(d)
    want = oracle.calculate_tensor_stats_simd(x)
    assert (st.min_val, st.max_val) == (want["min"], want["max"])
    assert st.mean == pytest.approx(want["mean"], rel=1e-6)
    assert st.variance == pytest.approx(want["variance"], rel=1e-6, abs=1e-12)
    assert st.std_dev == pytest.approx(want["std_dev"], rel=1e-6, abs=1e-12)
    one = ctx.tensor_stats(d, one_pass=True)
    mn, mx, mean, std = oracle.calculate_tensor_stats_cache_optimized(x)
    assert (one.min_val, one.max_val) == (mn, mx)
    assert one.mean == pytest.approx(mean, rel=1e-6)
    if n > 1:
        assert one.std_dev == pytest.approx(std, rel=2e-5)
        assert one.variance == pytest.approx(np.float32(std) ** 2, rel=4e-5)


def test_tensor_stats_known_answers_and_edges(ctx, hipq, golden):
    sv = golden["slice_variants"]
    c = sv["stats_simd"]
    st = ctx.tensor_stats(dev(np.array(c["x"], np.float32)))
    assert (st.min_val, st.max_val, st.mean) == (c["min"], c["max"], c["mean"])
    assert abs(st.std_dev - np.float32(np.sqrt(c["std_dev_f64_sqrt_of"]))) <= c["std_eps"]
    assert st.variance == 2.0
    c = sv["stats_cache_optimized"]
    st = ctx.tensor_stats(dev(np.array(c["x"], np.float32)), one_pass=True)
    assert (st.min_val, st.max_val) == (c["min"], c["max"]) and abs(st.mean - c["mean"]) < c["mean_eps"]
    assert st.std_dev == pytest.approx(np.sqrt(8.25), rel=1e-6)
    with pytest.raises(hipq.HipqError, match="Cannot calculate stats of empty tensor"):
        ctx.tensor_stats(torch.empty(0, device="cuda"))
    # NaN is ignored by the range (f32::min / max) and poisons the sums, as in the reference
    x = torch.tensor([1.0, float("nan"), 3.0], device="cuda")
    st = ctx.tensor_stats(x)
    assert (st.min_val, st.max_val) == (1.0, 3.0) and math.isnan(st.mean) and math.isnan(st.std_dev)
    # an unaligned view
    base = torch.arange(0, 1001, device="cuda", dtype=torch.float32)
    st = ctx.tensor_stats(base[1:])
    assert (st.min_val, st.max_val, st.mean) == (1.0, 1000.0, 500.5)
    assert st.variance == pytest.approx((1000 ** 2 - 1) / 12.0, rel=1e-6)


# ---- special schemes (int4, group-wise, binary, ternary) -----------------------------------------

def _view(shape, axis):
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return outer, shape[axis], inner


@pytest.mark.parametrize("shape,axis,group", [((24, 50, 6), 0, 4), ((24, 50, 6), 0, 5), ((24, 50, 6), 1, 10),
                                               ((24, 50, 6), 1, 7), ((24, 50, 6), 2, 4), ((64, 2048), 0, 1),
                                               ((64, 2048), 0, 8), ((3, 4096), 1, 128), ((7, 1000), 1, 32),
                                               ((5,), 0, 2)])
def test_group_wise_is_bit_exact(ctx, hipq, oracle, shape, axis, group):
    x = normal(sum(shape) + axis + group, shape, 1.7)
    outer, channels, inner = _view(shape, axis)
    for qmin, qmax in ((-128, 127), (-8, 7), (-63, 63)):
        q, scales, zps, status = ctx.quantize_per_group_auto(dev(x), outer, channels, inner, group,
                                                             hipq.PARAMS_ZERO_INCLUDED, qmin, qmax, hipq.FORM_DIV)
        want, ws, wz, _, _ = oracle.quantize_group_wise(x, axis, group, qmin, qmax)
        assert int(host(status)[0]) == 0
        np.testing.assert_array_equal(host(scales), ws)
        np.testing.assert_array_equal(host(zps), wz)
        np.testing.assert_array_equal(host(q).astype(np.float32), want)


def test_int4_per_tensor_and_per_channel_are_bit_exact(ctx, hipq, oracle, cal):
    for case in cal["special_schemes"]:
        if case["fn"] != "quantize_int4_per_tensor":
            continue
        x = np.float32(case["x"])
        q, scales, zps, _ = ctx.quantize_per_group_auto(dev(x), 1, 1, x.size, 1, hipq.PARAMS_ZERO_INCLUDED, -8, 7, hipq.FORM_DIV)
        want, s, z = oracle.quantize_int4_per_tensor(x)
        np.testing.assert_array_equal(host(q).astype(np.float32), want)
        assert host(scales)[0] == s and host(zps)[0] == z and case["zp_range"][0] <= z <= case["zp_range"][1]
    x = normal(13, (16, 33, 9), 0.8)
    for axis in range(3):
        outer, channels, inner = _view(x.shape, axis)
        q, scales, zps, _ = ctx.quantize_per_group_auto(dev(x), outer, channels, inner, 1, hipq.PARAMS_ZERO_INCLUDED, -8, 7,
                                                        hipq.FORM_DIV)
        want, ws, wz, _, _ = oracle.quantize_int4_per_channel(x, axis)
        np.testing.assert_array_equal(host(q).astype(np.float32), want)
        np.testing.assert_array_equal(host(scales), ws)
        np.testing.assert_array_equal(host(zps), wz)
    big = normal(14, 1 << 20, 2.0)
    q, scales, zps, _ = ctx.quantize_per_group_auto(dev(big), 1, 1, big.size, 1, hipq.PARAMS_ZERO_INCLUDED, -8, 7, hipq.FORM_DIV)
    want, s, z = oracle.quantize_int4_per_tensor(big)
    np.testing.assert_array_equal(host(q).astype(np.float32), want)
    assert host(scales)[0] == s and host(zps)[0] == z


def test_group_wise_argument_errors(ctx, hipq):
    x = dev(normal(1, (4, 8)))
    with pytest.raises(hipq.HipqError) as e:
        ctx.quantize_per_group_auto(x, 1, 4, 8, 0, hipq.PARAMS_ZERO_INCLUDED, -128, 127)
    assert "Group size must be greater than 0" in e.value.message
    with pytest.raises(hipq.HipqError):
        ctx.quantize_per_group_auto(x, 1, 4, 8, 2, hipq.PARAMS_ZERO_INCLUDED, -200, 127)
    with pytest.raises(hipq.HipqError):
        ctx.quantize_per_group_auto(x, 1, 4, 8, 2, 9, -128, 127)
    # a non-finite range is reported through the status word, not as garbage parameters
    bad = normal(2, (4, 8))
    bad[1, 3] = np.inf
    _, _, _, status = ctx.quantize_per_group_auto(dev(bad), 1, 4, 8, 2, hipq.PARAMS_ZERO_INCLUDED, -128, 127)
    assert int(host(status)[0]) == hipq.INVALID_ARGUMENT


@pytest.mark.parametrize("n", [1, 5, 63, 4096, 100003, 1 << 20])
def test_binary_and_ternary(ctx, hipq, oracle, n):
    x = normal(40 + n, n, 1.1)
    if n >= 63:
        x[::9] = 0.0            # zeros are +1 for the binary scheme and 0 for the ternary one
    q, params = ctx.quantize_binary(dev(x))
    want, s32, s64 = oracle.quantize_binary(x)
    p = ctx.read_qparams(params)
    np.testing.assert_array_equal(host(q).astype(np.float32), want)
    assert p.zero_point == 0 and p.status == 0
    assert p.scale == pytest.approx(s64, rel=1e-6) and p.scale == pytest.approx(float(s32), rel=1e-4)
    q, params = ctx.quantize_ternary(dev(x))
    want, s32, s64, thr = oracle.quantize_ternary(x)
    p = ctx.read_qparams(params)
    np.testing.assert_array_equal(host(q).astype(np.float32), want)
    assert p.min_val == thr and p.zero_point == 0
    assert p.scale == pytest.approx(s64, rel=1e-6) and p.scale == pytest.approx(float(s32), rel=1e-4)


@pytest.mark.parametrize("n", [1, 5, 63, 4096, 100003, 1 << 20])
def test_learned_threshold_binary_and_adaptive_ternary(ctx, hipq, oracle, n):
    """quantize_binary_learned_threshold (given and learned threshold) and quantize_ternary_adaptive: codes bit for
    bit and the threshold exactly against the oracle run with f64 sums (the order-free value of the reference's
    sequential f32 sums, which it must also agree with to their own rounding), scales to 1e-6 of the f64 mean."""
    x = normal(60 + n, n, 1.1)
    if n >= 63:
        x[::9] = 0.0
        x[1::11] = -0.0
    d = dev(x)
    for given in (0.4, -1.0, None):
        q, params = ctx.quantize_binary_learned_threshold(d, given)
        want, s32, s64, thr = oracle.quantize_binary_learned_threshold(x, given, f64_sums=True)
        p = ctx.read_qparams(params)
        assert p.min_val == thr and p.max_val == 0 and p.zero_point == 0 and p.status == 0
        np.testing.assert_array_equal(host(q).astype(np.float32), want)
        assert p.scale == pytest.approx(s64, rel=1e-6)
        _, s32_ref, _, thr_ref = oracle.quantize_binary_learned_threshold(x, given)  # the reference's f32 sums
        assert p.min_val == pytest.approx(float(thr_ref), rel=1e-4) and p.scale == pytest.approx(float(s32_ref), rel=1e-3)
    q, params = ctx.quantize_ternary_adaptive(d)
    want, s32, s64, thr, e32, e64 = oracle.quantize_ternary_adaptive(x, f64_sums=True)
    p = ctx.read_qparams(params)
    assert p.min_val == thr and p.max_val == np.abs(x).max() and p.zero_point == 0
    np.testing.assert_array_equal(host(q).astype(np.float32), want)
    assert p.scale == pytest.approx(s64, rel=1e-6)
    # the reference's own f32 sums pick the same threshold unless two candidates cost the same to f32 rounding
    order = np.sort(e64)
    if n == 1 or order[1] - order[0] > 1e-3 * order[0]:
        assert oracle.quantize_ternary_adaptive(x)[3] == thr


def test_learned_threshold_and_adaptive_golden_and_errors(ctx, hipq, cal):
    for case in cal["special_schemes"]:
        x = dev(np.float32(case["x"])) if "x" in case and case["fn"] in ("quantize_binary_learned_threshold",
                                                                          "quantize_ternary_adaptive") else None
        if case["fn"] == "quantize_binary_learned_threshold":
            q, params = ctx.quantize_binary_learned_threshold(x, case["threshold"])
            p = ctx.read_qparams(params)
            assert p.scale > 0 and p.zero_point == case["zp"] and p.min_val == np.float32(case["threshold_out"])
            np.testing.assert_array_equal(host(q), case["q"])
        elif case["fn"] == "quantize_ternary_adaptive":
            q, params = ctx.quantize_ternary_adaptive(x)
            p = ctx.read_qparams(params)
            assert p.scale > 0 and p.zero_point == case["zp"] and p.min_val > 0
            assert set(host(q).tolist()) <= set(case["values_in"])
            # by hand: every threshold from 0.3 to 2.7 costs 1.7, the first wins; +-0.5 keep their signs
            assert p.min_val == np.float32(3) * (np.float32(1) * np.float32(0.1)) and p.scale == 1.75
            np.testing.assert_array_equal(host(q), [-1, -1, 0, 1, 1])
    empty = torch.empty(0, device="cuda")
    with pytest.raises(hipq.HipqError, match="Cannot quantize empty tensor"):
        ctx.quantize_binary_learned_threshold(empty)
    with pytest.raises(hipq.HipqError, match="Cannot quantize empty tensor"):
        ctx.quantize_ternary_adaptive(empty)
    # unaligned views
    base = dev(normal(7, 4099, 1.0))
    for off in (1, 2, 3):
        v = base[off:]
        q, params = ctx.quantize_ternary_adaptive(v)
        q2, params2 = ctx.quantize_ternary_adaptive(v.clone())
        assert torch.equal(q, q2) and ctx.read_qparams(params).scale == ctx.read_qparams(params2).scale


def test_binary_ternary_golden_edges_and_errors(ctx, hipq, oracle, cal):
    for case in cal["special_schemes"]:
        if case["fn"] not in ("quantize_binary", "quantize_ternary"):
            continue
        x = np.float32(case["x"])
        fn = ctx.quantize_binary if case["fn"] == "quantize_binary" else ctx.quantize_ternary
        q, params = fn(dev(x))
        p = ctx.read_qparams(params)
        assert p.scale > 0 and p.zero_point == case["zp"] and set(host(q).tolist()) <= set(case["values_in"])
    zeros = torch.zeros(1000, device="cuda")
    q, params = ctx.quantize_binary(zeros)
    assert ctx.read_qparams(params).scale == 1.0 and (host(q) == 1).all()
    q, params = ctx.quantize_ternary(zeros)
    assert ctx.read_qparams(params).scale == 1.0 and (host(q) == 0).all()
    x = np.float32([10, 7, -7, 7.5, -10, float("nan")])
    np.testing.assert_array_equal(host(ctx.quantize_ternary(dev(x))[0]).astype(np.float32), oracle.quantize_ternary(x)[0])
    np.testing.assert_array_equal(host(ctx.quantize_binary(dev(x))[0]).astype(np.float32), oracle.quantize_binary(x)[0])
    empty = torch.empty(0, device="cuda")
    for fn in (ctx.quantize_binary, ctx.quantize_ternary):
        with pytest.raises(hipq.HipqError) as e:
            fn(empty)
        assert e.value.code == hipq.INVALID_ARGUMENT and "Cannot quantize empty tensor" in e.value.message
    # unaligned views
    base = normal(77, 10007)
    d = dev(base)
    for off in (1, 2, 3):
        np.testing.assert_array_equal(host(ctx.quantize_ternary(d[off:])[0]).astype(np.float32),
                                      oracle.quantize_ternary(base[off:])[0])
