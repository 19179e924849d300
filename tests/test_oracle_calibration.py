"""Pins the calibration / metrics part of the CPU oracle.

Three kinds of checks, none of which retypes the oracle's own formula:
  * the known answers the reference's unit tests assert (tests/golden/calibration_vectors.json);
  * closed forms: inputs built so every metric has a value one can write down by hand, and so that a
    swapped operand, a dropped factor or a wrong log base changes at least one of them;
  * brute force on small inputs with a differently organised computation (numpy's histogram
    counting, sorting, exact rational arithmetic).
"""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def cal():
    with open(os.path.join(ROOT, "tests", "golden", "calibration_vectors.json")) as f:
        return json.load(f)


def _floats(v):
    return np.array([float(t) for t in v], dtype=np.float32)


# ---- quality metrics -------------------------------------------------------------------------

def test_metrics_known_answers(oracle, cal):
    for case in cal["metrics"]:
        m = oracle.calculate_quantization_metrics(case["original"], case["quantized"], case["original_bits"],
                                                  case["quantized_bits"])
        a = case["assert"]
        assert m["compression_ratio"] == a["compression_ratio"], case["src"]
        if "mse_range" in a:
            assert a["mse_range"][0] < m["mse"] < a["mse_range"][1]
            assert a["mae_range"][0] < m["mae"] < a["mae_range"][1]
            assert m["psnr"] > 0 and m["snr"] > 0 and m["max_error"] >= 0
            assert 0 <= m["zero_error_percentage"] <= 100
            assert m["cosine_similarity"] > a["cosine_gt"]
        else:
            assert m["mse"] == a["mse"] and m["mae"] == a["mae"] and m["max_error"] == a["max_error"]
            assert m["zero_error_percentage"] == a["zero_error_percentage"]
            assert abs(m["cosine_similarity"] - a["cosine_within_1e-6_of"]) < 1e-6
            assert math.isinf(m["psnr"]) and m["psnr"] > 0 and math.isinf(m["snr"]) and m["snr"] > 0


def test_metrics_empty_is_default(oracle):
    m = oracle.calculate_quantization_metrics([], [])
    assert (m["mse"], m["psnr"], m["snr"], m["mae"], m["max_error"]) == (0, 0, 0, 0, 0)
    assert m["zero_error_percentage"] == 100 and m["cosine_similarity"] == 1 and m["compression_ratio"] == 1


def test_metrics_closed_form_constant_offset(oracle):
    # original = 4, quantized = 4.5 everywhere: every quantity is a hand value.
    n = 64
    m = oracle.calculate_quantization_metrics(np.full(n, 4.0), np.full(n, 4.5), 32, 4)
    assert m["mse"] == 0.25 and m["mae"] == 0.5 and m["max_error"] == 0.5
    assert m["zero_error_percentage"] == 0
    assert m["psnr"] == pytest.approx(20 * math.log10(4.0 / 0.5), rel=1e-6)        # 18.06 dB
    assert m["snr"] == pytest.approx(10 * math.log10(16.0 / 0.25), rel=1e-6)       # 18.06 dB as well
    assert m["cosine_similarity"] == pytest.approx(1.0, abs=1e-6)
    assert m["compression_ratio"] == 8.0


def test_metrics_closed_form_discriminates_operands(oracle):
    # original = [2, 0], quantized = [0, 4]: peak signal comes from the ORIGINAL (2, not 4), signal power from
    # the original (2, not 8), errors are symmetric, vectors are orthogonal.
    m = oracle.calculate_quantization_metrics([2.0, 0.0], [0.0, 4.0])
    assert m["mse"] == 10.0 and m["mae"] == 3.0 and m["max_error"] == 4.0
    assert m["psnr"] == pytest.approx(20 * math.log10(2.0 / math.sqrt(10.0)), rel=1e-6)   # -3.979 dB
    assert m["snr"] == pytest.approx(10 * math.log10(2.0 / 10.0), rel=1e-6)               # -6.990 dB
    assert m["cosine_similarity"] == 0.0
    # one exact match out of four
    m = oracle.calculate_quantization_metrics([1.0, 2.0, 3.0, 4.0], [1.0, 2.5, 2.0, 6.0])
    assert m["zero_error_percentage"] == 25.0 and m["max_error"] == 2.0
    assert m["mae"] == pytest.approx((0.5 + 1 + 2) / 4) and m["mse"] == pytest.approx((0.25 + 1 + 4) / 4)
    # zero original vector: cosine falls to 0, SNR and PSNR use signal 0
    m = oracle.calculate_quantization_metrics([0.0, 0.0], [1.0, 1.0])
    assert m["cosine_similarity"] == 0.0 and math.isinf(m["snr"]) and m["snr"] > 0
    assert math.isinf(m["psnr"]) and m["psnr"] < 0     # 20*log10(0 / 1)


def test_metrics_zero_error_threshold(oracle):
    # |a-b| < 1e-7 counts as zero error: 5e-8 does, 2e-7 does not.
    a = np.zeros(4, dtype=np.float32)
    b = np.array([0.0, 5e-8, 2e-7, -5e-8], dtype=np.float32)
    assert oracle.calculate_quantization_metrics(a, b)["zero_error_percentage"] == 75.0


def test_metrics_f32_and_f64_sums_agree_on_short_inputs(oracle):
    rng = np.random.default_rng(5)
    a = rng.standard_normal(2000).astype(np.float32)
    b = (a + rng.standard_normal(2000).astype(np.float32) * 0.01).astype(np.float32)
    m32 = oracle.calculate_quantization_metrics(a, b)
    m64 = oracle.calculate_quantization_metrics_f64(a, b)
    for k in m32:
        assert float(m32[k]) == pytest.approx(m64[k], rel=2e-5, abs=1e-9), k
    # exact rational arithmetic on the f32 inputs for the sums the f64 variant carries
    d = [Fraction(float(np.float32(x) - np.float32(y))) for x, y in zip(a, b)]
    mse = sum(t * t for t in d) / len(d)
    assert m64["mse"] == pytest.approx(float(mse), rel=1e-6)
    assert m64["mae"] == pytest.approx(float(sum(abs(t) for t in d) / len(d)), rel=1e-9)


# ---- observers -------------------------------------------------------------------------------

def test_observer_minmax_known_answers(oracle, cal):
    for case in cal["observer_minmax"]:
        ob = oracle.Observer(oracle.OBS_MINMAX)
        for batch, want in zip(case["batches"], case["min_max_after_each"]):
            ob.update(batch)
            assert ob.get_min_max() == tuple(np.float32(w) for w in want), case["src"]


def test_observer_histogram_known_answers(oracle, cal):
    for case in cal["observer_histogram"]:
        ob = oracle.Observer(oracle.OBS_HISTOGRAM, num_bins=case["num_bins"])
        for batch in case["batches"]:
            ob.update(batch)
        assert int(ob.histogram().sum()) == case["total_samples"] and ob.num_bins() == case["stat_num_bins"]


def test_observer_percentile_known_answers(oracle, cal):
    for case in cal["observer_percentile"]:
        ob = oracle.Observer(oracle.OBS_PERCENTILE, percentile=case["percentile"])
        ob.update(np.arange(case["arange"], dtype=np.float32))
        assert len(ob.values()) == case["total_values"]


def test_observer_qparams_errors_reset_known_answers(oracle, cal):
    for case in cal["observer_qparams"]:
        ob = oracle.Observer(oracle.OBS_MINMAX)
        for batch in case["batches"]:
            ob.update(batch)
        if case.get("error"):
            with pytest.raises(oracle.OracleError):
                ob.calculate_qparams(oracle.DTYPE_OTHER)
        else:
            s, z = ob.calculate_qparams(oracle.DTYPE_I8)
            assert s > 0 and case["zp_range"][0] <= z <= case["zp_range"][1]
    for case in cal["observer_errors"]:
        ob = oracle.Observer(oracle.OBS_MINMAX)
        if case["error"]:
            with pytest.raises(oracle.OracleError):
                ob.update(_floats(case["batch"]))
        else:
            ob.update(_floats(case["batch"]))
            assert ob.num_batches() == case["num_batches"]
    for case in cal["observer_reset"]:
        ob = oracle.Observer(oracle.OBS_MINMAX)
        ob.update(case["batch"])
        assert ob.num_batches() == case["num_batches_before"]
        ob.reset()
        assert ob.num_batches() == case["num_batches_after"]
        mn, mx = ob.get_min_max()
        assert mn == np.float32(float(case["min_after"])) and mx == np.float32(float(case["max_after"]))


def test_observer_qparams_closed_form(oracle):
    # MinMax over [-2, 2] with I8: range widened to include 0 (already does), scale = 4/255,
    # zero point = round(-128 + 2/scale) = round(-0.5) = -1 (half away from zero).
    ob = oracle.Observer(oracle.OBS_MINMAX)
    ob.update([-2.0, -1.0, 0.0, 1.0, 2.0])
    s, z = ob.calculate_qparams(oracle.DTYPE_I8)
    assert s == np.float32(4.0) / np.float32(255.0) and z in (-1, 0)
    exact = -128 + Fraction(2) / Fraction(float(s))
    assert z == (math.floor(exact + Fraction(1, 2)) if exact >= 0 else -math.floor(-exact + Fraction(1, 2)))
    # all-positive data: the range is extended down to 0, so zero_point = qmin exactly.
    ob = oracle.Observer(oracle.OBS_MINMAX)
    ob.update([1.0, 3.0])
    s, z = ob.calculate_qparams(oracle.DTYPE_U8)
    assert s == np.float32(3.0) / np.float32(255.0) and z == 0
    # constant zero data: scale falls back to 1
    ob = oracle.Observer(oracle.OBS_MINMAX)
    ob.update([0.0, 0.0])
    assert ob.calculate_qparams(oracle.DTYPE_I8) == (np.float32(1.0), -128)


def test_moving_average_starts_from_zero(oracle):
    # The first batch is averaged against 0, not adopted: avg = 0.01 * batch.
    ob = oracle.Observer(oracle.OBS_MOVING_AVERAGE)
    ob.update([-4.0, 10.0])
    amin, amax = ob.get_avg()
    assert amin == np.float32(0.01) * np.float32(-4.0) and amax == np.float32(0.01) * np.float32(10.0)
    ob.update([-8.0, 20.0])
    amin2, amax2 = ob.get_avg()
    assert amax2 == np.float32(0.01) * np.float32(20.0) + (np.float32(1.0) - np.float32(0.01)) * amax
    assert ob.get_min_max() == (np.float32(-8.0), np.float32(20.0))
    # calculate_qparams uses the global range, not the averages
    s, _ = ob.calculate_qparams(oracle.DTYPE_I8)
    assert s == np.float32(28.0) / np.float32(255.0)


def test_value_to_bin_index_brute_force(oracle):
    # Edges of [0, 10] with 10 bins: value k lands in bin k, the top edge in the last bin,
    # values outside clamp, non-finite and degenerate ranges go to bin 0.
    for k in range(10):
        assert oracle.value_to_bin_index(float(k), 0.0, 10.0, 10) == k
        assert oracle.value_to_bin_index(k + 0.999, 0.0, 10.0, 10) == k
    assert oracle.value_to_bin_index(10.0, 0.0, 10.0, 10) == 9
    assert oracle.value_to_bin_index(-3.0, 0.0, 10.0, 10) == 0
    assert oracle.value_to_bin_index(1e9, 0.0, 10.0, 10) == 9
    assert oracle.value_to_bin_index(float("nan"), 0.0, 10.0, 10) == 0
    assert oracle.value_to_bin_index(float("inf"), 0.0, 10.0, 10) == 0
    assert oracle.value_to_bin_index(5.0, 3.0, 3.0, 10) == 0 and oracle.value_to_bin_index(5.0, 4.0, 3.0, 10) == 0


def test_histogram_against_numpy_counting(oracle):
    # Values on an exact dyadic grid: (v - lo) / (hi - lo) * bins is exact in f32, so numpy's
    # histogram (a different algorithm: searchsorted on bin edges) must agree bin for bin.
    rng = np.random.default_rng(11)
    x = (rng.integers(0, 1024, size=20000) / np.float32(64.0)).astype(np.float32)    # [0, 16)
    lo, hi, bins = 0.0, 16.0, 32
    want, _ = np.histogram(x, bins=bins, range=(lo, hi))
    got = oracle.histogram_accumulate(x, lo, hi, bins)
    np.testing.assert_array_equal(got, want.astype(np.uint64))
    # accumulation across calls
    got2 = oracle.histogram_accumulate(x[:100], lo, hi, bins, counts=got)
    assert int(got2.sum()) == 20100


def test_histogram_observer_keeps_old_bins_when_range_grows(oracle):
    # Second batch widens the range; counts of the first batch stay where they were put.
    ob = oracle.Observer(oracle.OBS_HISTOGRAM, num_bins=4)
    ob.update([0.0, 1.0, 2.0, 3.0, 4.0])            # range [0,4]: bins 0,1,2,3,3
    np.testing.assert_array_equal(ob.histogram(), [1, 1, 1, 2])
    ob.update([8.0])                                  # range [0,8]: 8 -> last bin
    np.testing.assert_array_equal(ob.histogram(), [1, 1, 1, 3])
    assert ob.get_hist_range() == (np.float32(0.0), np.float32(8.0))


def test_histogram_range_trims_outliers(oracle):
    # 2000 samples in [0,1) plus one outlier at 100 with 100 bins over [0,100]: 0.5 % of 2001 = 10 samples may
    # be cut from each end, so the single outlier is dropped and the range collapses onto the first bin...
    x = np.concatenate([np.linspace(0, 0.99, 2000, dtype=np.float32), np.float32([100.0])])
    ob = oracle.Observer(oracle.OBS_HISTOGRAM, num_bins=100)
    ob.update(x)
    h = ob.histogram()
    assert h[0] == 2000 and h[99] == 1
    # ...where start_bin == end_bin == 0 makes the reference fall back to the global range.
    assert ob.histogram_range() == (np.float32(0.0), np.float32(100.0))
    # A spread-out case: uniform grid over 256 bins, 0.1 % of 25600 = 25 samples trimmed per side,
    # each bin holds 100, so nothing is trimmed and the range is the full one.
    y = np.repeat(np.arange(256, dtype=np.float32), 100)
    ob = oracle.Observer(oracle.OBS_HISTOGRAM)
    ob.update(y)
    np.testing.assert_array_equal(ob.histogram()[:255], np.full(255, 100))
    assert ob.histogram()[255] == 100
    assert ob.histogram_range() == (np.float32(0.0), np.float32(255.0))
    # Thin tails: one sample in each of the outer 20 bins per side, 5000 in each middle bin.
    z = np.concatenate([np.arange(0, 20), np.repeat(np.arange(20, 236), 5000), np.arange(236, 256)]).astype(np.float32)
    ob = oracle.Observer(oracle.OBS_HISTOGRAM)
    ob.update(z)
    mn, mx = ob.histogram_range()
    # total = 1,080,040 -> threshold 1080 samples: the 20 single-sample bins (20 < 1080) are skipped, then bin 20
    # (cumulative 5020 > 1080) starts the range; symmetric at the top.
    width = np.float32(255.0) / np.float32(256.0)
    assert mn == np.float32(0.0) + np.float32(20.0) * width
    assert mx == np.float32(0.0) + np.float32(236.0) * width


def test_percentile_range_brute_force(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(5000).astype(np.float32)
    ob = oracle.Observer(oracle.OBS_PERCENTILE, percentile=99.0)
    ob.update(x)
    lo, hi = ob.percentile_range()
    s = np.sort(x)
    # 1 % of 5000 = index 50 (the f32 product may land one below), 99 % = index 4950
    assert lo in (s[49], s[50]) and hi in (s[4949], s[4950])
    assert np.sum(x < lo) in (49, 50) and np.sum(x > hi) in (49, 50)


def test_percentile_sampling_above_100k(oracle):
    ob = oracle.Observer(oracle.OBS_PERCENTILE)
    x = np.arange(400000, dtype=np.float32)
    ob.update(x)
    v = ob.values()
    # sample rate 0.25: every 4th element is kept (i * 0.25 mod 1 < 0.25 exactly when i % 4 == 0)
    np.testing.assert_array_equal(v, x[::4])
    assert ob.get_min_max() == (np.float32(0.0), np.float32(399999.0))


# ---- model-level quantizer ---------------------------------------------------------------------

def test_model_params_known_answers(oracle, cal):
    for case in cal["model_params"]:
        s, z, amin, amax = oracle.model_calculate_quantization_params(case["min"], case["max"], case["qmin"], case["qmax"])
        assert s > 0 and case["zp_range"][0] <= z <= case["zp_range"][1]
        assert (amin, amax) == (np.float32(case["min"]), np.float32(case["max"]))


def test_model_params_closed_form(oracle):
    s, z, _, _ = oracle.model_calculate_quantization_params(0.0, 255.0, 0, 255)
    assert s == 1.0 and z == 0
    s, z, _, _ = oracle.model_calculate_quantization_params(-1.0, 1.0, -128, 127)
    assert s == np.float32(2.0) / np.float32(255.0) and z in (-1, 0)     # -128 + 127.5 = -0.5 up to rounding of 1/s
    # degenerate range is widened by 1e-4 on both sides
    s, z, amin, amax = oracle.model_calculate_quantization_params(3.0, 3.0, -128, 127)
    assert amin == np.float32(3.0) - np.float32(1e-4) and amax == np.float32(3.0) + np.float32(1e-4)
    assert s == (amax - amin) / np.float32(255.0) and z == -128          # -128 - 3/s clamps at qmin


def test_model_fake_quantize_closed_form(oracle):
    # scale 0.5, zp 3: 1.2 -> round(2.4)+3 = 5 -> (5-3)*0.5 = 1.0 ; 1.25 -> round(2.5)=3 -> 1.5 (half away)
    y = oracle.model_fake_quantize([1.2, 1.25, -1.25, 1000.0, -1000.0], 0.5, 3)
    np.testing.assert_array_equal(y, np.float32([1.0, 1.5, -1.5, (127 - 3) * 0.5, (-128 - 3) * 0.5]))
    # NaN goes through `as i32` -> 0 -> (0 - zp) * scale
    assert oracle.model_fake_quantize([float("nan")], 0.5, 3)[0] == np.float32(-1.5)
    # identity on the grid, idempotent
    x = (np.arange(-128, 128) * np.float32(0.25)).astype(np.float32)
    y = oracle.model_fake_quantize(x, 0.25, 0)
    np.testing.assert_array_equal(y, x)
    np.testing.assert_array_equal(oracle.model_fake_quantize(y, 0.25, 0), y)
    assert oracle.model_mse_error(x, x + np.float32(0.5)) == 0.25


# ---- special schemes (specialized.rs) ------------------------------------------------------------

def test_special_scheme_known_answers(oracle, cal):
    for case in cal["special_schemes"]:
        fn = case["fn"]
        if fn == "quantize_int4_per_tensor":
            q, s, z = oracle.quantize_int4_per_tensor(case["x"])
            assert s > 0 and case["zp_range"][0] <= z <= case["zp_range"][1]
            assert q.min() >= case["value_range"][0] and q.max() <= case["value_range"][1]
        elif fn == "quantize_binary":
            q, s, _ = oracle.quantize_binary(case["x"])
            assert s > 0 and set(q.tolist()) <= set(case["values_in"])
        elif fn == "quantize_ternary":
            q, s, _, _ = oracle.quantize_ternary(case["x"])
            assert s > 0 and set(q.tolist()) <= set(case["values_in"])
        elif fn == "quantize_group_wise":
            x = np.float32(case["x"])
            q, _, _, s, _ = oracle.quantize_group_wise(x, case["axis"], case["group_size"])
            assert s > 0 and q.shape == x.shape
        elif fn == "quantize_binary_learned_threshold":
            q, s, _, thr = oracle.quantize_binary_learned_threshold(case["x"], case["threshold"])
            assert s > 0 and thr == np.float32(case["threshold_out"])
            np.testing.assert_array_equal(q, case["q"])
        elif fn == "quantize_ternary_adaptive":
            q, s, _, thr, _, _ = oracle.quantize_ternary_adaptive(case["x"])
            assert s > 0 and thr > 0 and set(q.tolist()) <= set(case["values_in"]) and q.size == len(case["x"])
        else:
            with pytest.raises(oracle.OracleError):
                oracle.quantize_binary([])
            with pytest.raises(oracle.OracleError):
                oracle.quantize_ternary([])
            with pytest.raises(oracle.OracleError):
                oracle.quantize_group_wise(np.float32([1, 2, 3]), 5, 2)
            with pytest.raises(oracle.OracleError):
                oracle.quantize_group_wise(np.float32([1, 2, 3]), 0, 0)


def test_int4_closed_form(oracle):
    # [0, 15]: scale 1, zero point -8, value k -> k - 8.
    q, s, z = oracle.quantize_int4_per_tensor(np.arange(16, dtype=np.float32))
    assert (s, z) == (1.0, -8)
    np.testing.assert_array_equal(q, np.arange(16) - 8)
    # all-positive data away from 0: the range still starts at 0 ([0, 30] -> scale 2)
    q, s, z = oracle.quantize_int4_per_tensor(np.float32([10, 20, 30]))
    assert (s, z) == (2.0, -8)
    np.testing.assert_array_equal(q, [-3, 2, 7])
    # symmetric data [-7.5, 7.5]: scale 1, zero point round(-8 + 7.5) = round(-0.5) = -1 (half away)
    q, s, z = oracle.quantize_int4_per_tensor(np.float32([-7.5, 0.0, 7.5]))
    assert (s, z) == (1.0, -1)
    np.testing.assert_array_equal(q, [-8, -1, 7])       # round(-7.5) = -8 -> -9 clamps to -8; round(7.5) = 8 -> 7
    # all zeros: scale falls back to 1
    q, s, z = oracle.quantize_int4_per_tensor(np.zeros(4, np.float32))
    assert (s, z) == (1.0, -8) and (q == -8).all()


def test_int4_per_channel_equals_per_tensor_on_each_slice(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((3, 4, 5)).astype(np.float32)
    for axis in range(3):
        q, scales, zps, avg_s, avg_z = oracle.quantize_int4_per_channel(x, axis)
        for c in range(x.shape[axis]):
            sl = np.take(x, c, axis=axis)
            qc, sc, zc = oracle.quantize_int4_per_tensor(sl)
            np.testing.assert_array_equal(np.take(q, c, axis=axis), qc)
            assert (scales[c], zps[c]) == (sc, zc)
        seq = np.float32(0)
        for s in scales:
            seq = np.float32(seq + s)
        assert avg_s == np.float32(seq / np.float32(len(scales)))
        m = float(zps.sum()) / len(zps)
        assert avg_z == int(math.copysign(math.floor(abs(m) + 0.5), m))


def test_binary_and_ternary_closed_form(oracle):
    q, s, s64 = oracle.quantize_binary(np.float32([-2, -1, 0, 1, 2]))
    np.testing.assert_array_equal(q, [-1, -1, 1, 1, 1])            # 0 counts as positive
    assert s == np.float32(6.0 / 5.0) and s64 == pytest.approx(1.2)
    q, s, _ = oracle.quantize_binary(np.zeros(3, np.float32))
    assert s == 1.0 and (q == 1).all()
    assert oracle.quantize_binary(np.float32([float("nan")]))[0][0] == -1     # NaN >= 0 is false
    # ternary: threshold 0.7 * 3 = 2.1; only +-3 survive, scale = mean(3, 3) = 3
    q, s, s64, thr = oracle.quantize_ternary(np.float32([-3, -1, 0.1, 1, 3]))
    np.testing.assert_array_equal(q, [-1, 0, 0, 0, 1])
    assert s == 3.0 and thr == np.float32(3.0) * np.float32(0.7)
    # values exactly at the threshold become 0 (<=): max 10 -> threshold 7 exactly representable
    q, s, _, thr = oracle.quantize_ternary(np.float32([10, 7, -7, 7.5, -10]))
    assert thr == np.float32(10) * np.float32(0.7)
    want = [1, 1 if np.float32(7) > thr else 0, -1 if np.float32(7) > thr else 0, 1, -1]
    np.testing.assert_array_equal(q, want)
    # all zeros: nothing above the threshold, scale 1
    q, s, _, _ = oracle.quantize_ternary(np.zeros(5, np.float32))
    assert s == 1.0 and (q == 0).all()


def test_learned_threshold_and_adaptive_ternary_closed_form(oracle):
    # learned threshold = mean |x| = (2 + 0.1 + 0.1 + 0.5 + 2) / 5 = 0.94: only +-2 keep a sign, scale 2
    x = np.float32([-2, -0.1, 0.1, 0.5, 2])
    q, s, s64, thr = oracle.quantize_binary_learned_threshold(x)
    assert thr == pytest.approx(0.94, rel=1e-6) and s == 2.0 and s64 == 2.0
    np.testing.assert_array_equal(q, [-1, 0, 0, 0, 1])
    # given threshold 0.3: scale = (2 + 0.5 + 2) / 3; a value equal to the threshold becomes 0
    q, s, _, thr = oracle.quantize_binary_learned_threshold(x, 0.3)
    assert s == np.float32(4.5) / np.float32(3) and thr == np.float32(0.3)
    q, _, _, _ = oracle.quantize_binary_learned_threshold(np.float32([0.5, -0.5, 0.75]), 0.5)
    np.testing.assert_array_equal(q, [0, 0, 1])
    # a negative threshold keeps every element, and zero (of either sign) then counts as positive: x >= 0
    q, s, _, _ = oracle.quantize_binary_learned_threshold(np.float32([0.0, -0.0, -1.0]), -1.0)
    np.testing.assert_array_equal(q, [1, 1, -1])
    assert s == np.float32(1.0) / np.float32(3)
    # nothing above the threshold: scale 1
    q, s, _, _ = oracle.quantize_binary_learned_threshold(np.float32([0.1, -0.2]), 5.0)
    assert s == 1.0 and (q == 0).all()
    # adaptive, by hand for [-3, -0.5, 0, 0.5, 3]: thresholds 0.3 .. 2.7 all cost (4 + .25 + 0 + .25 + 4) / 5 = 1.7
    # (0.5 costs 0.25 kept or dropped), threshold 3.0 costs 18.5 / 5; the first minimum wins: 3 * 0.1
    q, s, _, thr, e32, e64 = oracle.quantize_ternary_adaptive(np.float32([-3, -0.5, 0, 0.5, 3]))
    np.testing.assert_allclose(e32, [1.7] * 9 + [3.7], rtol=1e-6)
    np.testing.assert_allclose(e64, [1.7] * 9 + [3.7], rtol=1e-12)
    assert thr == np.float32(3) * (np.float32(1) * np.float32(0.1))
    np.testing.assert_array_equal(q, [-1, -1, 0, 1, 1])
    assert s == np.float32(7.0) / np.float32(4)
    # values near 1 with small noise: a high threshold that zeroes the noise and keeps the ones wins
    x = np.float32([1.0, -1.0, 0.05, -0.05, 1.0, 0.02])
    q, s, _, thr, e32, _ = oracle.quantize_ternary_adaptive(x)
    np.testing.assert_array_equal(q, [1, -1, 0, 0, 1, 0])
    assert thr == np.float32(1) * (np.float32(1) * np.float32(0.1)) and s == 1.0
    assert int(np.argmin(e32)) == 0 and e32[9] > e32[0]            # threshold 1.0 drops the ones as well
    # zero (and -0.0) is never given a sign by the adaptive form (x > 0), whatever the threshold
    q, _, _, _, _, _ = oracle.quantize_ternary_adaptive(np.float32([0.0, -0.0, 2.0]))
    np.testing.assert_array_equal(q[:2], [0, 0])
    # brute force of the search in float64 on random data: same winner wherever the margin is clear
    rng = np.random.default_rng(4)
    x = (rng.standard_normal(2000) * 1.3).astype(np.float32)
    q, s, s64, thr, e32, e64 = oracle.quantize_ternary_adaptive(x)
    mx = np.abs(x).max()
    errs = []
    for i in range(1, 11):
        t = mx * (np.float32(i) * np.float32(0.1))
        code = np.where(np.abs(x) <= t, 0.0, np.sign(x)).astype(np.float64)
        errs.append(((x.astype(np.float64) - code) ** 2).mean())
    np.testing.assert_allclose(e64, errs, rtol=1e-6)
    np.testing.assert_allclose(e32, errs, rtol=1e-4)
    best = int(np.argmin(errs))
    assert thr == mx * (np.float32(best + 1) * np.float32(0.1))
    keep = np.abs(x) > thr
    assert s64 == pytest.approx(np.abs(x[keep]).astype(np.float64).mean(), rel=1e-12)
    np.testing.assert_array_equal(q, np.where(keep, np.sign(x), 0.0))
    for fn in (oracle.quantize_binary_learned_threshold, oracle.quantize_ternary_adaptive):
        with pytest.raises(oracle.OracleError):
            fn([])


def test_group_wise_equals_grouped_slices(oracle):
    # Each group is quantized with the zero-including rule over all its members, whatever the axis.
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((4, 7, 3)) * 2).astype(np.float32)
    for axis, gs in ((0, 2), (1, 3), (1, 7), (2, 2), (1, 100)):
        q, scales, zps, avg_s, avg_z = oracle.quantize_group_wise(x, axis, gs)
        groups = -(-x.shape[axis] // gs)
        assert len(scales) == groups
        for g in range(groups):
            idx = [slice(None)] * 3
            idx[axis] = slice(g * gs, min((g + 1) * gs, x.shape[axis]))
            sl = x[tuple(idx)]
            mn, mx = min(float(sl.min()), 0.0), max(float(sl.max()), 0.0)
            s = np.float32(np.float32(mx) - np.float32(mn)) / np.float32(255.0)
            assert scales[g] == s
            # the zero point follows from the scale by exact rational arithmetic
            exact = Fraction(-128) - Fraction(mn) / Fraction(float(s))
            lo, hi = math.floor(exact), math.ceil(exact)
            assert zps[g] in (max(-128, min(127, lo)), max(-128, min(127, hi)))
            want = np.clip(np.round(sl.astype(np.float64) / float(s)) + zps[g], -128, 127)
            got = q[tuple(idx)]
            assert np.abs(got - want).max() <= 1          # float64 rounding may differ on near-ties only
            assert (got != want).mean() < 0.02
    # group size 1 over the last axis with int4 range equals quantize_int4_per_channel
    q4, s4, z4, _, _ = oracle.quantize_int4_per_channel(x, 2)
    qg, sg, zg, _, _ = oracle.quantize_group_wise(x, 2, 1, -8, 7)
    np.testing.assert_array_equal(qg, q4)
    np.testing.assert_array_equal(sg, s4)
    np.testing.assert_array_equal(zg, z4)


def test_fake_quantize_known_answers(oracle, cal):
    """What the reference's own tests assert for fake_quantize.rs (ranges and lengths)."""
    for case in cal["fake_quantize"]:
        x = np.array(case["x"], np.float32)
        want = case["assert"]
        if case["fn"] == "fake_quantize_auto":
            y, scale, zp = oracle.fake_quantize_auto(x, oracle.DTYPE_I8, 0)
            assert len(y) == want["len"] and scale > 0 and -128 <= zp <= 127
            assert all(want["range"][0] <= v <= want["range"][1] for v in y)
        else:
            y = oracle.fake_quantize_per_tensor_affine(x, case["scale"], case.get("zero_point", 0))
            assert len(y) == len(x)
            if want.get("abs_error_le_scale"):
                assert np.all(np.abs(y - x) <= np.float32(case["scale"]))


def test_fake_quantize_closed_form(oracle):
    """Hand values: a dropped zero point, a clamp in the wrong order, round-half-even or the multiply form each
    change one of them."""
    # scale 0.5, zp 3: q = round(x / 0.5) + 3 clamped to [-128, 127]; y = 0.5 * (q - 3)
    x = np.array([0.25, -0.25, 0.75, 1e9, -1e9, np.nan, np.inf, -np.inf, 0.0], np.float32)
    want = np.array([0.5, -0.5, 1.0, 62.0, -65.5, -65.5, 62.0, -65.5, 0.0], np.float32)  # ties away; NaN -> qmin
    np.testing.assert_array_equal(oracle.fake_quantize_per_tensor_affine(x, 0.5, 3), want)
    # uint8 range, zp 10: negative inputs saturate at (0 - 10) * scale
    y = oracle.fake_quantize_per_tensor_affine(np.array([-100.0, 3.0, 1000.0], np.float32), 2.0, 10, 0, 255)
    np.testing.assert_array_equal(y, np.array([-20.0, 4.0, 490.0], np.float32))  # 3/2 = 1.5 -> 2 -> (12 - 10) * 2
    # division, not multiplication by the reciprocal: 3 * (1/0.3f) rounds differently from 3 / 0.3f in f32 for some x;
    # scan for such an x and check it went through the division
    s = np.float32(0.3)
    xs = (np.arange(1, 20001, dtype=np.float32) * np.float32(0.05)).astype(np.float32)
    div = np.round(xs / s)  # not used for ties here: pick non-tie disagreements
    mul = np.round(xs * (np.float32(1.0) / s))
    idx = np.nonzero((div != mul) & (np.abs(xs / s - np.trunc(xs / s)) != 0.5))[0]
    assert idx.size > 0
    pick = xs[idx[:8]]
    got = oracle.fake_quantize_per_tensor_affine(pick, float(s), 0, -(2 ** 20), 2 ** 20)
    np.testing.assert_array_equal(got, s * div[idx[:8]].astype(np.float32))


def test_fake_quantize_auto_closed_form(oracle):
    # [-2, 2] -> I8 affine: scale 4/255; zp = round(-128 + 2/scale) = round(-0.5) = -1 (half away from zero)
    y, scale, zp = oracle.fake_quantize_auto(np.array([-2, -1, 0, 1, 2], np.float32), oracle.DTYPE_I8, 0)
    assert scale == np.float32(4.0) / np.float32(255.0) and zp == -1
    # the range always includes 0: all-positive data keeps min = 0 -> zp = qmin
    y, scale, zp = oracle.fake_quantize_auto(np.array([1.0, 3.0], np.float32), oracle.DTYPE_U8, 0)
    assert scale == np.float32(3.0) / np.float32(255.0) and zp == 0
    np.testing.assert_array_equal(y, oracle.fake_quantize_per_tensor_affine(np.array([1.0, 3.0], np.float32), scale, 0, 0, 255))
    # constant zero: scale 0 becomes 1
    y, scale, zp = oracle.fake_quantize_auto(np.zeros(5, np.float32), oracle.DTYPE_I8, 0)
    assert scale == 1.0 and np.all(y == 0)
    # symmetric: same scale formula (not absmax / 127), zero point 0
    y, scale, zp = oracle.fake_quantize_auto(np.array([-1.0, 3.0], np.float32), oracle.DTYPE_I8, 1)
    assert scale == np.float32(4.0) / np.float32(255.0) and zp == 0
    # dtypes and schemes the reference rejects
    for dtype, scheme in ((5, 0), (oracle.DTYPE_I8, 2)):
        with pytest.raises(Exception):
            oracle.fake_quantize_auto(np.ones(3, np.float32), dtype, scheme)
