"""Pins the CPU oracle against the known-answer vectors the reference's own tests hold."""
import numpy as np
import pytest

DT = {"I8": 0, "U8": 1, "I16": 2, "I32": 3}


def test_quantize_known_answers(oracle, golden):
    for case in golden["quantize_per_tensor"]:
        x = np.array(case["x"], dtype=np.float32)
        want = np.array(case["q"], dtype=np.float32)[: x.size]
        # both branches of quantize_per_tensor_affine, and the i8 forms
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine(x, case["scale"], case["zp"]), want, case["src"])
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine_simd(x, case["scale"], case["zp"]), want, case["src"])
        np.testing.assert_array_equal(oracle.quantize_to_int8_simd(x, case["scale"], case["zp"]), want.astype(np.int8))
        np.testing.assert_array_equal(oracle.quantize_per_tensor_affine_i8(x, case["scale"], case["zp"]), want.astype(np.int8))


def test_dequantize_known_answers(oracle, golden):
    for case in golden["dequantize_per_tensor"]:
        q = np.array(case["q"], dtype=np.float32)
        y = oracle.dequantize_per_tensor_affine(q, case["scale"], case["zp"])
        np.testing.assert_allclose(y, np.array(case["y"], dtype=np.float32), atol=case["atol"], rtol=0, err_msg=case["src"])


def test_min_max_known_answers(oracle, golden):
    for case in golden["min_max"]:
        x = np.array(case["x"], dtype=np.float32)
        mn, mx = oracle.find_min_max(x)
        assert mn == np.float32(case["min"]) and mx == np.float32(case["max"]), case["src"]
        assert oracle.min_max_fold(x) == (mn, mx)


def test_affine_params_known_answers(oracle, golden):
    for case in golden["affine_params"]:
        if case.get("error"):
            with pytest.raises(oracle.OracleError):
                oracle.calculate_affine_params(case["min"], case["max"], DT[case["dtype"]])
            continue
        s, z = oracle.calculate_affine_params(case["min"], case["max"], DT[case["dtype"]])
        if "scale" in case:
            assert s == case["scale"] and z == case["zp"], case["src"]
        else:
            assert s > 0 and case["zp_range"][0] <= z <= case["zp_range"][1]


def test_symmetric_params_known_answers(oracle, golden):
    for case in golden["symmetric_params"]:
        s, z = oracle.calculate_symmetric_params(case["min"], case["max"], DT[case["dtype"]])
        assert z == case["zp"]
        if "scale" in case:
            assert s == case["scale"]
        else:
            assert s > 0


def test_dtype_range(oracle, golden):
    for case in golden["dtype_range"]:
        assert list(oracle.get_dtype_range(DT[case["dtype"]])) == case["range"]


def test_error_cases(oracle, golden):
    fns = {
        "quantize_per_tensor_affine": lambda x, s, z: oracle.quantize_per_tensor_affine(x, s, z),
        "dequantize_per_tensor_affine": lambda x, s, z: oracle.dequantize_per_tensor_affine(x, s, z),
        "quantize_tensor_auto": lambda x, s, z: oracle.quantize_tensor_auto(x, 0, oracle.PER_TENSOR_AFFINE),
        "quantize_per_tensor_affine_simd": lambda x, s, z: oracle.quantize_per_tensor_affine_simd(x, s, z),
        "find_min_max_simd": lambda x, s, z: oracle.find_min_max(x),
    }
    for case in golden["errors"]:
        with pytest.raises(oracle.OracleError):
            fns[case["fn"]](np.array(case["x"], dtype=np.float32), case["scale"], case["zp"])


def test_backend_value_helpers(oracle, golden):
    for case in golden["backend_value"]:
        if case["fn"] == "quantize_value":
            assert oracle.backend_quantize_value(case["v"], case["scale"], case["zp"], -128, 127) == case["q"]
        else:
            assert oracle.backend_dequantize_value(case["q"], case["scale"], case["zp"]) == case["y"]


def test_core_qint8(oracle, golden):
    for case in golden["core_qint8"]:
        assert oracle.qint8_quantize(case["v"], case["scale"], case["zp"]) == case["q"], case["src"]


def test_proptest_regressions(oracle, golden):
    for case in golden["proptest_regressions"]:
        x = np.array(case["x"], dtype=np.float32)
        q = oracle.quantize_per_tensor_affine(x, case["scale"], case["zp"])
        np.testing.assert_array_equal(q, np.array(case["q"], dtype=np.float32), case["src"])
        assert np.all(np.isfinite(q))
        y = oracle.dequantize_per_tensor_affine(q, case["scale"], case["zp"])
        if "recovered" in case:
            assert y[case["recovered_index"]] == np.float32(case["recovered"])


def test_per_channel_known_properties(oracle, golden):
    for case in golden["per_channel"]:
        x = np.array(case["x"], dtype=np.float32)
        scheme = oracle.PER_CHANNEL_AFFINE if case["scheme"] == "PerChannelAffine" else oracle.PER_CHANNEL_SYMMETRIC
        q, scales, zps = oracle.quantize_per_channel_auto(x, case["axis"], 0, scheme)
        assert q.shape == x.shape and scales.size == 2 and zps.size == 2
        assert scales[1] > scales[0]
        if "zps" in case:
            assert zps.tolist() == case["zps"]


def test_slice_variant_known_answers(oracle, golden):
    """The cache-aware / tiled / streaming / NEON / mobile twins and the tensor statistics against what the
    reference's tests assert for them."""
    sv = golden["slice_variants"]
    for case in sv["carrier"]:
        out = oracle.quantize_cache_aware(np.array(case["x"], np.float32), case["scale"], case["zp"])
        for idx, val in case["checks"]:
            assert out[idx] == np.float32(val), (case["fn"], case["src"])
    for case in sv["mobile"]:
        out = oracle.quantize_mobile_optimized(np.array(case["x"], np.float32), case["scale"], case["zp"], case["reduced"])
        if "q" in case:
            np.testing.assert_array_equal(out, np.array(case["q"], np.int8), case["src"])
        for idx, val in case.get("within_one_of", []):
            assert abs(float(out[idx]) - val) <= 1.0, case["src"]
    c = sv["stats_simd"]
    st = oracle.calculate_tensor_stats_simd(np.array(c["x"], np.float32))
    assert (st["min"], st["max"], st["mean"]) == (c["min"], c["max"], c["mean"])
    assert abs(st["std_dev"] - np.float32(np.sqrt(c["std_dev_f64_sqrt_of"]))) <= c["std_eps"]
    c = sv["stats_cache_optimized"]
    mn, mx, mean, std = oracle.calculate_tensor_stats_cache_optimized(np.array(c["x"], np.float32))
    assert (mn, mx) == (c["min"], c["max"]) and abs(mean - c["mean"]) < c["mean_eps"] and std > 0
    c = sv["min_max_neon"]
    mn, mx = oracle.find_min_max(np.array(c["x"], np.float32))  # find_min_max_neon folds with the same min / max
    assert (mn, mx) == (np.float32(c["min"]), np.float32(c["max"]))
    with pytest.raises(oracle.OracleError):
        oracle.quantize_cache_aware(np.ones(2, np.float32), sv["errors"]["bad_scale"], 0)
    with pytest.raises(oracle.OracleError):
        oracle.calculate_tensor_stats_simd(np.empty(0, np.float32))
    with pytest.raises(oracle.OracleError):
        oracle.calculate_tensor_stats_cache_optimized(np.empty(0, np.float32))


def test_slice_variant_closed_forms(oracle):
    """What the known answers leave open: the population (not sample) variance, the raw-moment form's f32
    roundings, ties and the 256-element switch of the mobile quantizer, the i8 clamp of the carrier."""
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(5000) * 3 + 7).astype(np.float32)
    st = oracle.calculate_tensor_stats_simd(x)
    xd = x.astype(np.float64)
    assert st["mean"] == np.float32(xd.mean())
    assert st["variance"] == pytest.approx(xd.var(ddof=0), rel=1e-6)          # a sample variance would be 2e-4 off
    assert st["std_dev"] == pytest.approx(xd.std(ddof=0), rel=1e-6)
    assert (st["min"], st["max"]) == (x.min(), x.max())
    mn, mx, mean, std = oracle.calculate_tensor_stats_cache_optimized(x)
    mean32 = np.float32(xd.sum() / x.size)
    var32 = np.float32((xd * xd).sum() / x.size - np.float64(mean32) ** 2)
    assert (mn, mx, mean) == (x.min(), x.max(), mean32)
    assert std == pytest.approx(np.sqrt(var32, dtype=np.float32), rel=1e-6)
    # constant data: raw moments cancel to ~0 (possibly slightly negative -> NaN std, as in the reference)
    mn, mx, mean, std = oracle.calculate_tensor_stats_cache_optimized(np.full(100, 0.1, np.float32))
    assert mean == np.float32(0.1) and (np.isnan(std) or std < 1e-3)
    # mobile: ties at +-2.5 and +-0.5 (scale 1): round goes away from zero, floor(v + 0.5) goes up
    ties = np.array([2.5, -2.5, 0.5, -0.5, 1.5, -1.5], np.float32)
    np.testing.assert_array_equal(oracle.quantize_mobile_optimized(ties, 1.0, 0, True), [3, -3, 1, -1, 2, -2])
    big = np.tile(ties, 50)  # 300 elements: past the 256-element switch
    np.testing.assert_array_equal(oracle.quantize_mobile_optimized(big, 1.0, 0, True)[:6], [3, -2, 1, 0, 2, -1])
    np.testing.assert_array_equal(oracle.quantize_mobile_optimized(big, 1.0, 0, False)[:6], [3, -3, 1, -1, 2, -2])
    # 0.49999997 + 0.5 rounds to 1.0 in f32: floor(v + 0.5) gives 1 where round gives 0
    edge = np.full(300, 0.49999997, np.float32)
    assert oracle.quantize_mobile_optimized(edge, 1.0, 0, True)[0] == 1
    assert oracle.quantize_mobile_optimized(edge, 1.0, 0, False)[0] == 0
    # saturation, NaN -> 0 in the i8 form, NaN kept in the carrier, zero point added after rounding
    sat = np.array([1e9, -1e9, np.nan, 3.4], np.float32)
    np.testing.assert_array_equal(oracle.quantize_mobile_optimized(sat, 1.0, 5, False), [127, -128, 0, 8])
    car = oracle.quantize_cache_aware(sat, 1.0, 5)
    assert car[0] == 127 and car[1] == -128 and np.isnan(car[2]) and car[3] == 8
    np.testing.assert_array_equal(oracle.quantize_cache_aware(x, 0.05, -3), oracle.quantize_per_tensor_affine_simd(x, 0.05, -3))
