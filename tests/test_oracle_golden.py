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
