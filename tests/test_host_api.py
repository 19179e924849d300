"""Runs the C++ host-layer test program (tests/host/host_api_test.cpp): the reference's own unit tests restated
against the mirrored C++ API, and parity of the device results with the CPU oracle.

The program is built ahead of time (``make -C tests/host``, also done by ``__graft_entry__.build()``); it is built
here only when no binary exists.  It runs once per session; each case is reported as its own pytest test."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host", "bin", "host_api_test")

CPU_CASES = [
    "test_calculate_affine_quantization_params",
    "test_calculate_symmetric_quantization_params",
    "test_params_match_oracle_on_random_ranges",
    "test_get_dtype_range",
    "test_quant_config",
    "test_error_cases_before_the_device",
    "test_backend_params_and_tensor",
    "test_module_shapes_before_the_device",
    "test_observer_creation_and_host_logic",
    "test_config_json_round_trip",
    "test_weight_file_round_trip_and_corruption",
    "test_model_quantizer_scalar_logic",
    "test_kernel_plugin_interface",
    "test_slice_variant_errors_before_the_device",
    "test_fake_quantize_errors_before_the_device",
    "test_scalar_quantized_types",
]
GPU_CASES = [
    "parity_torsh_nn_quantizer_and_qtype_slices",
    "parity_torsh_nn_quantized_helpers",
    "test_quantize_per_tensor_affine",
    "test_dequantize_per_tensor_affine",
    "test_quantize_tensor_auto",
    "test_quantize_with_config",
    "test_dequantize",
    "test_quantize_auto",
    "test_simd_slice_functions",
    "parity_quantize_tensor_auto_and_round_trip",
    "parity_quantize_per_channel_auto",
    "parity_backend_quantize_dequantize",
    "parity_backend_matmul",
    "parity_backend_qconv2d",
    "parity_quantized_linear_module",
    "parity_quantized_conv2d_module",
    "test_calculate_quantization_metrics",
    "test_compare_quantization_configs",
    "test_auto_calibrate_quantization",
    "parity_metrics_and_compare_configs",
    "test_observers",
    "parity_observers_against_the_oracle",
    "parity_quantize_batch_consistent",
    "test_slice_variants",
    "parity_slice_variants",
    "parity_model_quantizer",
    "test_quantized_modules_survive_a_weight_file",
    "test_special_schemes",
    "parity_special_schemes",
    "test_searched_thresholds_and_mixed_precision",
    "parity_searched_thresholds_and_mixed_precision",
    "parity_backend_qadd_qrelu",
    "test_kernel_plugin_dispatch",
    "test_fake_quantize",
    "parity_fake_quantize",
]


def _binary():
    if not os.path.exists(BIN):
        from oracle import pyoracle
        from torsh_amd import hipq

        hipq.load()
        pyoracle.lib()
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host")], check=True, capture_output=True)
    return BIN


def test_two_fma_division_equals_ieee_division():
    """The kernels divide by a per-row / per-tensor scale as fma(fma(-q0, b, a), y, q0) with y = 1/b; this sweeps every
    numerator significand for a few dozen denominators on the CPU and demands equality with a / b."""
    _binary()
    exe = os.path.join(ROOT, "tests", "host", "bin", "div_rn_check")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host"), "bin/div_rn_check"], check=True, capture_output=True)
    proc = subprocess.run([exe, "200"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert " 0 mismatches" in proc.stdout


def test_three_instruction_round_half_away_equals_roundf():
    """round(v) is computed as trunc(v + copysign(0.49999997, v)) on the device; this compares it with roundf for
    every finite float on the CPU."""
    _binary()
    exe = os.path.join(ROOT, "tests", "host", "bin", "round_away_check")
    if not os.path.exists(exe):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host"), "bin/round_away_check"], check=True,
                       capture_output=True)
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 mismatches" in proc.stdout


def _run(args):
    proc = subprocess.run([_binary(), *args], capture_output=True, text=True, timeout=300)
    results = {}
    for line in proc.stdout.splitlines():
        word, _, rest = line.partition(" ")
        if word in ("ok", "skip"):
            results[rest.strip()] = (word, "")
        elif word == "FAIL":
            name, _, why = rest.partition(":")
            results[name.strip()] = ("FAIL", why.strip())
        elif word == "run":
            results.setdefault(rest.strip(), ("crashed", proc.stderr[-2000:]))
    return results, proc


@pytest.fixture(scope="module")
def cpu_results():
    return _run(["--cpu-only"])


@pytest.fixture(scope="module")
def gpu_results():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return _run([])


@pytest.mark.parametrize("case", CPU_CASES)
def test_host_logic(cpu_results, case):
    results, proc = cpu_results
    assert case in results, f"case did not run; stderr: {proc.stderr[-1000:]}"
    assert results[case][0] == "ok", results[case][1]


def test_cpu_only_run_skips_every_device_case(cpu_results):
    results, _ = cpu_results
    assert all(results[c][0] == "skip" for c in GPU_CASES)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CPU_CASES + GPU_CASES)
def test_host_api_on_device(gpu_results, case):
    results, proc = gpu_results
    assert case in results, f"case did not run; stderr: {proc.stderr[-1000:]}"
    assert results[case][0] == "ok", results[case][1]
