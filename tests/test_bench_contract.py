"""The benchmark's command-line contract, as far as it can be checked without a GPU (CPU cases), and the shape of
the JSON line it prints on a GPU (gpu case, short run)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, BENCH, "--gpus", "2", "--steps", "1", "--warmup", "0"], capture_output=True,
                          text=True, timeout=120)
    assert proc.returncode != 0
    assert "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


def test_no_gpu_means_no_result_not_a_cpu_fallback():
    env = dict(os.environ, HIP_VISIBLE_DEVICES="-1", CUDA_VISIBLE_DEVICES="")
    proc = subprocess.run([sys.executable, BENCH, "--steps", "1", "--warmup", "0", "--no-cpu-baseline", "--no-extra"],
                          capture_output=True, text=True, timeout=300, env=env)
    assert proc.returncode != 0 and proc.stdout.strip() == ""
    assert "no GPU" in proc.stderr


def test_product_modules_do_not_import_the_oracle():
    """Only tests, the smoke check and the benchmark's CPU-baseline leg may touch oracle/."""
    offenders = []
    for base, _, files in os.walk(os.path.join(ROOT, "torsh_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".hpp")):
                text = open(os.path.join(base, f), errors="ignore").read()
                if "pyoracle" in text or "liboracle" in text or "torsh_quant_oracle" in text or "torsh_calib_oracle" in text:
                    offenders.append(os.path.join(base, f))
    assert not offenders, offenders
    bench = open(BENCH).read()
    # the benchmark names the oracle only inside cpu_baseline()
    head, _, rest = bench.partition("def cpu_baseline(")
    body, _, tail = rest.partition("\ndef ")
    assert "pyoracle" not in head and "pyoracle" not in tail and "pyoracle" in body


@pytest.mark.gpu
def test_json_line_has_the_contract_fields():
    proc = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "5", "--no-cpu-baseline", "--no-extra"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 5 and d["vs_baseline"] is None
    assert "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] in ("hbm", "mfma") and r["frac"] == pytest.approx(r["achieved"] / r["peak"])
    assert d["value"] > 0 and d["ms_per_step"] > 0
    # the metric's second half (quantize GB/s) travels inside `roofline`, on the bytes that move
    for key, nbytes in (("quantize", 5 << 24), ("dequantize", 5 << 24), ("minmax", 4 << 24)):
        h = r["hbm"][key]
        assert h["bytes"] == nbytes and h["peak"] == 8000.0 and h["unit"] == "GB/s"
        assert h["achieved"] == pytest.approx(nbytes / (h["us"] * 1e-6) / 1e9)
        assert h["frac"] == pytest.approx(h["achieved"] / h["peak"]) and 0 < h["frac"] < 1
