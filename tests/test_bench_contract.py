"""The benchmark's contract with its driver: one JSON line with the agreed keys, a refusal of more than one GPU, and CPU
baseline objects that say what they ran on."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KEYS = {"metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline"}


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + list(args), capture_output=True, text=True, timeout=600)


def test_more_than_one_gpu_is_refused_with_a_message():
    p = _bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert p.returncode != 0
    assert "one GPU" in (p.stderr + p.stdout)


def test_cpu_baseline_objects_name_the_cpu_and_both_thread_counts():
    sys.path.insert(0, ROOT)
    import bench
    from oracle import cpubaseline
    if not cpubaseline.available():
        pytest.skip("host CPU has no AVX512-VNNI")
    conv = bench.cpu_baseline_conv(16, 12, 12, 16, 3, 1, 1, budget_s=0.3)
    gemm = bench.cpu_baseline_gemm(256, 128, True, budget_s=0.3)
    for obj in (conv, gemm):
        assert obj["kind"] == "port" and obj["unit"] == "TOPS" and obj["value"] > 0 and obj["value_1_thread"] > 0
        assert obj["cores"] >= 1 and obj["logical_cpus"] >= obj["cores"] and isinstance(obj["cpu_model"], str) and "avx512_vnni" in obj["isa_flags"]
        assert "sample" in obj and len(obj["sample"]) > 20


@pytest.mark.gpu
@pytest.mark.parametrize("workload", ["gemm1024", "gemm:16x1024x512", "conv:64x56x56:64:k3", "blockquant:4096x4096x1", "mha:256x4:1:300", "net:mobilenetv2:1", "peak:launch:8"])
def test_bench_prints_one_json_line_with_the_agreed_keys(workload):
    p = _bench("--workload", workload, "--steps", "3", "--warmup", "1", "--no-cpu")
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    assert KEYS <= set(d), KEYS - set(d)
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert isinstance(d["config"], dict) and "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert {"bound", "achieved", "peak", "unit", "frac", "traffic"} <= set(r)
    assert np.isfinite(d["value"]) and d["value"] > 0
