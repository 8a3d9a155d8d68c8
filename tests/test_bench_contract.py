"""Host-side checks of bench.py that need no GPU: more than one GPU is refused with a message, and the CPU
baseline leg returns the fields the result line carries."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)


def test_cpu_baseline_fields_on_a_small_sample(monkeypatch):
    sys.path.insert(0, ROOT)
    import bench
    monkeypatch.setattr(bench, "M", 256)
    monkeypatch.setattr(bench, "N", 512)
    monkeypatch.setattr(bench, "K", 256)
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((256, 256)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    w = (rng.standard_normal((512, 256)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    out = bench.cpu_baseline(x, w, target_seconds=0.5)
    assert out["kind"] == "port" and out["unit"] == "TFLOP/s" and out["cores"] >= 1 and out["value"] > 0
    assert isinstance(out["sample"], str) and out["aten_linear_bf16_on_cpu"]["value"] > 0
    assert bench.GEMM_TRAFFIC_BYTES > 2 * (4096 * 7168 + 36864 * 7168)      # at least the operands once
