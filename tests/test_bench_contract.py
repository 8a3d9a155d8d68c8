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


def test_reported_gemm_traffic_belongs_to_the_kernel_as_it_is_now():
    """`roofline.traffic` comes from a rocprofv3 counter run kept under profiles/; the summary names the tiling it
    was measured on, and bench.py reports the figure only while csrc/gemm.hip still has that tiling.  This test
    fails when the tiling constants were changed without collecting the counters again (bench.py itself then
    reports null rather than a stale number)."""
    sys.path.insert(0, ROOT)
    import bench
    sig = bench.gemm_tiling_signature()
    assert "?" not in sig, sig
    traffic, source = bench.gemm_traffic_bytes()
    assert traffic is not None, source
    assert traffic > 2 * (4096 * 7168 + 36864 * 7168)      # at least the operands once
    assert source.startswith("profiles/")
