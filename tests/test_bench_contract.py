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


def test_reported_gemm_traffic_belongs_to_the_kernel_as_it_is_now(tmp_path, monkeypatch, capsys):
    """`roofline.traffic` comes from rocprofv3 counter runs kept under profiles/ together with the sha256 of the
    csrc/gemm.hip they were collected on.  bench.py reports the figures only while the source still has that digest;
    otherwise it reports null and says so loudly on stderr -- never a stale number."""
    sys.path.insert(0, ROOT)
    import bench
    digest = bench.gemm_source_digest()
    assert len(digest) == 64
    good = tmp_path / "good.md"
    good.write_text(f"...\ntraffic_bytes=1923015680 dram_path_bytes=1900000000 gemm_source_sha256={digest}\n")
    monkeypatch.setattr(bench, "PROFILE", str(good))
    traffic, source = bench.gemm_traffic_bytes()
    assert traffic == {"tcc_ea": 1923015680, "dram_path": 1900000000} and source == "profiles/good.md"
    stale = tmp_path / "stale.md"
    stale.write_text("traffic_bytes=1923015680 dram_path_bytes=1900000000 gemm_source_sha256=" + "0" * 64 + "\n")
    monkeypatch.setattr(bench, "PROFILE", str(stale))
    traffic, why = bench.gemm_traffic_bytes()
    assert traffic is None and "another version" in why
    assert "STALE TRAFFIC FIGURE NOT REPORTED" in capsys.readouterr().err
    monkeypatch.setattr(bench, "PROFILE", str(tmp_path / "absent.md"))
    assert bench.gemm_traffic_bytes() == (None, "no profile summary")
    # the committed summary: whatever its state, what bench.py reports is either its figures or null
    monkeypatch.undo()
    traffic, source = bench.gemm_traffic_bytes()
    if traffic is not None:
        assert traffic["tcc_ea"] > 2 * (4096 * 7168 + 36864 * 7168) and source.startswith("profiles/")      # at least the operands once
        assert 0 < traffic["dram_path"] <= traffic["tcc_ea"] * 1.05
