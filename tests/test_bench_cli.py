"""bench.py's command line on a machine without a GPU: what it refuses, and the helpers that
need no device."""
import json
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0
    assert "one GPU" in run.stderr and not run.stdout.strip()


def test_recorded_traffic_is_withheld_for_other_kernel_sources(monkeypatch):
    sys.path.insert(0, str(ROOT))
    import bench
    name = "grf::fused_wave_group_kernel<grf::SegmentWalkT<false>, 1, 1>"
    record = json.loads((ROOT / "profiles" / "fused_gemv_m1_qwen27b_mlp_traffic.json").read_text())
    monkeypatch.setattr(bench, "kernel_sources_sha256", lambda: record["kernel_sources_sha256"])
    figure, source = bench.recorded_traffic(False, 1, name)
    assert figure == record["traffic_bytes_per_launch"]["fused_wave_group_kernel"] and "recorded" in source
    monkeypatch.setattr(bench, "kernel_sources_sha256", lambda: "0" * 64)
    figure, source = bench.recorded_traffic(False, 1, name)
    assert figure is None and "other kernel sources" in source
    assert bench.recorded_traffic(False, 7, name)[0] is None  # no counter record for that batch
