"""Host-side pieces of bench.py that need no GPU: the source fingerprint and the HBM traffic figure
it reads out of the committed counter summaries."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402

WORKLOADS = ["headline_e64_zipf", "balanced_e16", "mixtral_e8", "fine_e256_top8"]


def test_fingerprint_is_stable_and_covers_the_sources():
    a, b = bench.source_fingerprint(), bench.source_fingerprint()
    assert a == b and len(a) == 16 and int(a, 16) >= 0


@pytest.mark.parametrize("workload", WORKLOADS)
def test_committed_traffic_summary_is_readable(workload):
    """Every profiled workload has a summary bench.py can read: a positive byte count that is at
    least the weights once (nothing can stream less than that) and below ten times that."""
    from aristos_amd import synth
    d = synth.WORKLOADS[workload].config.derive()
    nbytes, same_sources = bench.measured_traffic(workload)
    assert nbytes is not None and same_sources in (True, False)
    weights = 2.0 * d.E * d.H * d.I * d.elem_bytes
    assert 0.95 * weights < nbytes < 10.0 * weights


def test_unknown_workload_has_no_traffic_figure():
    assert bench.measured_traffic("no_such_workload") == (None, None)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) or "1 GPU" in (r.stdout + r.stderr) or "single" in (r.stdout + r.stderr).lower()


def test_the_json_line_says_what_ran_before_the_timed_region():
    """`warmup` alone under-reports the warm-up: the line also carries the launches of the per-phase
    measurements and the rehearsal passes, and what the first (cold) pass measured."""
    rec = bench.prewarm_protocol(steps=20, warmup=5, pass_ms=[0.3257, 0.3145, 0.2937, 0.3011])
    assert rec["prewarm_launches"] == (8 + 64) + (32 + 1536) + 3 * (5 + 20)
    assert rec["cold_ms_per_step"] == 0.3257 and rec["pass_ms_per_step"][-1] == 0.3011
    assert rec["prewarm_detail"]["rehearsal_passes"] == 3 and len(rec["pass_ms_per_step"]) == 4
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert "**prewarm_protocol(args.steps, args.warmup, pass_ms)" in src   # the keys reach the printed line


def test_power_sampler_reads_a_hwmon_node_and_reports_none_without_one(tmp_path, monkeypatch):
    """The socket-power figure comes from power1_input (microwatts) of the amdgpu hwmon node; a box
    without the node gets `power: null`, never a made-up number."""
    assert bench.sustained_power(0.3, lambda: None) is None or "mean_w" in bench.sustained_power(0.3, lambda: None)
    node = tmp_path / "power1_input"
    node.write_text("1399000000\n")
    (tmp_path / "power1_cap").write_text("1400000000\n")
    import glob
    monkeypatch.setattr(glob, "glob", lambda pattern: [str(node)])
    import time
    t0 = time.perf_counter()
    ps = bench.PowerSampler()
    ps.start()
    time.sleep(0.5)
    out = ps.stop(t0)
    assert out["mean_w"] == 1399.0 and out["max_w"] == 1399.0 and out["cap_w"] == 1400.0 and out["samples"] >= 2
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert '"power": power' in src
