"""What bench.py promises without a GPU: one GPU only, and traffic figures that trace back to the committed
profile summaries."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_every_measured_traffic_figure_has_its_summary_and_multi_launch_steps_add_up():
    sys.path.insert(0, ROOT)
    import bench
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        t = json.load(f)
    assert t.get("_measured_at_commit"), "traffic.json names the commit its counter runs were taken at"
    for w, rec in t.items():
        if w.startswith("_"):
            continue
        path = os.path.join(ROOT, "profiles", f"{rec['kernel']}_{w}.txt")
        assert os.path.exists(path), path
        text = open(path).read()
        assert f"--workload {w} " in text and "rocprofv3 --kernel-trace --stats" in text and "rocprofv3 --pmc FETCH_SIZE" in text
        assert bench.measured_traffic(w) == rec["hbm_bytes_per_launch"]
    chunks = ["c3_prefill_p0", "c3_prefill_p2048", "c3_prefill_p4096", "c3_prefill_p6144"]
    assert bench.measured_traffic("c3_chunked_prefill") == sum(t[c]["hbm_bytes_per_launch"] for c in chunks)
    assert bench.measured_traffic("c4_decode_mix") == 5 * t["c4_decode_sliding"]["hbm_bytes_per_launch"] + t["c4_decode_global"]["hbm_bytes_per_launch"]
    assert bench.measured_traffic("no_such_workload") is None
    for w in bench.WORKLOADS:      # every named workload can at least be described without a device
        assert isinstance(w, str) and w
