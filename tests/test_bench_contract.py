"""bench.py's command-line contract that needs no GPU."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    """One GPU stands in for the group: `--gpus N` with N > 1 exits and says why."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr) and "--gpus" in (r.stdout + r.stderr), r.stdout + r.stderr


def test_traffic_record_belongs_to_the_kernel_sources_in_the_tree():
    """profiles/traffic.json carries the digest of the kernel sources its counters were
    measured on; bench.py reports `roofline.traffic` only while that digest matches.  A change
    under moonep_amd/csrc without new counter runs would silently turn every traffic figure
    of the bench line into null."""
    import json

    sys.path.insert(0, ROOT)
    import bench

    with open(bench.TRAFFIC_FILE) as f:
        rec = json.load(f)
    assert rec["source_digest"] == bench.kernel_source_digest(), (
        "kernel sources changed since profiles/traffic.json was measured: repeat the two "
        "rocprofv3 --pmc runs named in profiles/bench_kernels_pmc_traffic.md")
    for key in ("dispatch_kernel", "combine_kernel", "plan_kernel", "prefetch_kernel@planner",
                "prefetch_pull_kernel@ring8", "grad_reduce_kernel@ring8", "dispatch_epilogue",
                "combine_prologue", "grouped_gemm_forward"):
        k = rec["kernels"][key]
        assert k["fetch_bytes"] > 0 and k["write_bytes"] > 0, key
        assert bench.measured_traffic(key, k.get("grid"))[0] == k["fetch_bytes"] + k["write_bytes"]
