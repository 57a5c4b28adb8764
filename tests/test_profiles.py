"""The counter summary the bench line quotes must belong to the kernel source in the tree."""
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_headline_traffic_summary_was_taken_on_this_kernel_source():
    import sys
    sys.path.insert(0, ROOT)
    import bench
    with open(os.path.join(ROOT, "profiles", "gemv_q4k_5120x5120_hbm_traffic.json")) as f:
        t = json.load(f)
    # sha256 over gemv.hip, common.hpp and deq_at.hpp: a change to the mat-vec kernel without a new counter run shows here
    assert t["kernel_source_sha16"] == bench.kernel_source_sha()
    assert bench.headline_traffic()["stale"] is False
    assert abs(t["hbm_bytes_per_launch"] / t["algorithmic_bytes"] - t["ratio"]) < 1e-3
