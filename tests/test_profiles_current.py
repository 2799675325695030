"""The hardware counters kept under profiles/ (read by bench.py for roofline.frac and roofline.traffic) were
taken with the kernel sources in the tree: bench.py refuses stale ones, and this test says so before a
benchmark run does."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_stored_counters_match_the_kernel_sources():
    import bench
    with open(bench.PROFILE_FILE) as f:
        stored = json.load(f)
    keys = [k for k in stored if not k.startswith("_")]
    assert "cfg2_default_b128:A:fwd" in keys and "cfg4_train_b128:A:bwd" in keys
    for key in keys:
        now = bench.kernel_fingerprint(key.rsplit(":", 1)[1])
        assert stored[key].get("kernel_sha16") == now, \
            f"profiles/traffic.json entry {key} is from other kernel sources: collect the counters again " \
            f"(profiles/*.md give the commands)"
