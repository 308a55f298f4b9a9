"""Host-side checks of bench.py that need no GPU: the measured-traffic table beside the profiles and the pinned graphs."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_measured_traffic_table_is_consistent_with_the_profiles():
    import bench
    with open(bench.TRAFFIC_FILE) as f:
        table = json.load(f)
    assert len(table) >= 4
    seen = set()
    for graph_hash, e in table.items():
        assert len(graph_hash) == 16 and int(graph_hash, 16) >= 0
        assert e["bytes"] == e["fetched"] + e["written"] and e["bytes"] > 0
        assert bench.measured_traffic(graph_hash) == e["bytes"]
        assert e["workload"] in bench.WORKLOADS and os.path.isfile(os.path.join(ROOT, e["profile"]))
        # the summary names the hash it was measured on
        assert graph_hash in open(os.path.join(ROOT, e["profile"])).read(), graph_hash
        seen.add(e["workload"])
    assert seen == {"C2", "C3", "C4", "C5"}
    assert bench.measured_traffic("0" * 16) is None
    # the committed winners that a run without time for a search falls back to are among the profiled graphs
    pins = {e["pin"] for e in table.values()}
    for key in ("C2", "C3", "C4", "C5"):
        assert bench.WORKLOADS[key][5] in pins, key
    for key, profile in bench.PROFILE_OF.items():
        assert os.path.isfile(os.path.join(ROOT, profile)), profile
