"""bench.py's counter figures come from profiles/counters.json: the file parses, names sources that exist, and a
figure read at other kernel sources than the tree's is flagged, not silently reported."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_counter_file_covers_the_bench_workloads():
    import bench

    with open(os.path.join(ROOT, "profiles", "counters.json")) as fh:
        configs = json.load(fh)["configs"]
    assert {"1", "2", "5", "6"} <= set(configs)
    for key, entry in configs.items():
        assert entry["traffic_bytes"] > 0 and entry["rocprof_avg_us"] > 0, key
        for f in entry["sources"] + entry["files"].split(", "):
            assert os.path.exists(os.path.join(ROOT, f)), (key, f)
        loaded = bench.load_counters(int(key))
        assert loaded["stale"] == (bench.sources_sha16(entry["sources"]) != entry["sources_sha16"])
    assert bench.load_counters(99) is None


def test_physical_fraction_and_model_fraction_are_kept_apart():
    import bench

    cnt = dict(traffic_bytes=250_000_000, files="f", library_commit="c", stale=True)
    roof = bench.physical_roofline({"bytes_per_launch": 450_000_000}, cnt, 0.05)
    assert roof["achieved"] == 5000.0 and roof["frac"] == 0.625 and roof["counters_stale"] is True
    assert roof["model_achieved"] == 9000.0 and roof["model_frac"] == 1.125
    none = bench.physical_roofline({"bytes_per_launch": 450_000_000}, None, 0.05)
    assert none["frac"] is None and none["traffic"] is None and none["model_frac"] == 1.125
