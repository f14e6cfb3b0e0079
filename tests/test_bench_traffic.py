"""bench.py reports HBM traffic only while the recorded counter figures belong to the present kernel sources."""
import json

import bench


def test_traffic_follows_the_source_hash(tmp_path, monkeypatch):
    table = {"calibration": {"fetch_factor": 2.0, "write_factor": 1.0, "profile": "profiles/copy_calibration_1GiB.md"},
             "kernels": {k: {"fetch_kib": 100.0, "write_kib": 50.0, "source_hash": "stale", "profile": "profiles/x.md"}
                         for k in bench.TRAFFIC_SOURCES}}
    path = tmp_path / "traffic.json"
    path.write_text(json.dumps(table))
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(path))
    got, note = bench.measured_traffic("decode")
    assert got is None and "changed" in note
    bench.record_traffic(["decode=200,10"])
    got, note = bench.measured_traffic("decode")
    assert got == 200 * 1024 * 2.0 + 10 * 1024 * 1.0 and note == "profiles/x.md"
    assert bench.measured_traffic("prefill")[0] is None  # only the recorded kernel is current
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(tmp_path / "missing.json"))
    assert bench.measured_traffic("decode")[0] is None


def test_the_committed_table_names_every_kernel_and_its_profile():
    import os
    with open(bench.TRAFFIC_FILE) as f:
        table = json.load(f)
    assert set(table["kernels"]) == set(bench.TRAFFIC_SOURCES)
    root = os.path.dirname(os.path.abspath(bench.__file__))
    for e in table["kernels"].values():
        assert os.path.exists(os.path.join(root, e["profile"]))
    assert os.path.exists(os.path.join(root, table["calibration"]["profile"]))
