"""bench.py's HBM traffic figure comes from a committed counter pass that is
stamped with a hash of the kernel sources: the figure is reported as stale
when the sources in the tree are not the ones that were measured."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location(
        "bench_under_test", os.path.join(ROOT, "bench.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def test_traffic_is_stale_exactly_when_the_sources_changed(tmp_path):
    bench = _bench()
    csrc = tmp_path / "poplibs_amd" / "csrc"
    csrc.mkdir(parents=True)
    (csrc / "a.hip").write_text("kernel one\n")
    (csrc / "b.hpp").write_text("header\n")
    (csrc / "notes.txt").write_text("not a source\n")
    (tmp_path / "profiles").mkdir()
    bench.ROOT = str(tmp_path)
    stamp = bench.kernel_sources_hash()
    traffic = {"kernel_sources_sha256": stamp,
               "c2": {"bytes_per_launch": 123}}
    path = tmp_path / "profiles" / "hbm_traffic.json"
    path.write_text(json.dumps(traffic))
    assert bench.measured_traffic("c2") == (123, False)
    assert bench.measured_traffic("c9") == (None, None)
    # files that are no kernel sources do not count
    (csrc / "notes.txt").write_text("changed\n")
    assert bench.measured_traffic("c2") == (123, False)
    # a changed source, a new source: stale
    (csrc / "a.hip").write_text("kernel two\n")
    assert bench.measured_traffic("c2") == (123, True)
    (csrc / "a.hip").write_text("kernel one\n")
    assert bench.measured_traffic("c2") == (123, False)
    (csrc / "c.cpp").write_text("new\n")
    assert bench.measured_traffic("c2") == (123, True)
    # an entry's own stamp, where it has one, goes before the file's
    (csrc / "c.cpp").unlink()
    traffic["c2"]["kernel_sources_sha256"] = "other"
    path.write_text(json.dumps(traffic))
    assert bench.measured_traffic("c2") == (123, True)
    # no file: no figure
    path.unlink()
    assert bench.measured_traffic("c2") == (None, None)


def test_committed_traffic_file_has_a_stamp_and_every_workload():
    with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
        data = json.load(f)
    assert len(data["kernel_sources_sha256"]) == 64
    for key in ("c2", "c3", "c4", "c5"):
        assert data[key]["bytes_per_launch"] > 0
