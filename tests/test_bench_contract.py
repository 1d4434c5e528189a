"""bench.py's side of the measurement contract that needs no GPU: it refuses a second GPU, and a
committed counter profile is reported only while the library's sources are the ones it was taken
on."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True)
    assert run.returncode != 0
    assert "one GPU" in run.stderr and "--gpus 1" in run.stderr


def test_counter_traffic_is_dated_by_the_library_sources(tmp_path, monkeypatch):
    import bench
    digest = bench.csrc_digest()
    assert len(digest) == 16 and digest == bench.csrc_digest()
    profiles = tmp_path / "profiles"
    profiles.mkdir()
    record = {"fetch_size_kib_per_dispatch": 1000, "fetch_scale": 2.0,
              "write_size_kib_per_dispatch": 10, "write_scale": 1.0, "head": "abc1234",
              "csrc_digest": digest}
    (profiles / "traffic_case.json").write_text(json.dumps(record))
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    monkeypatch.setattr(bench, "csrc_digest", lambda: digest)
    assert bench.measured_traffic("case") == (1024 * 2010, "abc1234", True)
    # the kernels changed after the profile was taken: the figure is withheld, its date is not
    monkeypatch.setattr(bench, "csrc_digest", lambda: "0" * 16)
    assert bench.measured_traffic("case") == (None, "abc1234", False)
    assert bench.measured_traffic("never_profiled") == (None, None, None)


def test_committed_traffic_profiles_name_their_commit_and_sources():
    import bench
    folder = os.path.join(ROOT, "profiles")
    names = [n for n in os.listdir(folder) if n.startswith("traffic_") and n.endswith(".json")]
    assert names
    for n in names:
        t = json.load(open(os.path.join(folder, n)))
        assert t.get("head") and t.get("csrc_digest"), n
        for key in ("fetch_size_kib_per_dispatch", "fetch_scale", "write_size_kib_per_dispatch",
                    "write_scale", "workload", "kernel", "source"):
            assert key in t, (n, key)
        assert os.path.exists(os.path.join(ROOT, t["source"].split(" ")[0])), (n, t["source"])
