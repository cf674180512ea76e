"""bench.py's contract on the command line, as far as it can be checked without
a GPU: one GPU only, the fp32 parity case is not a bench line, and the measured
HBM traffic is only quoted for the kernels and the split count it was taken on."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*flags):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True,
                          cwd=ROOT, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    res = _run("--gpus", "2")
    assert res.returncode == 2
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_the_fp32_parity_case_is_not_a_bench_line():
    res = _run("--workload", "1")
    assert res.returncode == 2
    assert "parity case" in res.stderr


def test_traffic_record_is_tied_to_sources_and_split_count(monkeypatch, tmp_path, capsys):
    sys.path.insert(0, ROOT)
    import bench

    rec = {"unit": "bytes", "workloads": {"w": {"splits": 3, "kernel_sources": bench.kernel_source_hash(),
                                                "attn": 1.0, "append": 2.0}}}
    path = tmp_path / "t.json"
    path.write_text(json.dumps(rec))
    monkeypatch.setattr(bench, "TRAFFIC_JSON", str(path))
    assert bench.measured_traffic("w", 3)["attn"] == 1.0
    assert bench.measured_traffic("w", 4) is None                    # another split count
    assert "collected again" in capsys.readouterr().err
    assert bench.measured_traffic("other", 3) is None                # no record
    rec["workloads"]["w"]["kernel_sources"] = "0" * 16
    path.write_text(json.dumps(rec))
    assert bench.measured_traffic("w", 3) is None                    # kernels changed since


def test_committed_traffic_record_matches_the_committed_kernels():
    sys.path.insert(0, ROOT)
    import bench

    doc = json.load(open(bench.TRAFFIC_JSON))
    for name, rec in doc["workloads"].items():
        assert rec["kernel_sources"] == bench.kernel_source_hash(), name
