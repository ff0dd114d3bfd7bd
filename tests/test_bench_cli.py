"""bench.py's command line: what can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_unknown_leg_is_refused():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--only", "nothing"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0 and "invalid choice" in proc.stderr


def test_traffic_of_a_summary_measured_on_other_sources_is_not_quoted(tmp_path):
    sys.path.insert(0, ROOT)
    import bench
    table = "pack_mixed_kernel   407755.5   53312.0   889628570   883097600   1.0074\n"
    stale = tmp_path / "stale.txt"
    stale.write_text("source_hash: 0123456789abcdef\n" + table)
    traffic, alg, note = bench.measured_traffic("pack_mixed_kernel", str(stale))
    assert traffic is None and alg is None and "stale" in note
    unmarked = tmp_path / "unmarked.txt"
    unmarked.write_text(table)
    assert bench.measured_traffic("pack_mixed_kernel", str(unmarked))[0] is None
    fresh = tmp_path / "fresh.txt"
    fresh.write_text("source_hash: %s\n" % bench.kernel_source_hash() + table)
    assert bench.measured_traffic("pack_mixed_kernel", str(fresh)) == (889628570, 883097600, None)
    assert bench.measured_traffic("no_such_kernel", str(fresh))[0] is None
