"""CPU checks of what bench.py promises without a GPU: every profile summary it reads its HBM traffic figure from exists and
carries the line it parses, and a request for more than one GPU is refused with a message."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_traffic_source_named_in_bench_has_its_line():
    sys.path.insert(0, ROOT)
    import bench
    src = open(os.path.join(ROOT, "bench.py")).read()
    names = set(re.findall(r'"([A-Za-z0-9_]+\.md)"', src))
    assert len(names) >= 7
    for fname in sorted(names):
        value, where = bench.profile_traffic(fname)
        assert where == "profiles/" + fname, fname
        assert isinstance(value, int) and value > 10_000_000, (fname, value)
    assert bench.profile_traffic("mla_decode_v3_b64_ctx8k.md", applies=False) == (None, None)
    assert bench.profile_traffic("no_such_summary.md") == (None, None)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr
