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


def test_parity_fields_and_the_exit_status_they_drive(capsys):
    """Every workload's comparison with the oracle carries the bar of its cache type and whether it was met; a missed bar, also in a
    secondary workload, turns into exit status 1 after the JSON line is out."""
    import json

    import pytest
    import torch
    sys.path.insert(0, ROOT)
    import bench
    ref = torch.ones(4, 8)
    ok = bench.parity_fields(torch.full((4, 8), 1.5e-3), ref, "bf16", pair=[1, 5])
    assert ok["parity_ok"] and ok["bar"] == {"max_abs": 2e-2, "mean_rel": 2e-3} and ok["pair"] == [1, 5]
    assert not bench.parity_fields(torch.full((4, 8), 2.2e-3), ref, "bf16")["parity_ok"]          # mean-rel over the bar
    spike = torch.zeros(4, 8)
    spike[0, 0] = 3e-2
    assert not bench.parity_fields(spike, ref, "bf16")["parity_ok"]                                # max-abs over the bar
    assert bench.parity_fields(torch.full((4, 8), 5e-3), ref, "fp8")["parity_ok"]
    bench.finish({"value": 1.0, "parity_ok": True, "secondary": {"configs[2]": {"parity_ok": True}}})
    assert json.loads(capsys.readouterr().out)["value"] == 1.0
    for res in ({"value": 1.0, "parity_ok": False},
                {"value": 1.0, "parity_ok": True, "secondary": {"configs[2]": {"parity_ok": False}}}):
        with pytest.raises(SystemExit) as e:
            bench.finish(res)
        assert e.value.code == 1
        out = capsys.readouterr()
        assert json.loads(out.out)["value"] == 1.0 and "parity bar missed" in out.err
