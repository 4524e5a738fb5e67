"""The decode entry point that allocates nothing (mla_decode_bf16_static: split-KV partials in a device array built into the
library) gives the bytes mla_decode_bf16 gives with a caller-owned workspace: two calls in a row through the C-ABI, the
second on a smaller input (the array keeps the first call's contents), then a shape beyond the array's size is refused."""
import ctypes

import pytest
import torch

from oracle import mla_oracle as O

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _decode_both(lib, dev, batch, heads, lo, hi, seed, splits):
    c = O.make_decode_case(batch, heads, lo, hi, seed=seed)
    g = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    qn, qr, nope, rope, bt, sl = (g[k] for k in ("q_nope", "q_rope", "nope", "rope", "block_table", "seq_lens"))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = [_ptr(qn), qn.stride(0), qn.stride(1), _ptr(qr), qr.stride(0), qr.stride(1),
              _ptr(nope), nope.stride(0), nope.stride(1), _ptr(rope), rope.stride(0), rope.stride(1), nope.shape[0],
              _ptr(bt), bt.stride(0), bt.shape[1], _ptr(sl), None, batch, 1, heads, float(c["scale"])]
    outs = []
    for static in (False, True):
        out = torch.full((batch, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device=dev)
        tail = [_ptr(out), out.stride(0), out.stride(1), _ptr(lse)]
        if static:
            rc = lib.mla_decode_bf16_static(*common, *tail, splits, stream)
        else:
            need = lib.mla_decode_workspace_bytes(batch, 1, heads, splits)
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
            rc = lib.mla_decode_bf16(*common, *tail, _ptr(ws), need, splits, stream)
        assert rc == 0, lib.mlahip_last_error_string()
        torch.cuda.synchronize()
        outs.append((out.cpu(), lse.cpu()))
    ref = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    return outs, ref


def test_static_scratch_decode_equals_the_workspace_decode(dev):
    from omni_npu_amd import _lib
    lib = _lib.load()
    # first call: 8 sequences x 128 heads, 3 splits; second call: smaller in every respect, over the first call's leftovers
    for batch, heads, lo, hi, seed, splits in ((8, 128, 700, 1500, 21, 3), (3, 16, 40, 300, 22, 2)):
        (with_ws, static), ref = _decode_both(lib, dev, batch, heads, lo, hi, seed, splits)
        assert torch.isfinite(static[0].float()).all() and torch.isfinite(static[1]).all()
        assert torch.equal(static[0].view(torch.int16), with_ws[0].view(torch.int16)), "outputs differ bit for bit"
        assert torch.equal(static[1], with_ws[1]), "log-sum-exps differ"
        assert (static[0].float() - ref).abs().max().item() <= 2e-2          # and both are right (bf16 bar of the decode tests)


def test_static_scratch_decode_refuses_what_does_not_fit(dev):
    from omni_npu_amd import _lib
    lib = _lib.load()
    batch, heads, q_len, splits = 256, 128, 2, 1                             # 136 MB of partials
    assert lib.mla_decode_workspace_bytes(batch, q_len, heads, splits) > (48 << 20)
    t = torch.zeros(64, dtype=torch.uint8, device=dev)
    p = _ptr(t)
    rc = lib.mla_decode_bf16_static(p, 512, 512, p, 64, 64, p, 65536, 512, p, 8192, 64, 1, p, 1, 1, p, None, batch, q_len, heads,
                                    0.1, p, 512, 512, None, splits, None)
    assert rc == -4 and b"built-in array" in lib.mlahip_last_error_string()


def test_static_scratch_decode_allocates_nothing_and_replays_from_a_graph(dev):
    """After one warm-up call outside capture (address lookup, LDS limit) a call moves neither the device's free memory
    nor the torch allocator's counters, and a call recorded into a HIP graph replays to the eager bytes every time, with
    the program's own eager work between the replays."""
    from omni_npu_amd import _lib
    lib = _lib.load()
    batch, heads, splits = 6, 128, 3
    c = O.make_decode_case(batch, heads, 300, 1200, seed=23)
    g = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in c.items()}
    qn, qr, nope, rope, bt, sl = (g[k] for k in ("q_nope", "q_rope", "nope", "rope", "block_table", "seq_lens"))
    out = torch.zeros(batch, heads, 512, dtype=torch.bfloat16, device=dev)
    lse = torch.zeros(batch, heads, dtype=torch.float32, device=dev)

    def call(splits=splits):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.mla_decode_bf16_static(_ptr(qn), qn.stride(0), qn.stride(1), _ptr(qr), qr.stride(0), qr.stride(1),
                                        _ptr(nope), nope.stride(0), nope.stride(1), _ptr(rope), rope.stride(0), rope.stride(1),
                                        nope.shape[0], _ptr(bt), bt.stride(0), bt.shape[1], _ptr(sl), None, batch, 1, heads,
                                        float(c["scale"]), _ptr(out), out.stride(0), out.stride(1), _ptr(lse), splits, stream)
        assert rc == 0, lib.mlahip_last_error_string()

    call()                                                    # warm-up outside capture
    torch.cuda.synchronize()
    free0, stats0 = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_stats(dev)
    call()
    torch.cuda.synchronize()
    free1, stats1 = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_stats(dev)
    assert free1 == free0, f"device free memory moved by {free0 - free1} bytes across a call"
    for k in ("allocation.all.allocated", "allocated_bytes.all.allocated", "segment.all.allocated", "reserved_bytes.all.allocated"):
        assert stats1[k] == stats0[k], k
    eager = (out.clone(), lse.clone())
    ref = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    assert (eager[0].float().cpu() - ref).abs().max().item() <= 2e-2

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        # eager work of the program between the replays: another static call on other lengths, then the outputs cleared
        sl.copy_((c["seq_lens"] // 2).to(dev))
        call()
        sl.copy_(c["seq_lens"].to(dev))
        out.zero_()
        lse.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager[0].view(torch.int16)), f"replay {rep}: output differs from eager"
        assert torch.equal(lse, eager[1]), f"replay {rep}: log-sum-exp differs from eager"

    # A launch with many more chunks takes another form of the split kernel (groups of 128 rows instead of 32), one that
    # this process may never have launched: the first static call has prepared every form, so this one is captured cold.
    many = 24
    assert lib.mla_decode_workspace_bytes(batch, 1, heads, many) <= (48 << 20)
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2):
        call(many)
    out.zero_()
    lse.zero_()
    graph2.replay()
    torch.cuda.synchronize()
    assert (out.float().cpu() - ref).abs().max().item() <= 2e-2
    assert torch.allclose(lse, eager[1], atol=1e-4, rtol=0)

