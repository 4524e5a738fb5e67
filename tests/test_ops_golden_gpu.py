"""The GPU merges and the gather against the vectors written by the reference's own torch implementations
(tests/golden/ops_vectors.npz), and the split-KV reduce fed hand-made partials (the N-way merge of
src/omni_npu/attention/ops.py:109-141 in the workspace layout of the decode kernels)."""
import ctypes

import pytest
import torch

from oracle import mla_oracle as O
from tests.test_ops_golden import gather_caches, same_with_inf, t

pytestmark = pytest.mark.gpu


def test_merge_states_kernel_matches_the_reference_vectors(dev):
    from omni_npu_amd import kernels as K
    from omni_npu_amd.attention import ops
    po, so = t("merge_prefix_out", torch.bfloat16).to(dev), t("merge_suffix_out", torch.bfloat16).to(dev)
    pl, sl = t("merge_prefix_lse").to(dev), t("merge_suffix_lse").to(dev)
    out = torch.full(po.shape, float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full(pl.shape, float("nan"), dtype=torch.float32, device=dev)
    ops.merge_attn_states(out, po, pl, so, sl, lse)           # the reference's own signature
    assert torch.allclose(out.cpu(), t("merge_out"), atol=2e-6, rtol=2e-6)
    assert same_with_inf(lse.cpu(), t("merge_out_lse"), 2e-6)
    out16 = torch.empty(po.shape, dtype=torch.bfloat16, device=dev)
    K.merge_states(po, pl, so, sl, out16)
    assert torch.equal(out16.cpu(), t("merge_out").bfloat16())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_attention_update_is_one_launch_and_matches_the_reference_vectors(dev, dtype):
    from omni_npu_amd.attention import ops
    outs, lses = t("update_outs").to(dtype), t("update_lses")
    ref_out, ref_lse = (t("update_out"), t("update_lse")) if dtype != torch.bfloat16 else O.attention_update(outs, lses)
    out, lse = ops.attention_update_torch(outs.to(dev), lses.to(dev))
    assert out.dtype == torch.float32 and out.shape == ref_out.shape and lse.shape == ref_lse.shape
    assert torch.allclose(out.cpu(), ref_out, atol=2e-6, rtol=2e-6)
    assert same_with_inf(lse.cpu(), ref_lse, 2e-6)
    # the list form of the reference
    out2, lse2 = ops.attention_update_torch([o for o in outs.to(dev)], [l for l in lses.to(dev)])
    assert torch.equal(out2, out) and torch.equal(lse2.isfinite(), lse.isfinite())
    # garbage behind a weightless partial does not leak
    bad = outs.clone()
    bad[1:, 4] = float("nan")                                 # row 4: only partial 0 is alive
    out3, _ = ops.attention_update_torch(bad.to(dev), lses.to(dev))
    assert torch.equal(out3[4].cpu(), out[4].cpu())


def test_gather_kernel_matches_the_reference_vector(dev):
    from omni_npu_amd import kernels as K
    nope, rope = gather_caches()
    cu = t("gather_cu")
    dst = torch.full((int(cu[-1]), 576), -7.0, dtype=torch.bfloat16, device=dev)
    K.gather_paged(nope.to(dev), rope.to(dev), dst, t("gather_block_table").to(dev), cu.to(dev), 3,
                   seq_starts=t("gather_seq_starts").to(dev))
    assert torch.equal(dst.float().cpu(), t("gather_dst"))


def _plan(seq_lens, splits):
    """Which (chunk, sequence) pairs hold 32-key blocks, as the split kernels cut the work: partial number = chunk + b."""
    units = [((l + 31) // 32 + 8) if l > 0 else 0 for l in seq_lens]
    tot, g = sum(units), len(seq_lens) * splits
    start, parts = 0, []
    for b, u in enumerate(units):
        mine = []
        for c in range(g):
            cb, ce = c * tot // g, (c + 1) * tot // g
            lo, hi = max(cb, start), min(ce, start + u)
            if max(hi - start - 8, 0) > max(lo - start - 8, 0):
                mine.append(c + b)
        parts.append(mine)
        start += u
    return parts


def test_splitkv_reduce_on_hand_made_partials(dev):
    """mla_splitkv_reduce merges exactly the partials the plan names, with the conventions of attention_update_torch:
    +inf reads as -inf, a row without weight gives zeros and -inf."""
    from omni_npu_amd import _lib
    lib = _lib.load()
    seq_lens, splits, heads = [700, 1200, 0, 40], 3, 4
    batch, r_max = len(seq_lens), heads
    parts = _plan(seq_lens, splits)
    assert len(parts[0]) >= 3 and len(parts[1]) >= 2 and parts[2] == [] and len(parts[3]) >= 1
    assert _plan([700, 1200], 3) == [[0, 1, 2], [4, 5, 6]]     # (worked by hand: 76 units in 6 chunks)
    slots = batch * (splits + 1)
    rows = slots * r_max
    need = lib.mla_decode_workspace_bytes(batch, 1, heads, splits)
    assert need == rows * (1024 + 16) + batch * 8
    g = torch.Generator().manual_seed(99)
    o_part = torch.randn(slots, r_max, 512, generator=g).half()
    lse_part = torch.randn(slots, r_max, generator=g) * 3
    inf = float("inf")
    lse_part[parts[0][1], 0] = inf                            # +inf reads as -inf
    for j, sl_ in enumerate(parts[0]):
        lse_part[sl_, 1] = inf if j == 1 else -inf              # a row with no weight at all
    lse_part[parts[1][0], 2] = -inf
    o_part[parts[1][0], 2] = float("nan")                     # garbage behind a weightless partial
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    ws[: rows * 1024] = o_part.view(torch.uint8).flatten().to(dev)
    ws[rows * 1024: rows * 1028] = lse_part.view(torch.uint8).flatten().to(dev)
    # correction factors stay zero (no dominant-key record); their row pointers must still be readable addresses
    ptrs = torch.full((rows,), ws.data_ptr(), dtype=torch.int64)
    ws[rows * 1032: rows * 1040] = ptrs.view(torch.uint8).flatten().to(dev)
    seg = torch.zeros(batch, 2, dtype=torch.int32)
    for b, mine in enumerate(parts):
        if mine:
            seg[b, 0], seg[b, 1] = mine[0], mine[-1]
    ws[rows * 1040: rows * 1040 + batch * 8] = seg.view(torch.uint8).flatten().to(dev)
    sl = torch.tensor(seq_lens, dtype=torch.int32, device=dev)
    out = torch.full((batch, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device=dev)
    rc = lib.mla_splitkv_reduce(ws.data_ptr(), need, sl.data_ptr(), None, batch, 1, heads, splits, out.data_ptr(), out.stride(0),
                                out.stride(1), lse.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.mlahip_last_error_string()
    torch.cuda.synchronize()
    for b, mine in enumerate(parts):
        if not mine:                                          # an empty sequence: zeros and -inf
            assert (out[b].float() == 0).all() and (lse[b] == -inf).all()
            continue
        ref_o, ref_l = O.attention_update(torch.nan_to_num(o_part[mine].float()), lse_part[mine])
        assert torch.allclose(out[b].float().cpu(), ref_o, atol=2e-2, rtol=2 ** -7), b
        assert same_with_inf(lse[b].cpu(), ref_l, 1e-5), b
    assert (out[0, 1].float() == 0).all() and lse[0, 1] == -inf
