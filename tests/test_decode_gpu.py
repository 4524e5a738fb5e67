"""Parity of the HIP absorbed-MLA paged decode (through the C-ABI) against the CPU oracle.

Tolerance (bf16 cache): max-abs 2e-2, mean-rel 2e-3 against the fp32 oracle.
"""
import math

import pytest
import torch

from oracle import mla_oracle as O
from tests.conftest import attn_close

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_REL = 2e-2, 2e-3


def _run(case, dev, num_splits=None, head_major=False, with_lse=False):
    from omni_npu_amd import kernels as K
    q_nope, q_rope = case["q_nope"].to(dev), case["q_rope"].to(dev)
    nope, rope = case["nope"].to(dev), case["rope"].to(dev)
    bt, sl = case["block_table"].to(dev), case["seq_lens"].to(dev)
    t, n, _ = q_nope.shape
    if head_major:
        buf = torch.full((n, t, 512), float("nan"), dtype=torch.bfloat16, device=dev)
        out = buf.transpose(0, 1)
    else:
        buf = out = torch.full((t, n, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.empty(t, n, dtype=torch.float32, device=dev) if with_lse else None
    K.decode(q_nope, q_rope, nope, rope, bt, sl, case["scale"], out, q_len=case["q_len"], lse_out=lse,
             num_splits=num_splits)
    torch.cuda.synchronize()
    return buf, lse


@pytest.mark.parametrize("num_splits", [1, 3, None])
def test_decode_config1_plumbing(dev, num_splits):
    """16 heads, batch 4, lens in [128,1024], shuffled block tables."""
    case = O.make_decode_case(4, 16, 128, 1024, seed=0)
    ref, ref_lse = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                                     case["seq_lens"], case["scale"], return_lse=True)
    got, lse = _run(case, dev, num_splits, with_lse=True)
    attn_close(got, ref, MAX_ABS, MEAN_REL)
    assert torch.allclose(lse.cpu(), ref_lse, atol=2e-2, rtol=0)


@pytest.mark.parametrize("heads,num_splits", [(16, 1), (16, 3), (64, 2)])
def test_small_forms_leave_no_dominant_key_records(dev, heads, num_splits):
    """With at most 64 query rows per request every probability goes through P.V as two bf16 numbers (value and rounding
    remainder), so there is nothing for the merge phase to add back: the correction factors stay zero, and the result is
    the output rounding away from the oracle."""
    from omni_npu_amd import kernels as K
    from omni_npu_amd import _lib
    case = O.make_decode_case(4, heads, 128, 1024, seed=0)
    b, n = 4, heads
    ws = torch.zeros(_lib.load().mla_decode_workspace_bytes(b, 1, n, num_splits), dtype=torch.uint8, device=dev)
    out = torch.empty(b, n, 512, dtype=torch.bfloat16, device=dev)
    K.decode(case["q_nope"].to(dev), case["q_rope"].to(dev), case["nope"].to(dev), case["rope"].to(dev),
             case["block_table"].to(dev), case["seq_lens"].to(dev), case["scale"], out, q_len=1, num_splits=num_splits,
             workspace=ws)
    torch.cuda.synchronize()
    rows = b * (num_splits + 1) * n
    off = rows * 512 * 2 + rows * 4
    assert not ws.cpu()[off:off + rows * 4].view(torch.float32).any()
    ref = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"])
    ma, mr = attn_close(out, ref, MAX_ABS, MEAN_REL)
    assert mr <= 1.6e-3, mr


@pytest.mark.parametrize("heads,num_splits", [(128, 1), (128, 2), (128, 3)])
def test_decode_dominant_key_records_name_the_right_cache_row(dev, heads, num_splits):
    """The split phase leaves, per partial row, the cache row of the chunk's most probable key when that key carries more
    than 1/16 of the chunk's weight (the merge phase takes the bf16 rounding of that probability out again).  A record
    that names another key of the same 32-key block still passes the attention tolerance most of the time, so the
    records are checked directly: every recorded row must be the most probable key of its head within its 32-key block
    (chunks are cut at multiples of 32 keys, so blocks are 32-aligned within the sequence), and keys with more than 1/8 of their whole
    row's weight must be recorded."""
    from omni_npu_amd import kernels as K
    from omni_npu_amd import _lib
    b, n = 256 // (2 * num_splits) + 2, heads            # enough chunks that the launch takes the 128-row form, which is
    case = O.make_decode_case(b, heads, 128, 1024, seed=0)  # the one that leaves records (fewer: the rows are cut instead)
    nope = case["nope"].to(dev)
    ws = torch.zeros(_lib.load().mla_decode_workspace_bytes(b, 1, n, num_splits), dtype=torch.uint8, device=dev)
    out = torch.empty(b, n, 512, dtype=torch.bfloat16, device=dev)
    K.decode(case["q_nope"].to(dev), case["q_rope"].to(dev), nope, case["rope"].to(dev), case["block_table"].to(dev),
             case["seq_lens"].to(dev), case["scale"], out, q_len=1, num_splits=num_splits, workspace=ws)
    torch.cuda.synchronize()
    rows = b * (num_splits + 1) * n                      # partial rows: fp16 outputs, then lse, scale, row address
    w = ws.cpu()
    off = rows * 512 * 2 + rows * 4
    corr_scale = w[off:off + rows * 4].view(torch.float32)
    corr_row = w[off + rows * 4:off + rows * 12].view(torch.int64)
    row_bytes = nope.stride(-2) * 2
    recorded = {}                                        # (cache slot, head) of every record
    for i in torch.nonzero(corr_scale).flatten().tolist():
        delta = int(corr_row[i]) - nope.data_ptr()
        assert delta % row_bytes == 0 and 0 <= delta // row_bytes < nope.shape[0] * nope.shape[1]
        recorded[(delta // row_bytes, i % n)] = i
    assert len(recorded) >= 8                            # the case has peaked rows; an empty set would test nothing
    checked = expected = found = 0
    for s in range(b):
        L = int(case["seq_lens"][s])
        slots = O.slots_for(case["block_table"], s, 0, L)
        kn = case["nope"].view(-1, 512)[slots].float()
        kr = case["rope"].view(-1, 64)[slots].float()
        sc = (case["q_nope"][s].float() @ kn.T + case["q_rope"][s].float() @ kr.T) * case["scale"]
        p = torch.softmax(sc, -1)
        pos_of = {int(v): t for t, v in enumerate(slots.tolist())}
        for (slot, h), i in recorded.items():
            if slot not in pos_of:
                continue
            t = pos_of[slot]
            blk = p[h, (t // 32) * 32:min(L, (t // 32) * 32 + 32)]
            assert p[h, t] >= blk.max() * (1 - 1e-4), (s, h, t, int(blk.argmax()) + (t // 32) * 32)
            checked += 1
        top = p.argmax(-1)
        for h in range(n):
            if p[h, top[h]] > 1 / 8:
                expected += 1
                found += (int(slots[top[h]]), h) in recorded
    assert checked == len(recorded)                      # every record points into one of the four sequences
    # A dominant key in the first 32-key block of its chunk has probability exactly 1 against that block's reference
    # maximum, which bf16 holds exactly: its correction is zero and reads as "no record".  That is about one block in
    # ten here; anything beyond that would be records getting lost.
    assert expected >= 8 and found >= 0.8 * expected, (found, expected)


@pytest.mark.parametrize("lens", [(1, 1), (1, 70), (63, 65), (127, 129), (200, 300)])
def test_decode_ragged_edges(dev, lens):
    """Sequence lengths around tile (64) and page (128) boundaries, 128 heads, head-major output."""
    case = O.make_decode_case(5, 128, lens[0], lens[1], seed=3)
    ref = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"])
    got, _ = _run(case, dev, num_splits=2, head_major=True)
    attn_close(got.transpose(0, 1), ref, MAX_ABS, MEAN_REL)


@pytest.mark.parametrize("batch,heads,q_len,lo,hi,splits", [(1, 128, 1, 9000, 9000, 200), (2, 16, 2, 3000, 7000, 40),
                                                            (1, 128, 1, 20000, 20000, None), (3, 128, 1, 50, 400, 24),
                                                            (2, 128, 2, 1, 5000, 13)])
def test_decode_many_partials_per_sequence(dev, batch, heads, q_len, lo, hi, splits):
    """Few sequences and long contexts: dozens to hundreds of partials per row, merged by a workgroup per row (four
    wavefronts, every fourth partial each); the fourth case has more chunks than work units, so some chunks are empty
    and the partial list is found by testing chunk by chunk."""
    case = O.make_decode_case(batch, heads, lo, hi, seed=21 + batch, q_len=q_len)
    ref, ref_lse = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                                     case["seq_lens"], case["scale"], return_lse=True)
    got, lse = _run(case, dev, splits, with_lse=True)
    attn_close(got, ref, MAX_ABS, MEAN_REL)
    assert torch.allclose(lse.cpu(), ref_lse, atol=2e-2, rtol=0)


@pytest.mark.parametrize("batch,heads,q_len,lo,hi", [(130, 128, 1, 1, 300), (70, 128, 2, 2, 260)])
def test_decode_large_batch_one_chunk_per_sequence(dev, batch, heads, q_len, lo, hi):
    """More than 16384 query rows and one chunk per sequence: every row has one partial, or two where a chunk border
    falls inside its sequence, and the merge runs four rows per wavefront."""
    case = O.make_decode_case(batch, heads, lo, hi, seed=batch, q_len=q_len)
    ref, ref_lse = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                                     case["seq_lens"], case["scale"], return_lse=True)
    got, lse = _run(case, dev, 1, with_lse=True)
    attn_close(got, ref, MAX_ABS, MEAN_REL)
    assert torch.allclose(lse.cpu(), ref_lse, atol=2e-2, rtol=0)


def test_decode_single_key_returns_the_row(dev):
    """L = 1: softmax over one key is 1, the output is that latent row exactly (in bf16)."""
    case = O.make_decode_case(3, 128, 1, 1, seed=5)
    got, _ = _run(case, dev, num_splits=1)
    for b in range(3):
        row = case["nope"][case["block_table"][b, 0].long(), 0]
        assert torch.equal(got[b].cpu(), row.view(1, -1).expand(128, -1))


def _plant(case, b, pos, head, gain):
    """Overwrite the latent row of key `pos` of sequence b with gain * (query of `head`): its score for that head jumps
    by about gain * |q|^2 * scale ~ 37 * gain (natural units), far beyond anything N(0,1) data produces."""
    page = case["block_table"][b, pos // 128].long()
    case["nope"][page, pos % 128] = (gain * case["q_nope"][b * case["q_len"], head].float()).bfloat16()


@pytest.mark.parametrize("heads", [128, 16, 48])
@pytest.mark.parametrize("num_splits", [1, 4])
def test_decode_scores_that_outgrow_the_first_block(dev, num_splits, heads):
    """The kernel fixes each row's softmax reference at its first block and restarts a segment when a later score exceeds
    it by more than 2^100: keys planted late in the sequences with scores ~110 and ~220 (natural units) above the
    rest exercise one and two restarts, a planted key in the very first block exercises a reference that is already
    the maximum, and a moderately dominant key (weight ~0.5) exercises the correction of the dominant probability.
    16 and 48 heads take the kernel forms for at most 32 / 64 query rows, where some wavefronts own no rows."""
    case = O.make_decode_case(4, heads, 1500, 2500, seed=21)
    lens = case["seq_lens"].tolist()
    _plant(case, 0, lens[0] - 40, 3, 3.0)                      # one restart, late in the last chunk
    _plant(case, 1, 700, 5, 3.0)
    _plant(case, 1, 1400, 5, 6.0)                              # two restarts for head 5 of sequence 1
    _plant(case, 2, 7, 9, 4.0)                                 # the maximum sits in the first block
    _plant(case, 3, 900, 11, 0.17)                             # about e^6 above the crowd: weight of the order of 0.5
    ref = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"])
    got, _ = _run(case, dev, num_splits)
    got = got.float().cpu()
    # the planted rows dominate their heads completely: the output is that latent row (values up to ~25, so the bf16
    # rounding of the output alone exceeds the absolute bar: these three (sequence, head) pairs are checked relatively)
    for b, pos, head in ((0, lens[0] - 40, 3), (1, 1400, 5), (2, 7, 9)):
        row = case["nope"][case["block_table"][b, pos // 128].long(), pos % 128].float()
        assert (got[b, head] - row).abs().max().item() <= 2 ** -8 * row.abs().max().item()
        assert (ref[b, head] - row).abs().max().item() <= 1e-3 * row.abs().max().item()
    # the planted rows hold values up to ~25 and leak into other heads of their sequences, so the absolute bar is scaled by
    # the magnitude of each output row (it is the unchanged 2e-2 wherever the outputs are of order one)
    err = (got - ref).abs()
    bar = MAX_ABS * ref.abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    assert (err <= bar).all(), f"worst excess {(err / bar).max().item():.3f} x the bar"
    assert (err.sum() / ref.abs().sum()).item() <= MEAN_REL


def test_decode_empty_and_tiny_sequences_in_one_batch(dev):
    """Lengths 0, 1, 31, 32, 33 and a long one side by side: empty sequences give zeros and lse = -inf, and the balanced
    chunk plan (more chunks than blocks for most of these) must still route every partial."""
    case = O.make_decode_case(6, 128, 1, 1, seed=8)
    big = O.make_decode_case(1, 128, 3000, 3000, seed=9)
    lens = [0, 1, 31, 32, 33, 3000]
    pages = sum((l + 127) // 128 for l in lens) + 1
    g = torch.Generator().manual_seed(10)
    case["nope"] = torch.randn(pages, 128, 512, generator=g).bfloat16()
    case["rope"] = torch.randn(pages, 128, 64, generator=g).bfloat16()
    bt = torch.zeros(6, (3000 + 127) // 128, dtype=torch.int32)
    perm = torch.randperm(pages, generator=g).tolist()
    for b, l in enumerate(lens):
        for j in range((l + 127) // 128):
            bt[b, j] = perm.pop()
    case["block_table"], case["seq_lens"] = bt, torch.tensor(lens, dtype=torch.int32)
    ref, ref_lse = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], bt, case["seq_lens"],
                                     case["scale"], return_lse=True)
    for splits in (1, 3):
        got, lse = _run(case, dev, splits, with_lse=True)
        assert (got[0].float() == 0).all() and torch.isinf(lse[0]).all() and (lse[0] < 0).all()
        attn_close(got[1:], ref[1:], MAX_ABS, MEAN_REL)
        assert torch.allclose(lse[1:].cpu(), ref_lse[1:], atol=2e-2, rtol=0)


def test_decode_row_groups_renumbered_onto_one_xcd(dev):
    """256 query rows per sequence (two row groups) and a chunk count that is a multiple of eight: the kernel renumbers
    its workgroups so that the groups of a chunk share an XCD; results must not change."""
    case = O.make_decode_case(4, 128, 200, 900, seed=13, q_len=2)
    ref = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"])
    for splits in (2, 4):                                     # 8 and 16 chunks
        got, _ = _run(case, dev, num_splits=splits)
        attn_close(got, ref, MAX_ABS, MEAN_REL)
    got3, _ = _run(case, dev, num_splits=3)                   # 12 chunks: launch order kept
    got2, _ = _run(case, dev, num_splits=2)
    assert (got3.float() - got2.float()).abs().max().item() <= 8e-3


@pytest.mark.parametrize("q_len,heads", [(2, 128), (3, 16), (2, 40)])
def test_decode_mtp_right_down_causal(dev, q_len, heads):
    """q_len > 1: token i of a request sees keys [0, L - q_len + i]."""
    case = O.make_decode_case(4, heads, 130, 600, seed=7, q_len=q_len)
    ref = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"])
    got, _ = _run(case, dev, num_splits=3)
    attn_close(got, ref, MAX_ABS, MEAN_REL)


def test_decode_varlen_query_start_loc(dev):
    from omni_npu_amd import kernels as K
    case = O.make_decode_case(3, 16, 100, 400, seed=9, q_len=3)
    qsl = [0, 3, 4, 6]                                  # request lengths 3, 1, 2 (tokens 0..5 used)
    ref = O.absorbed_decode(case["q_nope"][:6], case["q_rope"][:6], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"], query_start_loc=qsl)
    out = torch.zeros(6, 16, 512, dtype=torch.bfloat16, device=dev)
    K.decode(case["q_nope"][:6].to(dev), case["q_rope"][:6].to(dev), case["nope"].to(dev), case["rope"].to(dev),
             case["block_table"].to(dev), case["seq_lens"].to(dev), case["scale"], out, q_len=3,
             query_start_loc=torch.tensor(qsl, dtype=torch.int32, device=dev), num_splits=2)
    attn_close(out, ref, MAX_ABS, MEAN_REL)


def test_decode_strided_q_views(dev):
    """q_rope as a slice of a wider q tensor, as the reference passes it (mla.py:902-904)."""
    from omni_npu_amd import kernels as K
    case = O.make_decode_case(4, 32, 64, 512, seed=11)
    ref = O.absorbed_decode(case["q_nope"], case["q_rope"], case["nope"], case["rope"], case["block_table"],
                            case["seq_lens"], case["scale"])
    q = torch.zeros(4, 32, 192, dtype=torch.bfloat16, device=dev)
    q[..., 128:] = case["q_rope"].to(dev)
    ql = case["q_nope"].to(dev).transpose(0, 1).contiguous().transpose(0, 1)     # [T,N,512] view of [N,T,512]
    out = torch.zeros(4, 32, 512, dtype=torch.bfloat16, device=dev)
    K.decode(ql, q[..., 128:], case["nope"].to(dev), case["rope"].to(dev), case["block_table"].to(dev),
             case["seq_lens"].to(dev), case["scale"], out)
    attn_close(out, ref, MAX_ABS, MEAN_REL)


def test_decode_headline_shape_properties(dev):
    """128 heads, batch 64, lens in [4096,8192]: a sample of sequences against the oracle, and invariance of
    the whole output under the split count and under a re-shuffle of the physical pages."""
    from omni_npu_amd import kernels as K
    case = O.make_decode_case(64, 128, 4096, 8192, seed=0)
    got8, _ = _run(case, dev, num_splits=8)
    got5, _ = _run(case, dev, num_splits=5)
    assert (got8.float() - got5.float()).abs().max().item() <= 8e-3
    for b in (0, 17, 63):
        sub = dict(case)
        ref = O.absorbed_decode(case["q_nope"][b:b + 1], case["q_rope"][b:b + 1], case["nope"], case["rope"],
                                case["block_table"][b:b + 1], case["seq_lens"][b:b + 1], case["scale"])
        attn_close(got8[b:b + 1], ref, MAX_ABS, MEAN_REL)
    # physical page permutation: move every page, rewrite the tables, same answer bit for bit
    nblk = case["nope"].shape[0]
    perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nblk)
    c2 = dict(case)
    c2["nope"], c2["rope"] = case["nope"][perm], case["rope"][perm]
    c2["block_table"] = inv[case["block_table"].long()].to(torch.int32)
    got_perm, _ = _run(c2, dev, num_splits=8)
    assert torch.equal(got_perm, got8)


def test_decode_step_with_many_partials_replayed_from_a_hip_graph(dev):
    """Cache write + decode of two long sequences (dozens of chunks each, merged by a workgroup per row) captured once and
    replayed with new lengths, slots, queries and rows written into the same device buffers; eager work runs between the
    replays, every replay must equal the eager step bit for bit, and the eager step must match the oracle."""
    from omni_npu_amd import kernels as K
    batch, heads = 2, 128
    c = O.make_decode_case(batch, heads, 5000, 9000, seed=77)
    qn, qr = c["q_nope"].to(dev), c["q_rope"].to(dev)
    nope, rope = c["nope"].to(dev), c["rope"].to(dev)
    new_c, new_r = c["new_c"].to(dev), c["new_r"].to(dev)
    lens, slots, bt = c["seq_lens"].to(dev), c["slot_mapping"].to(dev), c["block_table"].to(dev)
    out = torch.empty(batch, heads, 512, dtype=torch.bfloat16, device=dev)
    max_len = bt.shape[1] * 128
    splits = K.default_num_splits(batch, 1, heads, max_len)
    assert splits + 1 > 12                                    # enough partials per row for the workgroup-per-row merge
    ws = torch.empty(K._lib.load().mla_decode_workspace_bytes(batch, 1, heads, splits), dtype=torch.uint8, device=dev)

    def step():
        K.cache_write(new_c, new_r, slots, nope, rope)
        K.decode(qn, qr, nope, rope, bt, lens, c["scale"], out, num_splits=splits, workspace=ws, max_seq_len=max_len)

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    ref_nope, ref_rope = c["nope"].clone(), c["rope"].clone()
    O.cache_write(ref_nope, c["slot_mapping"], c["new_c"])   # the warm-up step wrote the case's own new rows
    O.cache_write(ref_rope, c["slot_mapping"], c["new_r"])
    for trial in range(3):
        g = torch.Generator().manual_seed(200 + trial)
        new_lens = (c["seq_lens"] - torch.randint(0, 3000, (batch,), generator=g).to(torch.int32)).clamp_min(1)
        sl = torch.cat([O.slots_for(c["block_table"], b, int(new_lens[b]) - 1, int(new_lens[b])) for b in range(batch)])
        q1 = torch.randn(batch, heads, 512, generator=g).bfloat16()
        r1 = torch.randn(batch, 512, generator=g).bfloat16()
        lens.copy_(new_lens.to(dev)); slots.copy_(sl.to(dev)); qn.copy_(q1.to(dev)); new_c.copy_(r1.to(dev))
        before_n, before_r = nope.clone(), rope.clone()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        nope.copy_(before_n); rope.copy_(before_r)
        out.zero_()
        step()
        torch.cuda.synchronize()
        assert torch.equal(got, out), f"replay {trial} differs from the eager step"
        O.cache_write(ref_nope, sl, r1)
        O.cache_write(ref_rope, sl, c["new_r"])
        ref = O.absorbed_decode(q1, c["q_rope"], ref_nope, ref_rope, c["block_table"], new_lens, c["scale"])
        attn_close(got, ref, MAX_ABS, MEAN_REL)


@pytest.mark.parametrize("batch,heads,q_len,lo,hi,splits", [
    (5, 128, 1, 100, 900, 3), (4, 128, 2, 31, 700, 2), (3, 128, 4, 30, 40, 1), (6, 16, 1, 60, 500, 2), (3, 40, 2, 64, 66, 5),
    (2, 128, 3, 1025, 1100, 4), (7, 8, 2, 2, 300, None),
])
def test_decode_step_with_the_cache_write_folded_in_equals_the_two_launches(dev, batch, heads, q_len, lo, hi, splits):
    """mla_decode_bf16_step (the new tokens' rows stored by the split kernel's workgroups before they read) leaves the
    caches and the output exactly as mla_cache_write_bf16 followed by mla_decode_bf16 does: query tokens whose keys
    straddle block and chunk borders, padded slots, ragged query lengths."""
    from omni_npu_amd import kernels as K
    c = O.make_decode_case(batch, heads, lo, hi, seed=77 + batch, q_len=q_len)
    t = batch * q_len
    slots = c["slot_mapping"].clone()
    if batch > 3:
        slots[q_len * 2] = -1                                  # a padded slot: that row is not written by either path
    outs, caches = [], []
    for fused in (False, True):
        nope, rope = c["nope"].to(dev), c["rope"].to(dev)
        out = torch.full((t, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full((t, heads), float("nan"), dtype=torch.float32, device=dev)
        args = [c[k].to(dev) for k in ("q_nope", "q_rope")] + [nope, rope, c["block_table"].to(dev), c["seq_lens"].to(dev)]
        new = (c["new_c"].to(dev), c["new_r"].to(dev), slots.to(dev))
        if fused:
            K.decode(*args, c["scale"], out, q_len=q_len, num_splits=splits, lse_out=lse, new_rows=new)
        else:
            K.cache_write(new[0], new[1], new[2], nope, rope)
            K.decode(*args, c["scale"], out, q_len=q_len, num_splits=splits, lse_out=lse)
        torch.cuda.synchronize()
        outs.append((out.cpu(), lse.cpu()))
        caches.append((nope.cpu(), rope.cpu()))
    assert torch.equal(caches[0][0].view(torch.int16), caches[1][0].view(torch.int16)), "latent cache differs"
    assert torch.equal(caches[0][1].view(torch.int16), caches[1][1].view(torch.int16)), "rope cache differs"
    assert not torch.equal(caches[1][0], c["nope"])           # (and rows were written at all)
    assert torch.equal(outs[0][0].view(torch.int16), outs[1][0].view(torch.int16)), "outputs differ"
    assert torch.equal(outs[0][1], outs[1][1]), "log-sum-exps differ"
    ref_n, ref_r = c["nope"].clone(), c["rope"].clone()
    O.cache_write(ref_n, slots, c["new_c"])
    O.cache_write(ref_r, slots, c["new_r"])
    assert torch.equal(caches[1][0], ref_n) and torch.equal(caches[1][1], ref_r)
