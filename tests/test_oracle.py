"""Pins for the CPU oracle: each check is chosen so that a plausible mistake (a dropped term, a wrong sign or
index, a transposed operand) fails it.  Nothing here re-types an oracle formula and compares it with itself:
the references are brute-force float64 loops, torch library routines, closed forms and invariants."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import mla_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---- paging, cache write, gather ------------------------------------------------------------------
def test_slot_formula_and_cache_write_brute_force():
    """slot = block_id * 128 + pos % 128 (reference tests/integration/attention/test_npu_mla_math.py:201-223)."""
    bt = torch.tensor([[3, 0, 5], [1, 4, 2]], dtype=torch.int32)
    for b in range(2):
        got = O.slots_for(bt, b, 100, 300).tolist()
        want = [int(bt[b, p // 128]) * 128 + p % 128 for p in range(100, 300)]
        assert got == want
    cache = torch.zeros(6, 128, 64)
    src = torch.arange(5 * 64, dtype=torch.float32).view(5, 64)
    slots = torch.tensor([700, -1, 5, 129, -1])
    O.cache_write(cache, slots, src)
    flat = cache.view(-1, 64)
    for t, s in enumerate(slots.tolist()):
        if s >= 0:
            assert torch.equal(flat[s], src[t])
    assert flat.abs().sum() == src[[0, 2, 3]].abs().sum()          # nothing else was touched


def test_gather_inverts_scatter():
    c = O.make_decode_case(3, 4, 50, 400, seed=1)
    starts = torch.tensor([0, 10, 130], dtype=torch.int32)
    lens = torch.tensor([50, 20, 7], dtype=torch.int32)
    cu = torch.tensor([0, 50, 70, 77], dtype=torch.int32)
    dst = torch.zeros(77, 576, dtype=torch.bfloat16)
    O.gather_paged(c["nope"], c["rope"], dst, c["block_table"], cu, 3, starts)
    for i in range(3):
        for j in range(int(lens[i])):
            pos = int(starts[i]) + j
            blk, off = int(c["block_table"][i, pos // 128]), pos % 128
            row = dst[int(cu[i]) + j]
            assert torch.equal(row[:512], c["nope"][blk, off]) and torch.equal(row[512:], c["rope"][blk, off])


# ---- LSE merges --------------------------------------------------------------------------------------
def _softmax_attend(s, v):
    return torch.softmax(s, -1) @ v, torch.logsumexp(s, -1)


def test_merge_equals_one_softmax_over_the_concatenation():
    g = torch.Generator().manual_seed(0)
    t, n, d = 5, 3, 16
    s1, s2, s3 = (torch.randn(t, n, k, generator=g, dtype=torch.float64) * 3 for k in (7, 11, 4))
    v1, v2, v3 = (torch.randn(t, n, k, d, generator=g, dtype=torch.float64) for k in (7, 11, 4))
    att = lambda s, v: (torch.einsum("tnk,tnkd->tnd", torch.softmax(s, -1), v), torch.logsumexp(s, -1))
    o1, l1 = att(s1, v1)
    o2, l2 = att(s2, v2)
    o3, l3 = att(s3, v3)
    oa, la = att(torch.cat([s1, s2, s3], -1), torch.cat([v1, v2, v3], 2))
    m12, ml12 = O.merge_attn_states(o1, l1.unsqueeze(-1), o2, l2.unsqueeze(-1))
    m, ml = O.merge_attn_states(m12, ml12, o3, l3.unsqueeze(-1))
    assert torch.allclose(m.double(), oa, atol=1e-5) and torch.allclose(ml.squeeze(-1).double(), la, atol=1e-5)
    # N-way merge == pairwise fold (associativity); layout [n_parts, T*N, D] / [n_parts, T*N]
    outs = torch.stack([o1, o2, o3]).reshape(3, t * n, d)
    lses = torch.stack([l1, l2, l3]).reshape(3, t * n)
    o_n, l_n = O.attention_update(outs, lses)
    assert torch.allclose(o_n.double(), oa.reshape(t * n, d), atol=1e-5)
    assert torch.allclose(l_n.double(), la.reshape(t * n), atol=1e-5)


def test_merge_special_cases():
    """ops.py:66-72 (+inf -> -inf) and :84-102 (both empty -> zeros, -inf)."""
    o1, o2 = torch.full((1, 1, 4), 2.0), torch.full((1, 1, 4), 5.0)
    ninf, pinf, fin = (torch.full((1, 1, 1), v) for v in (float("-inf"), float("inf"), 0.3))
    m, l = O.merge_attn_states(o1, ninf, o2, fin)
    assert torch.equal(m, o2) and l.item() == pytest.approx(0.3)
    m, l = O.merge_attn_states(o1, fin, o2, pinf)
    assert torch.equal(m, o1) and l.item() == pytest.approx(0.3)
    m, l = O.merge_attn_states(o1, ninf, o2, ninf)
    assert (m == 0).all() and l.item() == float("-inf")
    o, l = O.attention_update(torch.stack([o1.view(1, 4), o2.view(1, 4)]), torch.tensor([[float("-inf")], [float("inf")]]))
    assert (o == 0).all() and l.item() == float("-inf")


# ---- absorbed decode --------------------------------------------------------------------------------
def test_decode_brute_force_float64():
    c = O.make_decode_case(2, 3, 5, 140, seed=4, q_len=2)
    out, lse = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"],
                                 c["scale"], return_lse=True)
    for b in range(2):
        L = int(c["seq_lens"][b])
        for i in range(2):
            t = b * 2 + i
            vis = L - 2 + i + 1
            for h in range(3):
                sc = []
                for pos in range(vis):
                    blk, off = int(c["block_table"][b, pos // 128]), pos % 128
                    kc, kr = c["nope"][blk, off].double(), c["rope"][blk, off].double()
                    sc.append(c["scale"] * (float(c["q_nope"][t, h].double() @ kc) + float(c["q_rope"][t, h].double() @ kr)))
                mx = max(sc)
                w = [math.exp(x - mx) for x in sc]
                z = sum(w)
                acc = torch.zeros(512, dtype=torch.float64)
                for pos in range(vis):
                    blk, off = int(c["block_table"][b, pos // 128]), pos % 128
                    acc += (w[pos] / z) * c["nope"][blk, off].double()
                assert torch.allclose(out[t, h].double(), acc, atol=2e-5)
                assert lse[t, h].item() == pytest.approx(mx + math.log(z), abs=1e-4)


def test_decode_invariants():
    c = O.make_decode_case(3, 4, 1, 1, seed=2)                                   # L = 1: the output is that row
    out = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    for b in range(3):
        assert torch.allclose(out[b], c["nope"][int(c["block_table"][b, 0]), 0].float().expand(4, -1))
    c = O.make_decode_case(2, 4, 200, 300, seed=3)
    base = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    # all keys equal -> uniform softmax -> output = the shared row, whatever q is
    c2 = dict(c)
    c2["nope"] = c["nope"][0, 0].expand_as(c["nope"]).contiguous()
    c2["rope"] = c["rope"][0, 0].expand_as(c["rope"]).contiguous()
    eq = O.absorbed_decode(c["q_nope"], c["q_rope"], c2["nope"], c2["rope"], c["block_table"], c["seq_lens"], c["scale"])
    assert torch.allclose(eq, c["nope"][0, 0].float().expand_as(eq), atol=1e-5)
    # moving the physical pages and rewriting the tables changes nothing
    perm = torch.randperm(c["nope"].shape[0], generator=torch.Generator().manual_seed(9))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    moved = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"][perm], c["rope"][perm],
                              inv[c["block_table"].long()].to(torch.int32), c["seq_lens"], c["scale"])
    assert torch.equal(moved, base)


def test_absorbed_decode_equals_non_absorbed_attention():
    """Ties decode to prefill: absorb -> latent attention -> v-up-proj  ==  attention on the
    up-projected keys/values (weight layout of tests/integration/attention/test_npu_mla_math.py:302-313)."""
    g = torch.Generator().manual_seed(7)
    n, p, v, L = 4, 128, 128, 37
    w_kv_b = torch.randn(512, n * (p + v), generator=g) * 0.05
    kvw = w_kv_b.view(512, n, p + v)
    w_uk_t = kvw[..., :p].permute(1, 2, 0).contiguous()          # [N,P,512]
    w_uv = kvw[..., p:].transpose(0, 1).contiguous()             # [N,512,V]
    kc, kr = torch.randn(L, 512, generator=g), torch.randn(L, 64, generator=g)
    q_nope, q_pe = torch.randn(1, n, p, generator=g), torch.randn(1, n, 64, generator=g)
    scale = 192 ** -0.5
    nope, rope = torch.zeros(1, 128, 512), torch.zeros(1, 128, 64)
    nope[0, :L], rope[0, :L] = kc, kr
    o_lat = O.absorbed_decode(O.q_absorb(q_nope, w_uk_t), q_pe, nope, rope, torch.zeros(1, 1, dtype=torch.int32),
                              torch.tensor([L]), scale)
    got = O.v_up_proj(o_lat.transpose(0, 1).contiguous(), w_uv)                  # [1, N*V]
    k_nope, vv = O.kv_up_proj(kc, w_kv_b, n, p, v)
    ref, _ = O.attention_varlen(q_nope, q_pe, k_nope, kr, vv, [0, 1], [0, L], scale, causal=False)
    assert torch.allclose(got, ref.reshape(1, -1), atol=1e-4)


def test_v_up_proj_identity_known_answer():
    """The reference's own KAT (tests/unit/attention/backends/test_mla.py:190-259): input is N-major [N*B, 512],
    W_UV[h, :128, :] = I  ->  out[b, h*128:(h+1)*128] = x[h*B + b, :128]."""
    n, bsz, vd = 32, 2, 128
    x = torch.randn(n * bsz, 512, generator=torch.Generator().manual_seed(0)).bfloat16()
    w = torch.zeros(n, 512, vd, dtype=torch.bfloat16)
    w[:, :vd, :] = torch.eye(vd, dtype=torch.bfloat16)
    out = O.v_up_proj(x.view(n, bsz, 512), w)
    for b in range(bsz):
        for h in range(n):
            assert torch.allclose(out[b, h * vd:(h + 1) * vd], x[h * bsz + b, :vd].float(), atol=1e-3)


# ---- prefill ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("causal", [False, True])
def test_attention_varlen_against_torch_sdpa(causal):
    g = torch.Generator().manual_seed(11)
    n, p, r, v = 3, 128, 64, 128
    cu_q, cu_k = [0, 5, 12], [0, 9, 16] if not causal else [0, 5, 12]
    if causal:
        cu_k = [0, 8, 20]                                      # more keys than queries: right-down alignment
    tq, tk = cu_q[-1], cu_k[-1]
    qn, qp = torch.randn(tq, n, p, generator=g), torch.randn(tq, n, r, generator=g)
    kn, kp, vv = torch.randn(tk, n, p, generator=g), torch.randn(tk, r, generator=g), torch.randn(tk, n, v, generator=g)
    scale = 0.07
    out, lse = O.attention_varlen(qn, qp, kn, kp, vv, cu_q, cu_k, scale, causal)
    for b in range(2):
        q = torch.cat([qn, qp], -1)[cu_q[b]:cu_q[b + 1]].transpose(0, 1)                         # [N,sq,192]
        k = torch.cat([kn, kp.unsqueeze(1).expand(-1, n, -1)], -1)[cu_k[b]:cu_k[b + 1]].transpose(0, 1)
        val = vv[cu_k[b]:cu_k[b + 1]].transpose(0, 1)
        sq, sk = q.shape[1], k.shape[1]
        mask = None
        if causal:
            mask = torch.arange(sk).view(1, -1) <= torch.arange(sq).view(-1, 1) + (sk - sq)
        ref = F.scaled_dot_product_attention(q, k, val, attn_mask=mask, scale=scale)
        assert torch.allclose(out[cu_q[b]:cu_q[b + 1]].transpose(0, 1), ref, atol=1e-5)


def test_chunked_prefill_equals_attention_over_context_plus_suffix():
    """The identity the reference's chunked-prefill test states (tests/integration/attention/
    test_mla_chunked_prefill.py:10-20, :226-252): context 48 in chunks [32,16], suffix 16, causal in the suffix."""
    g = torch.Generator().manual_seed(5)
    bsz, ctx, suf, n = 2, 48, 16, 4
    w = torch.randn(512, n * 256, generator=g) * 0.02
    nblk = bsz
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    bt = torch.tensor([[1], [0]], dtype=torch.int32)
    q = torch.randn(bsz * suf, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(bsz * suf, 512, generator=g).bfloat16(), torch.randn(bsz * suf, 64, generator=g).bfloat16()
    cu_q = [0, suf, 2 * suf]
    chunks = [(torch.tensor([0, 32, 64], dtype=torch.int32), torch.tensor([0, 0], dtype=torch.int32)),
              (torch.tensor([0, 16, 32], dtype=torch.int32), torch.tensor([32, 32], dtype=torch.int32))]
    scale = 192 ** -0.5
    got = O.chunked_prefill(q, kvc, kpe, w, nope, rope, bt, cu_q, chunks, scale).view(bsz * suf, n, 128)
    for b in range(bsz):
        blk = int(bt[b, 0])
        lat = torch.cat([nope[blk, :ctx].float(), kvc[b * suf:(b + 1) * suf].float()])
        pe = torch.cat([rope[blk, :ctx].float(), kpe[b * suf:(b + 1) * suf].float()])
        kn, vv = O.kv_up_proj(lat, w, n, 128, 128)
        qb = q[b * suf:(b + 1) * suf].float()
        for t in range(suf):
            vis = ctx + t + 1
            s = (torch.einsum("nd,knd->nk", qb[t, :, :128], kn[:vis]) + qb[t, :, 128:] @ pe[:vis].t()) * scale
            ref = torch.einsum("nk,knd->nd", torch.softmax(s, -1), vv[:vis])
            assert torch.allclose(got[b * suf + t], ref, atol=1e-5)


# ---- fp8 ----------------------------------------------------------------------------------------------------
def test_fp8_block_quant_closed_form():
    x = torch.randn(7, 512, generator=torch.Generator().manual_seed(1)) * 3
    x[0, :128] = 0
    q, s = O.fp8_quant_block(x)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (7, 4)
    assert s[0, 0] == 1.0 and (q[0, :128].float() == 0).all()
    amax = x.view(7, 4, 128).abs().amax(-1)
    assert torch.equal(s[1:], amax[1:] / 448.0)
    deq = O.fp8_dequant_block(q, s)
    rel = ((deq - x).abs() / x.abs().clamp_min(1e-3))[1:]
    assert (deq - x).abs().max() <= (amax.max() / 448.0) * 16 + 1e-6       # half an ulp at the top binade (ulp = 32)
    assert rel.median() < 2 ** -4
    # values already on the e4m3 grid survive exactly (amax = 448 -> scale 1)
    grid = torch.tensor([448.0, -240.0, 1.5, 0.015625, 0.0] + [0.0] * 123)
    q2, s2 = O.fp8_quant_block(grid.view(1, 128))
    assert s2.item() == 1.0 and torch.equal(q2.float().view(-1), grid)


# ---- DSA ----------------------------------------------------------------------------------------------------
def test_indexer_scores_brute_force():
    g = torch.Generator().manual_seed(3)
    h, L = 64, 9
    q8, qs = O.fp8_quant_token(torch.randn(h, 128, generator=g))
    k8, ks = O.fp8_quant_token(torch.randn(L, 128, generator=g))
    w = torch.randn(h, generator=g)
    got = O.indexer_scores(q8, qs, k8, ks, w)
    for s in range(L):
        acc = 0.0
        for i in range(h):
            d = float(q8[i].double() @ k8[s].double())
            acc += float(w[i]) * float(qs[i]) * max(d, 0.0)
        assert got[s].item() == pytest.approx(acc * float(ks[s]), rel=1e-4, abs=1e-4)


def test_topk_selection_invariant_and_ties():
    x = torch.tensor([1.0, 3.0, 3.0, -1.0, 3.0, 0.5, 3.0])
    assert O.topk_stable(x, 3).tolist() == [1, 2, 4]                    # ties: lowest positions first
    assert O.topk_stable(x, 9, 4).tolist() == [1, 2, 0, 3, -1, -1, -1, -1, -1]
    g = torch.Generator().manual_seed(0)
    y = torch.round(torch.randn(500, generator=g) * 2) / 2
    sel = O.topk_stable(y, 100)
    keep = set(sel.tolist())
    worst = y[sel.long()].min()
    rest = [i for i in range(500) if i not in keep]
    assert all(y[i] <= worst for i in rest)
    tied_out = [i for i in rest if y[i] == worst]
    tied_in = [i for i in keep if y[i] == worst]
    assert not tied_out or max(tied_in) < min(tied_out)


def test_sparse_decode_full_coverage_equals_dense():
    c = O.make_decode_case(2, 4, 10, 200, seed=6)
    k = 256
    idx = torch.full((2, 1, k), -1, dtype=torch.int32)
    for b in range(2):
        L = int(c["seq_lens"][b])
        idx[b, 0, :L] = torch.randperm(L, generator=torch.Generator().manual_seed(b)).to(torch.int32)
    sp = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx, c["scale"])
    de = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    assert torch.allclose(sp, de, atol=1e-5)
    # a strict subset: only the listed keys matter (brute force on one head)
    idx2 = torch.tensor([[[3, 0, 7, -1]], [[1, -1, -1, -1]]], dtype=torch.int32)
    sp2 = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx2, c["scale"])
    blk = int(c["block_table"][1, 0])
    assert torch.allclose(sp2[1], c["nope"][blk, 1].float().expand(4, -1))


# ---- committed fixture ------------------------------------------------------------------------------------
def test_config1_fixture_is_reproduced():
    """tests/golden/config1_decode.npz was written by tests/golden/make_config1.py (oracle on the CPU-plumbing
    configuration).  It guards the oracle and the input generator against silent drift."""
    f = np.load(os.path.join(GOLDEN, "config1_decode.npz"))
    c = O.make_decode_case(4, 16, 128, 1024, seed=0)
    assert c["seq_lens"].tolist() == f["seq_lens"].tolist()
    assert torch.equal(c["block_table"], torch.from_numpy(f["block_table"]))
    out, lse = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"],
                                 c["scale"], return_lse=True)
    assert torch.allclose(out, torch.from_numpy(f["out"]).float(), atol=2e-3)        # stored as fp16
    assert torch.allclose(lse, torch.from_numpy(f["lse"]), atol=1e-5)
