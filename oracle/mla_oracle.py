"""CPU oracle for the MLA / DSA attention hot path.

TEST INFRASTRUCTURE ONLY.  This module is a plain-torch, fp32, CPU restatement of the
arithmetic the reference backend performs (or asks its vendor kernels to perform) on this
path.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it; nothing under the product package does, and the product path
raises when its HIP library is missing instead of falling back to anything here.

Every function cites the reference lines it follows (paths relative to the reference root).

Pinning status (what checks each function beyond re-typing its formula lives in
``tests/test_oracle.py``):

* ``cache_write``                 closed form (row scatter); slot formula from
                                  tests/integration/attention/test_npu_mla_math.py:201-223.  pinned.
* ``gather_paged``                restates attention/ops.py:5-41; pinned by the scatter/gather round trip,
                                  by brute-force indexing, and by a vector written by the reference function
                                  itself (tests/golden/ops_vectors.npz, tests/test_ops_golden.py).
* ``merge_attn_states``,
  ``attention_update``            restate attention/ops.py:44-106 and :109-141; pinned by the identity
                                  "merge of chunk results == one softmax over the concatenation", by the
                                  -inf / +inf special cases, by fold associativity, and - for the conventions
                                  mathematics does not fix (+inf reads as -inf, rows without weight) - by
                                  vectors written by the reference functions themselves
                                  (tests/golden/make_ops_vectors.py imports that one file, which needs only torch).
* ``absorbed_decode``             restates tests/integration/attention/test_npu_mla_math.py:516-539;
                                  pinned by L=1, all-equal-K, block-table permutation invariance, a
                                  float64 brute-force loop, and the absorbed == non-absorbed equivalence.
* ``prefill_varlen``,
  ``chunked_prefill``             restate tests/integration/attention/test_mla_chunked_prefill.py:226-252
                                  and attention/backends/mla.py:377-450, 573-616; pinned against
                                  torch.nn.functional.scaled_dot_product_attention and the merge identity.
* ``v_up_proj``                   restates attention/backends/mla.py:309-315; pinned by the identity-weight
                                  known answer of tests/unit/attention/backends/test_mla.py:190-259.
* ``sink_decode``, ``sink_prefill``  restate the static-sink / sliding-window branches of
                                  attention/backends/mla.py:463-560 and :705-779 (two attentions with LSE and
                                  their merge; band mask pre_tokens = window - 1).  The reference holds no test
                                  of them; pinned by a per-token brute force over the union of the sink keys and
                                  the windowed keys, by "window >= L == no window", by "sink_len keys moved into
                                  the sequence == plain decode", and against
                                  torch.nn.functional.scaled_dot_product_attention with an explicit mask.
* ``indexer_scores``, ``topk_stable``, ``sparse_decode``
                                  PARITY UNPINNED against the reference: its lightning indexer and sparse
                                  flash attention are closed vendor ops with mock-only tests
                                  (tests/unit/layers/test_npu_dsa.py:122-138).  They are pinned only
                                  against the mathematics: float64 brute force, the selection invariant
                                  (every kept score >= every dropped score, lowest index on ties), and
                                  "k >= L  ==> sparse == dense decode".
* ``rms_norm``, ``interleave_rope``,
  ``kv_rmsnorm_rope_cache``       restate the reference's own torch formulation of the fused vendor op
                                  (layers/rotary_embedding/rotary_embedding_torch_npu.py:146-173 for the
                                  rotation and its cat(c, c) tables; the kv_a_layernorm + npu_interleave_rope
                                  branch of v1/layers/attention/npu_dsa.py:405-408).  The vendor op itself is
                                  closed: PARITY UNPINNED against it.  Pinned against the mathematics:
                                  torch.nn.functional.rms_norm, a float64 loop, rotation invariants (pair norms,
                                  position 0 = de-interleave only, q.k depends on the position difference only)
                                  and agreement of the two output layouts up to the fixed permutation.
* ``fp8 quantise / dequantise``   PARITY UNPINNED against the reference (it has no fp8 KV format,
                                  attention/ops.py:11-12 ignores its scale); the block and the per-token
                                  quantiser are each pinned by their closed form: scale = amax / 448 exactly
                                  (1.0 for zeros), the extreme lands on +-448, half-ulp error bound per binade,
                                  grid values and ties-to-even survive exactly, power-of-two scaling invariance.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import torch

PAGE = 128          # attention/backends/mla.py:794 (block_size=128), platform.py:122-124
D_NOPE = 512        # kv_lora_rank; attention/backends/mla.py:68
D_ROPE = 64         # qk_rope_head_dim; attention/backends/mla.py:68
FP8_MAX = 448.0     # largest finite float8_e4m3fn
FP8_BLOCK = 128     # one fp32 scale per 128 latent elements


# --------------------------------------------------------------------------------------
# paging helpers
# --------------------------------------------------------------------------------------
def slots_for(block_table: torch.Tensor, b: int, start: int, end: int, page: int = PAGE) -> torch.Tensor:
    """Flat cache rows of logical positions [start, end) of sequence ``b``.

    slot = block_id * page + pos % page  (tests/integration/attention/test_npu_mla_math.py:201-210).
    """
    pos = torch.arange(start, end, dtype=torch.long)
    blk = block_table[b, pos // page].to(torch.long)
    return blk * page + pos % page


def cache_write(cache: torch.Tensor, slot_mapping: torch.Tensor, src: torch.Tensor) -> None:
    """``cache.flatten(0, -2)[slot[t]] = src[t]``; negative (pad) slots are skipped.

    Follows ``store_kv`` in attention/backends/mla.py:868-881 and dsa.py:359-362; pad slots are
    PAD_SLOT_ID = -1 (dsa.py:172-177).
    """
    flat = cache.view(-1, cache.shape[-1])
    src = src.reshape(-1, cache.shape[-1])
    n = min(slot_mapping.numel(), src.shape[0])
    slots = slot_mapping.reshape(-1)[:n].to(torch.long)
    keep = slots >= 0
    flat[slots[keep]] = src[:n][keep].to(cache.dtype)


def gather_paged(nope_cache, rope_cache, dst, block_table, cu_seq_lens, batch_size, seq_starts=None):
    """dst[cu[i]:cu[i+1]] = cat(nope[blk, slot], rope[blk, slot]) for positions
    seq_starts[i] .. seq_starts[i] + len_i  (attention/ops.py:5-41; no dequantisation happens there).
    """
    page = nope_cache.shape[1]
    nope = nope_cache.reshape(-1, nope_cache.shape[-1])
    rope = rope_cache.reshape(-1, rope_cache.shape[-1])
    for i in range(batch_size):
        d0, d1 = int(cu_seq_lens[i]), int(cu_seq_lens[i + 1])
        n = d1 - d0
        if n <= 0:
            continue
        s0 = 0 if seq_starts is None else int(seq_starts[i])
        rows = slots_for(block_table, i, s0, s0 + n, page)
        dst[d0:d1] = torch.cat([nope[rows], rope[rows]], dim=-1).to(dst.dtype)


# --------------------------------------------------------------------------------------
# LSE merges
# --------------------------------------------------------------------------------------
def merge_attn_states(prefix_out, prefix_lse, suffix_out, suffix_lse):
    """Two-way merge in fp32 (attention/ops.py:44-106).

    out [T,N,D], lse [T,N,1].  +inf LSE is treated as -inf (:66-72); when both sides are empty the
    output is zero and the merged LSE is -inf (:84-102).  Returns (out fp32, lse fp32).
    """
    po, so = prefix_out.float(), suffix_out.float()
    ninf = torch.tensor(float("-inf"))
    pl = torch.where(prefix_lse == float("inf"), ninf, prefix_lse.float())
    sl = torch.where(suffix_lse == float("inf"), ninf, suffix_lse.float())
    m = torch.maximum(pl, sl)
    pe, se = torch.exp(pl - m), torch.exp(sl - m)
    # exp(-inf - -inf) is nan: both sides empty -> weights forced to zero below
    pe, se = torch.nan_to_num(pe, nan=0.0), torch.nan_to_num(se, nan=0.0)
    tot = pe + se
    ok = tot > 0
    lse = torch.where(ok, torch.log(tot) + m, ninf)
    pw = torch.where(ok, pe / tot, torch.zeros_like(pe))
    sw = torch.where(ok, se / tot, torch.zeros_like(se))
    return po * pw + so * sw, lse


def attention_update(outs: torch.Tensor, lses: torch.Tensor):
    """N-way merge (attention/ops.py:109-141): outs [n,T,D], lses [n,T] -> out [T,D], lse [T] (fp32)."""
    o = outs.transpose(0, 1).float()
    l = lses.transpose(0, 1).float()
    ninf = torch.tensor(float("-inf"))
    l = torch.where(l == float("inf"), ninf, l)
    m = l.max(dim=-1)[0]
    e = torch.nan_to_num(torch.exp(l - m.view(-1, 1)), nan=0.0)
    tot = e.sum(-1)
    ok = tot > 0
    lse = torch.where(ok, torch.log(tot) + m, ninf)
    w = torch.where(ok.view(-1, 1), e / tot.view(-1, 1), torch.zeros_like(e)).unsqueeze(2)
    return (o * w).sum(1), lse


# --------------------------------------------------------------------------------------
# absorb / up-projection GEMMs
# --------------------------------------------------------------------------------------
def q_absorb(q_nope: torch.Tensor, w_uk_t: torch.Tensor) -> torch.Tensor:
    """ql[b,n,:] = q_nope[b,n,:] @ W_UK_T[n]  (attention/backends/mla.py:900-912). fp32 result."""
    return torch.einsum("bnp,npl->bnl", q_nope.float(), w_uk_t.float())


def v_up_proj(o_head_major: torch.Tensor, w_uv: torch.Tensor) -> torch.Tensor:
    """[N,T,512] x [N,512,V] -> [T, N*V]  (attention/backends/mla.py:309-315). fp32 result."""
    n, t, _ = o_head_major.shape
    out = torch.bmm(o_head_major.float(), w_uv.float())       # [N,T,V]
    return out.transpose(0, 1).reshape(t, -1)


# --------------------------------------------------------------------------------------
# absorbed paged decode
# --------------------------------------------------------------------------------------
def absorbed_decode(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, scale,
                    query_start_loc: Optional[Sequence[int]] = None, return_lse: bool = False,
                    causal: bool = True, window: Optional[int] = None):
    """Absorbed MLA decode over the paged latent cache.

    For sequence b with L_b cached tokens (new tokens included) and s_b query tokens, query token i
    (0-based inside the request) sees keys [0, L_b - s_b + i]  (right-down causal: sparse_mode=3 with the
    shared lower-triangular mask, attention/backends/mla.py:298-302, 783-799).  score = scale * (q_nope . Kc + q_rope . Kr), softmax in fp32,
    out = P @ Kc  (tests/integration/attention/test_npu_mla_math.py:516-539).

    q_nope [T,N,512], q_rope [T,N,64]; caches [nblk,page,512] / [nblk,page,64] (a singleton head dim is
    accepted); returns out fp32 [T,N,512] (token-major) and optionally lse [T,N].

    ``causal=False`` lets every query token see all L_b keys (the sink call of mla.py:723-737 passes no mask);
    ``window`` keeps only the last ``window`` visible keys of each row (sparse_mode=4 with
    pre_tokens = sliding_window - 1, mla.py:740-756).
    """
    t_tot, n, _ = q_nope.shape
    nb = len(seq_lens)
    if query_start_loc is None:
        assert t_tot % nb == 0
        s = t_tot // nb
        query_start_loc = [i * s for i in range(nb + 1)]
    page = nope_cache.shape[1]
    kc_flat = nope_cache.reshape(-1, nope_cache.shape[-1])
    kr_flat = rope_cache.reshape(-1, rope_cache.shape[-1])
    out = torch.zeros(t_tot, n, kc_flat.shape[-1], dtype=torch.float32)
    lse = torch.full((t_tot, n), float("-inf"), dtype=torch.float32)
    for b in range(nb):
        L = int(seq_lens[b])
        q0, q1 = int(query_start_loc[b]), int(query_start_loc[b + 1])
        s = q1 - q0
        if s <= 0 or L <= 0:
            continue
        rows = slots_for(block_table, b, 0, L, page)
        kc = kc_flat[rows].float()                           # [L,512]
        kr = kr_flat[rows].float()                           # [L,64]
        qn = q_nope[q0:q1].float().reshape(s * n, -1)
        qr = q_rope[q0:q1].float().reshape(s * n, -1)
        sc = (qn @ kc.t() + qr @ kr.t()) * scale             # [s*n, L]
        lim = (L - s + torch.arange(s) + 1).repeat_interleave(n) if causal else torch.full((s * n,), L)
        if s > 1 and causal:
            sc = sc.masked_fill(torch.arange(L).view(1, -1) >= lim.view(-1, 1), float("-inf"))
        if window is not None:
            sc = sc.masked_fill(torch.arange(L).view(1, -1) < (lim - window).view(-1, 1), float("-inf"))
        lse_b = torch.logsumexp(sc, dim=-1)
        p = torch.nan_to_num(torch.softmax(sc, dim=-1), nan=0.0)
        out[q0:q1] = (p @ kc).view(s, n, -1)
        lse[q0:q1] = lse_b.view(s, n)
    return (out, lse) if return_lse else out


# --------------------------------------------------------------------------------------
# non-absorbed prefill (suffix + chunked context)
# --------------------------------------------------------------------------------------
def kv_up_proj(kv_c: torch.Tensor, w_kv_b: torch.Tensor, n_heads: int, p: int, v: int):
    """kv_b_proj: latent [T,512] @ W [512, N*(P+V)] -> k_nope [T,N,P], v [T,N,V]
    (attention/backends/mla.py:476-482)."""
    kv = (kv_c.float() @ w_kv_b.float()).view(-1, n_heads, p + v)
    return kv[..., :p], kv[..., p:]


def attention_varlen(q_nope, q_pe, k_nope, k_pe, v, cu_q, cu_k, scale, causal: bool, window: Optional[int] = None):
    """Varlen non-absorbed attention with LSE.

    q_nope [T,N,P], q_pe [T,N,R], k_nope [Tk,N,P], k_pe [Tk,R] (shared by all heads,
    attention/backends/mla.py:579), v [Tk,N,V].  ``causal`` is right-down aligned
    (sparse_mode=3, attention/backends/mla.py:584-585); with ``window`` only the last ``window`` visible keys
    of a row stay (sparse_mode=4, pre_tokens = sliding_window - 1, mla.py:525-541).  Empty key ranges give
    out = 0, lse = -inf.
    Returns out fp32 [T,N,V], lse fp32 [T,N].
    """
    t, n, _ = q_nope.shape
    out = torch.zeros(t, n, v.shape[-1], dtype=torch.float32)
    lse = torch.full((t, n), float("-inf"), dtype=torch.float32)
    for b in range(len(cu_q) - 1):
        q0, q1, k0, k1 = int(cu_q[b]), int(cu_q[b + 1]), int(cu_k[b]), int(cu_k[b + 1])
        sq, sk = q1 - q0, k1 - k0
        if sq <= 0 or sk <= 0:
            continue
        sc = (torch.einsum("tnd,snd->nts", q_nope[q0:q1].float(), k_nope[k0:k1].float())
              + torch.einsum("tnd,sd->nts", q_pe[q0:q1].float(), k_pe[k0:k1].float())) * scale
        if causal:
            last = torch.arange(sq).view(-1, 1) + (sk - sq)                 # last visible key of each row
            vis = torch.arange(sk).view(1, -1) <= last
            if window is not None:
                vis &= torch.arange(sk).view(1, -1) > last - window
            sc = sc.masked_fill(~vis.unsqueeze(0), float("-inf"))
        l = torch.logsumexp(sc, dim=-1)                       # [n, sq]
        p = torch.nan_to_num(torch.softmax(sc, dim=-1), nan=0.0)
        out[q0:q1] = torch.einsum("nts,snd->tnd", p, v[k0:k1].float())
        lse[q0:q1] = l.t()
    return out, lse


def chunked_prefill(q, kv_c_suffix, k_pe_suffix, w_kv_b, nope_cache, rope_cache, block_table,
                    cu_q, context_chunks, scale, p_dim=128, v_dim=128):
    """Chunked-context prefill (attention/backends/mla.py:452-483, 573-616 with :377-450).

    q [T,N,P+R]; suffix latent [T,512] / [T,64]; ``context_chunks`` is a list of
    (cu_seq_lens [B+1], starts [B]) pairs, one per context chunk (the schedule vLLM's builder hands
    over, mla.py:391-405).  Suffix attention is causal inside the chunk; each context chunk is gathered
    from the paged cache, up-projected, attended without a mask and folded in with the two-way merge.
    Returns out fp32 [T, N*V] (the reference casts it to bf16, mla.py:616).
    """
    t, n, _ = q.shape
    q_nope, q_pe = q[..., :p_dim], q[..., p_dim:]
    k_nope, v = kv_up_proj(kv_c_suffix, w_kv_b, n, p_dim, v_dim)
    out, lse = attention_varlen(q_nope, q_pe, k_nope, k_pe_suffix.reshape(t, -1), v, cu_q, cu_q, scale, True)
    ctx_out, ctx_lse = None, None
    nb = len(cu_q) - 1
    for cu_k, starts in context_chunks:
        toks = int(cu_k[-1])
        ws = torch.zeros(toks, nope_cache.shape[-1] + rope_cache.shape[-1], dtype=nope_cache.dtype)
        gather_paged(nope_cache, rope_cache, ws, block_table, cu_k, nb, starts)
        ck_nope, cv = kv_up_proj(ws[:, :nope_cache.shape[-1]], w_kv_b, n, p_dim, v_dim)
        o_i, l_i = attention_varlen(q_nope, q_pe, ck_nope, ws[:, nope_cache.shape[-1]:], cv, cu_q, cu_k, scale, False)
        if ctx_out is None:
            ctx_out, ctx_lse = o_i, l_i
        else:
            ctx_out, l3 = merge_attn_states(ctx_out, ctx_lse.unsqueeze(-1), o_i, l_i.unsqueeze(-1))
            ctx_lse = l3.squeeze(-1)
    if ctx_out is not None:
        out, _ = merge_attn_states(ctx_out, ctx_lse.unsqueeze(-1), out, lse.unsqueeze(-1))
    return out.reshape(t, -1)


# --------------------------------------------------------------------------------------
# the step in front of the path: RMSNorm + rotary embedding + cache write
# --------------------------------------------------------------------------------------
def rope_tables(positions: torch.Tensor, rotary_dim: int = D_ROPE, base: float = 10000.0, layout: str = "half",
                dtype=torch.bfloat16):
    """cos / sin rows for ``positions``: inv_freq = base^(-2i/d), angle = pos * inv_freq
    (layers/rotary_embedding/deepseek_scaling_rope.py:51-87 without the YaRN blend).  layout "half" gives the rows
    the reference hands to its fused ops, cat(c, c) (rotary_embedding_torch_npu.py:170-173); "repeat" repeats
    every entry (c0, c0, c1, c1, ...), the layout tests/integration/attention/test_npu_mla_math.py:125-144 reads
    with [..., ::2]."""
    inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    ang = torch.outer(positions.float(), inv_freq)
    c, s = ang.cos(), ang.sin()
    if layout == "half":
        return torch.cat((c, c), -1).to(dtype), torch.cat((s, s), -1).to(dtype)
    return c.repeat_interleave(2, -1).to(dtype), s.repeat_interleave(2, -1).to(dtype)


def rms_norm(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * gamma over the last dim, in float64, rounded once to x.dtype
    (the kv_a_layernorm of v1/layers/attention/npu_dsa.py:405)."""
    xd = x.double()
    inv = torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + eps)
    return (xd * inv * gamma.double()).to(x.dtype)


def yarn_rope_tables(positions, rotary_dim: int = D_ROPE, base: float = 10000.0, scaling_factor: float = 40.0,
                     original_max_position: int = 4096, beta_fast: float = 32, beta_slow: float = 1, mscale: float = 1.0,
                     mscale_all_dim: float = 0.0, attn_factor: float = 1.0, dtype=torch.bfloat16):
    """cos / sin rows cat(c, c) of the YaRN-scaled rotary embedding DeepSeek-V2/V3 use
    (layers/rotary_embedding/deepseek_scaling_rope.py:51-87; the helper functions it imports from vLLM are not in the
    reference tree: this is the published YaRN formulation, written as loops over the pairs in float64).
    Pair i rotates at f_i = base^(-2i/d); pairs that turn more than beta_fast times over the original context keep f_i,
    pairs that turn less than beta_slow times get f_i / factor, a linear ramp over the pair index lies between; the
    values are scaled by (0.1 m ln(factor) + 1) / (0.1 m_all ln(factor) + 1) * attn_factor."""
    import math
    half = rotary_dim // 2

    def corr(rot):
        return rotary_dim * math.log(original_max_position / (rot * 2 * math.pi)) / (2 * math.log(base))

    low, high = max(math.floor(corr(beta_fast)), 0), min(math.ceil(corr(beta_slow)), rotary_dim - 1)
    if low == high:
        high += 0.001

    def ms(m):
        return 1.0 if scaling_factor <= 1 else 0.1 * m * math.log(scaling_factor) + 1.0

    scale = ms(mscale) / ms(mscale_all_dim) * attn_factor
    inv = []
    for i in range(half):
        f = float(base) ** (-2.0 * i / rotary_dim)
        ramp = min(max((i - low) / (high - low), 0.0), 1.0)      # 0: keep (extrapolate), 1: divide (interpolate)
        inv.append(f * (1.0 - ramp) + f / scaling_factor * ramp)
    inv = torch.tensor(inv, dtype=torch.float64)
    ang = torch.outer(torch.as_tensor(positions).double(), inv)
    c, s = ang.cos() * scale, ang.sin() * scale
    return torch.cat((c, c), -1).to(dtype), torch.cat((s, s), -1).to(dtype)


def interleave_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, table: str = "half",
                    interleaved_out: bool = False) -> torch.Tensor:
    """x [T, ..., D] with pairs (2i, 2i+1); cos / sin [T, W] rows.  x1 = x[..., 0::2], x2 = x[..., 1::2],
    o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin, result cat(o1, o2)
    (layers/rotary_embedding/rotary_embedding_torch_npu.py:146-163, non-neox branch).  ``interleaved_out`` puts
    the pairs back in place instead.  float64, rounded once."""
    d = x.shape[-1]
    step = {"half": 1, "repeat": 2}[table]
    c = cos.reshape(cos.shape[0], -1)[:, 0:(d // 2) * step:step].double()
    s = sin.reshape(sin.shape[0], -1)[:, 0:(d // 2) * step:step].double()
    while c.dim() < x.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    x1, x2 = x[..., 0::2].double(), x[..., 1::2].double()
    o1, o2 = x1 * c - x2 * s, x2 * c + x1 * s
    if interleaved_out:
        return torch.stack((o1, o2), -1).reshape(x.shape).to(x.dtype)
    return torch.cat((o1, o2), -1).to(x.dtype)


def rotary_mul(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, table: str = "half") -> torch.Tensor:
    """Half-rotation pairing: x = cat(x1, x2) on the last dim, o1 = x1*cos - x2*sin, o2 = x2*cos + x1*sin, result
    cat(o1, o2) (layers/rotary_embedding/rotary_embedding_torch_npu.py:146-163, neox branch; what
    torch_npu.npu_rotary_mul computes at v1/layers/attention/npu_dsa.py:120, 130 with rows cat(c, c)).  float64, rounded
    once."""
    d = x.shape[-1]
    step = {"half": 1, "repeat": 2}[table]
    c = cos.reshape(cos.shape[0], -1)[:, 0:(d // 2) * step:step].double()
    s = sin.reshape(sin.shape[0], -1)[:, 0:(d // 2) * step:step].double()
    while c.dim() < x.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    x1, x2 = x[..., : d // 2].double(), x[..., d // 2:].double()
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), -1).to(x.dtype)


def kv_rmsnorm_rope_cache(kv, gamma, cos, sin, slot_mapping, nope_cache, rope_cache, eps, table="half",
                          interleaved_out=False):
    """The fused vendor op torch_npu.npu_kv_rmsnorm_rope_cache (v1/layers/attention/npu_mla.py:196-206) as the
    composition the reference itself uses when it does not fuse (npu_dsa.py:405-408 + the cache scatter of
    attention/backends/mla.py:868-881).  Returns (k_pe_rotated, kv_a_normed); the caches are updated in place."""
    kv = kv.reshape(kv.shape[0], -1)
    kv_a = rms_norm(kv[:, :D_NOPE], gamma, eps)
    k_pe = interleave_rope(kv[:, D_NOPE:], cos, sin, table, interleaved_out)
    cache_write(nope_cache, slot_mapping, kv_a)
    cache_write(rope_cache, slot_mapping, k_pe)
    return k_pe, kv_a


# --------------------------------------------------------------------------------------
# fp8-e4m3 block-scaled latent cache (no reference format exists; closed form)
# --------------------------------------------------------------------------------------
def fp8_quant_block(x: torch.Tensor, block: int = FP8_BLOCK):
    """Per-``block`` quantisation along the last dim: scale = amax/448 (1.0 for an all-zero block),
    q = round-to-nearest-even e4m3 of x/scale.  Returns (q float8_e4m3fn, scale fp32 [..., D/block])."""
    xs = x.float().reshape(*x.shape[:-1], -1, block)
    amax = xs.abs().amax(-1, keepdim=True)
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    q = (xs / scale).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.reshape(x.shape), scale.squeeze(-1)


def fp8_dequant_block(q: torch.Tensor, scale: torch.Tensor, block: int = FP8_BLOCK) -> torch.Tensor:
    xs = q.float().reshape(*q.shape[:-1], -1, block)
    return (xs * scale.unsqueeze(-1)).reshape(q.shape)


def gather_paged_fp8(q8, scales, rope_cache, dst, block_table, cu_seq_lens, batch_size, seq_starts=None):
    """gather_paged over a block-scaled fp8 latent cache: q8 [nblk, page, 512] e4m3 with scales [nblk, page, 4] and the bf16
    rope cache; a destination row is cat(bf16(q8 * scale), rope) (one rounding: the fp32 product to bf16).  The chunked
    context of attention/backends/mla.py:377-450 over a quantised cache; no reference format exists (closed form)."""
    nope = fp8_dequant_block(q8, scales).to(torch.bfloat16)
    gather_paged(nope, rope_cache, dst, block_table, cu_seq_lens, batch_size, seq_starts)


def fp8_quant_token(x: torch.Tensor):
    """Per-token (last-dim) quantisation with one fp32 scale = amax/448 (DSA indexer q/k)."""
    amax = x.float().abs().amax(-1, keepdim=True)
    scale = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
    q = (x.float() / scale).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scale.squeeze(-1)


# --------------------------------------------------------------------------------------
# DSA: lightning indexer, top-k, sparse decode
# --------------------------------------------------------------------------------------
def indexer_scores(q8, q_scale, k8, k_scale, weights):
    """score[s] = k_scale[s] * sum_h (w[h] * q_scale[h]) * relu(q8[h] . k8[s])   for one query token.

    q8 [H,128] fp8 (or float), q_scale [H], k8 [L,128], k_scale [L], weights [H].  This is the DeepSeek-V3.2
    lightning-indexer score in its published closed form; the reference passes the raw weights_proj output
    (v1/layers/attention/npu_dsa.py:141-142) to a closed op (npu_dsa.py:92-103).  fp32 accumulation.
    """
    dots = torch.relu(q8.float() @ k8.float().t())            # [H, L]
    wq = (weights.float() * q_scale.float()).view(1, -1)      # [1, H]
    return (wq @ dots).view(-1) * k_scale.float()


def topk_stable(scores: torch.Tensor, k: int, length: Optional[int] = None) -> torch.Tensor:
    """Indices of the k largest scores among [0, length), ties to the lower index, as int32 [k]
    in descending-score order; -1 pads when length < k (v1/layers/attention/npu_dsa.py:553-555).
    """
    length = scores.numel() if length is None else int(length)
    order = torch.sort(scores[:length].float(), descending=True, stable=True)[1][:k].to(torch.int32)
    out = torch.full((k,), -1, dtype=torch.int32)
    out[: order.numel()] = order
    return out


def sparse_decode(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, sparse_indices, scale,
                  return_lse: bool = False):
    """Absorbed MLA restricted to the listed key positions (attention/backends/dsa.py:259-291).

    q_nope [T,N,512], q_rope [T,N,64] with one query token per sequence (T == B); sparse_indices
    [T,1,K] or [T,K] int32 logical positions, -1 = unused.  Indices >= seq_len are ignored as well.
    Returns fp32 [T,N,512] token-major.
    """
    t, n, _ = q_nope.shape
    page = nope_cache.shape[1]
    idx = sparse_indices.reshape(t, -1).to(torch.long)
    kc_flat = nope_cache.reshape(-1, nope_cache.shape[-1])
    kr_flat = rope_cache.reshape(-1, rope_cache.shape[-1])
    out = torch.zeros(t, n, kc_flat.shape[-1], dtype=torch.float32)
    lse = torch.full((t, n), float("-inf"), dtype=torch.float32)
    for b in range(t):
        L = int(seq_lens[b])
        pos = idx[b][(idx[b] >= 0) & (idx[b] < L)]
        if pos.numel() == 0:
            continue
        rows = block_table[b, pos // page].to(torch.long) * page + pos % page
        kc, kr = kc_flat[rows].float(), kr_flat[rows].float()
        sc = (q_nope[b].float() @ kc.t() + q_rope[b].float() @ kr.t()) * scale
        lse[b] = torch.logsumexp(sc, -1)
        out[b] = torch.softmax(sc, -1) @ kc
    return (out, lse) if return_lse else out


# --------------------------------------------------------------------------------------
# static sink tokens (+ sliding window)
# --------------------------------------------------------------------------------------
def sink_decode(q_nope, q_rope, nope_cache, rope_cache, block_table, seq_lens, sink_len: int, scale,
                window: Optional[int] = None, query_start_loc: Optional[Sequence[int]] = None):
    """Decode with static sink tokens (attention/backends/mla.py:705-779).

    The first sink_len / 128 pages of every block-table row hold the sink keys (sink_len must be a multiple of the
    page, mla.py:719-721); ``seq_lens`` counts the keys behind them.  One attention over the sink keys (no mask,
    mla.py:723-737), one over the sequence's own keys through block_table[:, sink pages:] (causal tail for several
    query tokens, optionally only the last ``window`` keys, mla.py:740-773), merged by their LSEs (mla.py:776-779).
    Returns fp32 [T,N,512] token-major."""
    page = nope_cache.shape[1]
    if sink_len % page != 0:
        raise ValueError(f"sink_len {sink_len} must align with block size")
    nsb = sink_len // page
    nb = len(seq_lens)
    o_s, l_s = absorbed_decode(q_nope, q_rope, nope_cache, rope_cache, block_table, [sink_len] * nb, scale,
                               query_start_loc, return_lse=True, causal=False)
    o_n, l_n = absorbed_decode(q_nope, q_rope, nope_cache, rope_cache, block_table[:, nsb:], seq_lens, scale,
                               query_start_loc, return_lse=True, window=window)
    m = torch.maximum(l_s, l_n)
    w_s, w_n = torch.exp(l_s - m).unsqueeze(-1), torch.exp(l_n - m).unsqueeze(-1)
    return (o_s * w_s + o_n * w_n) / (w_s + w_n)


def insert_sink_rows(x: torch.Tensor, sink: torch.Tensor, cu_q: Sequence[int]) -> torch.Tensor:
    """The sink rows in front of every sequence's rows (mla.py:929-949)."""
    parts = []
    for b in range(len(cu_q) - 1):
        parts += [sink, x[int(cu_q[b]):int(cu_q[b + 1])]]
    return torch.cat(parts, 0)


def sink_prefill(q, kv_c, k_pe, w_kv_b, sink_kv_c, sink_k_pe, cu_q, scale, window: Optional[int] = None,
                 p_dim: int = 128, v_dim: int = 128):
    """Prefill with static sink tokens (attention/backends/mla.py:463-560).  No cached context is read
    (has_context is forced off, mla.py:497).

    Without a window the sink latents are put in front of every sequence's new latents and one right-down causal
    attention runs over sink_len + s_b keys (mla.py:463-491, 546-572).  With a window the sink keys get their own
    unmasked attention, the new keys a causal band of ``window`` keys, and the two are merged by LSE with the
    sink as the prefix (mla.py:498-557).  q [T,N,P+R]; kv_c [T,512], k_pe [T,64]; sink_kv_c [S,512], sink_k_pe
    [S,64].  Returns fp32 [T, N*V]."""
    t, n, _ = q.shape
    q_nope, q_pe = q[..., :p_dim], q[..., p_dim:]
    nb = len(cu_q) - 1
    s_len = sink_kv_c.shape[0]
    cu_q = [int(x) for x in cu_q]
    if window is None:
        k_nope, v = kv_up_proj(insert_sink_rows(kv_c, sink_kv_c, cu_q), w_kv_b, n, p_dim, v_dim)
        cu_k = [cu_q[i] + s_len * i for i in range(nb + 1)]
        out, _ = attention_varlen(q_nope, q_pe, k_nope, insert_sink_rows(k_pe, sink_k_pe, cu_q), v, cu_q, cu_k, scale, True)
        return out.reshape(t, -1)
    ks_nope, vs = kv_up_proj(sink_kv_c, w_kv_b, n, p_dim, v_dim)
    o_s, l_s = attention_varlen(q_nope, q_pe, ks_nope.repeat(nb, 1, 1), sink_k_pe.repeat(nb, 1), vs.repeat(nb, 1, 1),
                                cu_q, [s_len * i for i in range(nb + 1)], scale, False)
    k_nope, v = kv_up_proj(kv_c, w_kv_b, n, p_dim, v_dim)
    o_n, l_n = attention_varlen(q_nope, q_pe, k_nope, k_pe, v, cu_q, cu_q, scale, True, window=window)
    out, _ = merge_attn_states(o_s, l_s.unsqueeze(-1), o_n, l_n.unsqueeze(-1))
    return out.reshape(t, -1)


# --------------------------------------------------------------------------------------
# seeded synthetic inputs shared by tests, smoke and bench (generated on the CPU so that the
# oracle and the GPU see identical bits)
# --------------------------------------------------------------------------------------
def make_decode_case(batch, n_heads, len_lo, len_hi, seed=0, q_len=1, page=PAGE, dtype=torch.bfloat16,
                     extra_blocks=0, shuffle=True):
    """Paged absorbed-decode case: lens uniform in [len_lo, len_hi], block tables = consecutive slices of a
    random permutation of the pages, q and caches N(0,1), new-token rows at positions L-q_len .. L-1."""
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(len_lo, len_hi + 1, (batch,), generator=g)
    nblk_seq = (lens + page - 1) // page
    nblk = int(nblk_seq.sum()) + extra_blocks
    perm = torch.randperm(nblk, generator=g) if shuffle else torch.arange(nblk)
    max_blk = int(nblk_seq.max())
    bt = torch.zeros(batch, max_blk, dtype=torch.int32)
    o = 0
    for b in range(batch):
        k = int(nblk_seq[b])
        bt[b, :k] = perm[o:o + k].to(torch.int32)
        o += k
    nope = torch.randn(nblk, page, D_NOPE, generator=g).to(dtype)
    rope = torch.randn(nblk, page, D_ROPE, generator=g).to(dtype)
    t = batch * q_len
    q_nope = torch.randn(t, n_heads, D_NOPE, generator=g).to(dtype)
    q_rope = torch.randn(t, n_heads, D_ROPE, generator=g).to(dtype)
    new_c = torch.randn(t, D_NOPE, generator=g).to(dtype)
    new_r = torch.randn(t, D_ROPE, generator=g).to(dtype)
    slots = torch.empty(t, dtype=torch.long)
    for b in range(batch):
        L = int(lens[b])
        slots[b * q_len:(b + 1) * q_len] = slots_for(bt, b, L - q_len, L, page)
    return dict(seq_lens=lens.to(torch.int32), block_table=bt, nope=nope, rope=rope, q_nope=q_nope,
                q_rope=q_rope, new_c=new_c, new_r=new_r, slot_mapping=slots, q_len=q_len,
                scale=1.0 / math.sqrt(192.0))
