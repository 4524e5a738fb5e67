"""Non-absorbed varlen prefill attention (HIP, through the C-ABI) against the oracle.
Tolerance: max-abs 2e-2 / mean-rel 2e-3 (the reference's own bar is atol = rtol = 2e-2,
tests/integration/attention/test_npu_mla_math.py:147-151)."""
import pytest
import torch

from oracle import mla_oracle as O
from tests.conftest import attn_close

pytestmark = pytest.mark.gpu


def _case(seed, q_lens, k_lens, n):
    g = torch.Generator().manual_seed(seed)
    cu_q = [0]
    cu_k = [0]
    for a, b in zip(q_lens, k_lens):
        cu_q.append(cu_q[-1] + a)
        cu_k.append(cu_k[-1] + b)
    tq, tk = cu_q[-1], cu_k[-1]
    q = torch.randn(tq, n, 192, generator=g).bfloat16()
    kv = (torch.randn(tk, n, 256, generator=g)).bfloat16()          # k_nope | v interleaved per head, as kv_b_proj emits
    k_pe = torch.randn(tk, 1, 64, generator=g).bfloat16()
    return q, kv, k_pe, cu_q, cu_k


@pytest.mark.parametrize("causal,q_lens,k_lens,n", [
    (True, [16, 160, 1], [16, 160, 1], 4),           # the reference's shapes (B,S) = (1,16), (8,160) and a 1-token edge
    (True, [300, 129], [300, 129], 3),               # crosses 128-row and 64-key tile boundaries
    (False, [16, 48, 7], [32, 100, 64], 4),          # context chunk: no mask, more keys than queries
    (True, [40, 70], [100, 70], 2),                  # right-down alignment: more keys than queries
    (False, [5, 9], [0, 33], 2),                     # an empty key range: zeros and lse = -inf
    (True, [300, 129, 64], [300, 200, 64], 8),       # 24 (sequence, head) pairs: the XCD-aware renumbering is active
    (False, [130, 260], [500, 70], 16),              # the same without a mask
])
def test_prefill_varlen_matches_oracle(dev, causal, q_lens, k_lens, n):
    from omni_npu_amd import kernels as K
    q, kv, k_pe, cu_q, cu_k = _case(len(q_lens) * 7 + n, q_lens, k_lens, n)
    scale = 192 ** -0.5
    ref, ref_lse = O.attention_varlen(q[..., :128], q[..., 128:], kv[..., :128], k_pe.view(-1, 64), kv[..., 128:], cu_q,
                                      cu_k, scale, causal)
    dq, dkv, dpe = q.to(dev), kv.to(dev), k_pe.to(dev)
    out = torch.full((q.shape[0], n, 128), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((q.shape[0], n), float("nan"), dtype=torch.float32, device=dev)
    K.prefill_varlen(dq[..., :128], dq[..., 128:], dkv[..., :128], dpe, dkv[..., 128:],
                     torch.tensor(cu_q, dtype=torch.int32, device=dev), torch.tensor(cu_k, dtype=torch.int32, device=dev),
                     max(q_lens), scale, causal, out, lse)
    attn_close(out, ref, 2e-2, 4e-4)                          # fp32 result: only the fp16 rounding of P (2^-12 each) is left
    got_lse = lse.cpu()
    fin = torch.isfinite(ref_lse)
    assert torch.equal(torch.isfinite(got_lse), fin)
    assert torch.allclose(got_lse[fin], ref_lse[fin], atol=2e-2)
    out_bf = torch.empty(q.shape[0], n, 128, dtype=torch.bfloat16, device=dev)
    K.prefill_varlen(dq[..., :128], dq[..., 128:], dkv[..., :128], dpe, dkv[..., 128:],
                     torch.tensor(cu_q, dtype=torch.int32, device=dev), torch.tensor(cu_k, dtype=torch.int32, device=dev),
                     max(q_lens), scale, causal, out_bf)
    # bf16 output: its rounding alone is 1.4e-3 of mean relative error; the probabilities go through P.V as fp16 (11
    # significant bits), which leaves the rest of the 2e-3 bar unused whatever the number of keys
    attn_close(out_bf, ref, 2e-2, 2e-3)
    # keys and values handed over as fp16 (what a caller with an fp16 up-projection GEMM has): both products on fp16, no
    # tile converted; the same numbers, so the same oracle, at the same bars
    out_h = torch.full((q.shape[0], n, 128), float("nan"), dtype=torch.float32, device=dev)
    lse_h = torch.full((q.shape[0], n), float("nan"), dtype=torch.float32, device=dev)
    hkv, hpe = dkv.to(torch.float16), dpe.to(torch.float16)
    K.prefill_varlen(dq[..., :128], dq[..., 128:], hkv[..., :128], hpe, hkv[..., 128:],
                     torch.tensor(cu_q, dtype=torch.int32, device=dev), torch.tensor(cu_k, dtype=torch.int32, device=dev),
                     max(q_lens), scale, causal, out_h, lse_h)
    attn_close(out_h, ref, 2e-2, 4e-4)
    assert torch.equal(torch.isfinite(lse_h.cpu()), fin) and torch.allclose(lse_h.cpu()[fin], ref_lse[fin], atol=2e-2)
    with pytest.raises(TypeError):                            # all three, or none
        K.prefill_varlen(dq[..., :128], dq[..., 128:], hkv[..., :128], dpe, dkv[..., 128:],
                         torch.tensor(cu_q, dtype=torch.int32, device=dev), torch.tensor(cu_k, dtype=torch.int32, device=dev),
                         max(q_lens), scale, causal, out_h)


def test_chunked_context_flow_gather_attend_merge(dev):
    """gather -> up-project -> unmasked attention with LSE -> two-way merges -> merge with the causal suffix
    (the loop of src/omni_npu/attention/backends/mla.py:377-450 and :573-616) equals the oracle's chunked prefill,
    on the reference test's schedule: context 48 = chunks [32,16], suffix 16."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(5)
    bsz, ctx, suf, n = 2, 48, 16, 4
    w = (torch.randn(512, n * 256, generator=g) * 0.02).bfloat16()
    nope = torch.randn(bsz, 128, 512, generator=g).bfloat16()
    rope = torch.randn(bsz, 128, 64, generator=g).bfloat16()
    bt = torch.tensor([[1], [0]], dtype=torch.int32)
    q = torch.randn(bsz * suf, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(bsz * suf, 512, generator=g).bfloat16(), torch.randn(bsz * suf, 64, generator=g).bfloat16()
    cu_q = torch.tensor([0, suf, 2 * suf], dtype=torch.int32)
    chunks = [(torch.tensor([0, 32, 64], dtype=torch.int32), torch.tensor([0, 0], dtype=torch.int32)),
              (torch.tensor([0, 16, 32], dtype=torch.int32), torch.tensor([32, 32], dtype=torch.int32))]
    scale = 192 ** -0.5
    ref = O.chunked_prefill(q, kvc, kpe, w, nope, rope, bt, cu_q.tolist(), chunks, scale)

    d = lambda x: x.to(dev)
    dq, dw = d(q), d(w)
    t = bsz * suf
    kv_s = (d(kvc) @ dw).view(t, n, 256)
    out_s = torch.empty(t, n, 128, dtype=torch.bfloat16, device=dev)
    lse_s = torch.empty(t, n, dtype=torch.float32, device=dev)
    K.prefill_varlen(dq[..., :128], dq[..., 128:], kv_s[..., :128], d(kpe), kv_s[..., 128:], d(cu_q), d(cu_q), suf, scale,
                     True, out_s, lse_s)
    ctx_out = ctx_lse = None
    ws = torch.empty(64, 576, dtype=torch.bfloat16, device=dev)
    for cu_k, starts in chunks:
        toks = int(cu_k[-1])
        K.gather_paged(d(nope), d(rope), ws, d(bt), d(cu_k), bsz, d(starts), total_rows=toks)
        kv_c = (ws[:toks, :512] @ dw).view(toks, n, 256)
        o_i = torch.empty(t, n, 128, dtype=torch.bfloat16, device=dev)
        l_i = torch.empty(t, n, dtype=torch.float32, device=dev)
        K.prefill_varlen(dq[..., :128], dq[..., 128:], kv_c[..., :128], ws[:toks, 512:], kv_c[..., 128:], d(cu_q), d(cu_k),
                         suf, scale, False, o_i, l_i)
        if ctx_out is None:
            ctx_out, ctx_lse = o_i, l_i
        else:
            o2, l2 = torch.empty_like(o_i), torch.empty_like(l_i)
            K.merge_states(ctx_out, ctx_lse, o_i, l_i, o2, l2)
            ctx_out, ctx_lse = o2, l2
    merged = torch.empty(t, n, 128, dtype=torch.float32, device=dev)
    K.merge_states(ctx_out, ctx_lse, out_s, lse_s, merged)
    # the reference's bar for this flow is atol = rtol = 3e-2 (tests/integration/attention/test_mla_chunked_prefill.py:72-76)
    attn_close(merged.view(t, -1), ref, 3e-2, 6e-3)


def test_chunked_context_flow_with_continued_launches(dev):
    """The same schedule with no merge launch: every context chunk's attention continues from the running result, and the
    causal suffix continues from the context's (mla_prefill_varlen_continue); in place (out is the earlier result)."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(5)
    bsz, ctx, suf, n = 2, 48, 16, 4
    w = (torch.randn(512, n * 256, generator=g) * 0.02).bfloat16()
    nope = torch.randn(bsz, 128, 512, generator=g).bfloat16()
    rope = torch.randn(bsz, 128, 64, generator=g).bfloat16()
    bt = torch.tensor([[1], [0]], dtype=torch.int32)
    q = torch.randn(bsz * suf, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(bsz * suf, 512, generator=g).bfloat16(), torch.randn(bsz * suf, 64, generator=g).bfloat16()
    cu_q = torch.tensor([0, suf, 2 * suf], dtype=torch.int32)
    chunks = [(torch.tensor([0, 32, 64], dtype=torch.int32), torch.tensor([0, 0], dtype=torch.int32)),
              (torch.tensor([0, 16, 32], dtype=torch.int32), torch.tensor([32, 32], dtype=torch.int32))]
    scale = 192 ** -0.5
    ref = O.chunked_prefill(q, kvc, kpe, w, nope, rope, bt, cu_q.tolist(), chunks, scale)
    d = lambda x: x.to(dev)
    dq, dw = d(q), d(w)
    t = bsz * suf
    run_o = torch.empty(t, n, 128, dtype=torch.float32, device=dev)
    run_l = torch.empty(t, n, dtype=torch.float32, device=dev)
    ws = torch.empty(64, 576, dtype=torch.bfloat16, device=dev)
    for i, (cu_k, starts) in enumerate(chunks):
        toks = int(cu_k[-1])
        K.gather_paged(d(nope), d(rope), ws, d(bt), d(cu_k), bsz, d(starts), total_rows=toks)
        kv_c = (ws[:toks, :512] @ dw).view(toks, n, 256)
        K.prefill_varlen(dq[..., :128], dq[..., 128:], kv_c[..., :128], ws[:toks, 512:], kv_c[..., 128:], d(cu_q), d(cu_k),
                         suf, scale, False, run_o, run_l, prev_out=run_o if i else None, prev_lse=run_l if i else None)
    kv_s = (d(kvc) @ dw).view(t, n, 256)
    out = torch.empty(t, n, 128, dtype=torch.bfloat16, device=dev)
    K.prefill_varlen(dq[..., :128], dq[..., 128:], kv_s[..., :128], d(kpe), kv_s[..., 128:], d(cu_q), d(cu_q), suf, scale,
                     True, out, prev_out=run_o, prev_lse=run_l)
    attn_close(out.view(t, -1), ref, 3e-2, 6e-3)


@pytest.mark.parametrize("n,q_lens,k1,k2,causal2", [(4, [5, 130, 64], [40, 0, 300], [7, 200, 0], False),
                                                    (16, [33, 1], [100, 64], [33, 1], True),
                                                    (2, [257], [0], [257], True)])
def test_prefill_continued_equals_attention_over_all_keys(dev, n, q_lens, k1, k2, causal2):
    """Two launches, the second continuing from the first, against ONE oracle attention over the concatenated keys: the
    first unmasked over k1 keys per sequence (some sequences have none: lse = -inf, the row starts empty), the second over
    k2 keys (causal: the sequence's own tokens, right-down aligned).  fp32 and bf16 output, log-sum-exp included; a launch
    without keys of its own returns the earlier result."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(n + len(q_lens))
    bf = lambda *sh: torch.randn(*sh, generator=g).bfloat16()
    t = sum(q_lens)
    cu_q = [0]
    for x in q_lens:
        cu_q.append(cu_q[-1] + x)
    cu1, cu2 = [0], [0]
    for a, b in zip(k1, k2):
        cu1.append(cu1[-1] + a)
        cu2.append(cu2[-1] + b)
    qn, qp = bf(t, n, 128), bf(t, n, 64)
    kn1, kp1, v1 = bf(cu1[-1], n, 128), bf(cu1[-1], 64), bf(cu1[-1], n, 128)
    kn2, kp2, v2 = bf(cu2[-1], n, 128), bf(cu2[-1], 64), bf(cu2[-1], n, 128)
    scale = 192 ** -0.5
    # the oracle over the union: keys of part 1 in front of the keys of part 2 (a causal part 2 is right-down aligned, so
    # part 1 is visible to every row)
    kn = torch.cat([torch.cat([kn1[cu1[i]:cu1[i + 1]], kn2[cu2[i]:cu2[i + 1]]]) for i in range(len(q_lens))])
    kp = torch.cat([torch.cat([kp1[cu1[i]:cu1[i + 1]], kp2[cu2[i]:cu2[i + 1]]]) for i in range(len(q_lens))])
    vv = torch.cat([torch.cat([v1[cu1[i]:cu1[i + 1]], v2[cu2[i]:cu2[i + 1]]]) for i in range(len(q_lens))])
    cu_all = [a + b for a, b in zip(cu1, cu2)]
    ref, ref_lse = O.attention_varlen(qn, qp, kn, kp, vv, cu_q, cu_all, scale, causal2)
    d = lambda x: x.to(dev)
    ti = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    o1 = torch.empty(t, n, 128, dtype=torch.float32, device=dev)
    l1 = torch.empty(t, n, dtype=torch.float32, device=dev)
    K.prefill_varlen(d(qn), d(qp), d(kn1), d(kp1), d(v1), ti(cu_q), ti(cu1), max(q_lens), scale, False, o1, l1)
    for dt in (torch.float32, torch.bfloat16):
        o2 = torch.full((t, n, 128), float("nan"), dtype=dt, device=dev)
        l2 = torch.empty(t, n, dtype=torch.float32, device=dev)
        K.prefill_varlen(d(qn), d(qp), d(kn2), d(kp2), d(v2), ti(cu_q), ti(cu2), max(q_lens), scale, causal2, o2, l2,
                         prev_out=o1, prev_lse=l1)
        attn_close(o2, ref, 2e-2, 4e-4 if dt == torch.float32 else 2e-3)
        fin = torch.isfinite(ref_lse)
        assert torch.equal(torch.isfinite(l2.cpu()), fin)
        assert torch.allclose(l2.cpu()[fin], ref_lse[fin], atol=2e-2, rtol=0)
    # nothing new to attend to: the earlier result comes back (through the kernel: cu_k all zero but keys present)
    o3 = torch.empty_like(o1)
    l3 = torch.empty_like(l1)
    K.prefill_varlen(d(qn), d(qp), d(kn2[:1] if cu2[-1] else kn1[:1]), d(kp2[:1] if cu2[-1] else kp1[:1]),
                     d(v2[:1] if cu2[-1] else v1[:1]), ti(cu_q), ti([0] * len(cu_q)), max(q_lens), scale, False, o3, l3,
                     prev_out=o1, prev_lse=l1)
    keep = torch.isfinite(l1)
    assert torch.equal(o3[keep], o1[keep]) and torch.equal(l3[keep], l1[keep])
    assert (o3[~keep] == 0).all() and torch.isinf(l3[~keep]).all()


def _random_prefill_cases(n_cases, seed):
    import random
    rng = random.Random(seed)
    cases = []
    for i in range(n_cases):
        b = rng.randint(1, 4)
        n = rng.choice([1, 2, 8, 16])
        causal = rng.random() < 0.6
        q_lens = [rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 200, 257]) for _ in range(b)]
        if causal:                                            # at least as many keys as queries (right-down alignment)
            k_lens = [q + rng.choice([0, 0, 1, 63, 64, 65, 300]) for q in q_lens]
        else:
            k_lens = [rng.choice([0, 1, 31, 64, 65, 129, 500]) for _ in range(b)]
        cases.append((i, causal, q_lens, k_lens, n))
    return cases


@pytest.mark.parametrize("i,causal,q_lens,k_lens,n", _random_prefill_cases(32, seed=7))
def test_prefill_varlen_random_shapes(dev, i, causal, q_lens, k_lens, n):
    """Seeded sweep over batch, heads, ragged query and key lengths around the 32 / 64 / 128 tile edges, with and
    without the causal mask (empty key ranges included: zeros and lse = -inf)."""
    from omni_npu_amd import kernels as K
    q, kv, k_pe, cu_q, cu_k = _case(500 + i, q_lens, k_lens, n)
    scale = 192 ** -0.5
    ref, ref_lse = O.attention_varlen(q[..., :128], q[..., 128:], kv[..., :128], k_pe.view(-1, 64), kv[..., 128:], cu_q,
                                      cu_k, scale, causal)
    dq, dkv, dpe = q.to(dev), kv.to(dev), k_pe.to(dev)
    out = torch.full((q.shape[0], n, 128), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((q.shape[0], n), float("nan"), dtype=torch.float32, device=dev)
    K.prefill_varlen(dq[..., :128], dq[..., 128:], dkv[..., :128], dpe, dkv[..., 128:],
                     torch.tensor(cu_q, dtype=torch.int32, device=dev), torch.tensor(cu_k, dtype=torch.int32, device=dev),
                     max(q_lens), scale, causal, out, lse)
    attn_close(out, ref, 2e-2, 4e-4)                          # fp32 result: only the fp16 rounding of P (2^-12 each) is left
    got_lse = lse.cpu()
    fin = torch.isfinite(ref_lse)
    assert torch.equal(torch.isfinite(got_lse), fin)
    assert torch.allclose(got_lse[fin], ref_lse[fin], atol=2e-2)



@pytest.mark.parametrize("seed", [0, 1, 2])
def test_flat_attention_over_unrelated_values_keeps_the_bf16_bar(dev, seed):
    """The recipe of the chunked-prefill benchmark, reduced: q, k and v independent N(0,1), scale 1/sqrt(192), a 256-token
    chunk over 4096 cached keys continued by the causal suffix.  Scores then have unit variance (flat softmax) and the
    values have nothing to do with the keys: the case in which probabilities rounded to bf16 cost 1.7e-3 by themselves
    and a bf16 result cannot meet 2e-3.  With fp16 probabilities the bf16 result stays below 1.6e-3."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(100 + seed)
    n, q_len, ctx = 4, 256, 4096
    scale = 192 ** -0.5
    bf = lambda *shape: torch.randn(*shape, generator=g).bfloat16()
    qn, qp = bf(q_len, n, 128), bf(q_len, n, 64)
    kc_n, kc_p, vc = bf(ctx, n, 128), bf(ctx, 64), bf(ctx, n, 128)
    ks_n, ks_p, vs = bf(q_len, n, 128), bf(q_len, 64), bf(q_len, n, 128)
    ref, _ = O.attention_varlen(qn, qp, torch.cat([kc_n, ks_n]), torch.cat([kc_p, ks_p]), torch.cat([vc, vs]), [0, q_len],
                                [0, ctx + q_len], scale, True)
    d = lambda x: x.to(dev)
    ti = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    o_c = torch.empty(q_len, n, 128, dtype=torch.float32, device=dev)
    l_c = torch.empty(q_len, n, dtype=torch.float32, device=dev)
    out = torch.empty(q_len, n, 128, dtype=torch.bfloat16, device=dev)
    K.prefill_varlen(d(qn), d(qp), d(kc_n), d(kc_p), d(vc), ti([0, q_len]), ti([0, ctx]), q_len, scale, False, o_c, l_c)
    K.prefill_varlen(d(qn), d(qp), d(ks_n), d(ks_p), d(vs), ti([0, q_len]), ti([0, q_len]), q_len, scale, True, out,
                     prev_out=o_c, prev_lse=l_c)
    ma, mr = attn_close(out, ref, 2e-2, 2e-3)
    assert mr <= 1.6e-3, f"mean_rel={mr:.4g}: the headroom that fp16 probabilities buy is gone"


def test_values_outside_the_fp16_range_saturate_and_stay_finite(dev):
    """V goes through P.V as fp16: magnitudes above 65504 saturate there (never an infinity), magnitudes below 2^-14
    lose at most 2^-25 absolute.  Rows that only see ordinary values are not affected by an outlier elsewhere."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(7)
    n, q_len = 2, 64
    scale = 192 ** -0.5
    bf = lambda *shape: torch.randn(*shape, generator=g).bfloat16()
    qn, qp, kn, kp, v = bf(q_len, n, 128), bf(q_len, n, 64), bf(q_len, n, 128), bf(q_len, 64), bf(q_len, n, 128)
    v[40, 0, 3] = 3.0e38                                      # far beyond fp16
    v[41, 1, 5] = 1.0e-7                                      # an fp16 denormal
    v[42, 1, 6] = 0.0
    ref, _ = O.attention_varlen(qn, qp, kn, kp, v, [0, q_len], [0, q_len], scale, True)
    d = lambda x: x.to(dev)
    ti = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    out = torch.empty(q_len, n, 128, dtype=torch.float32, device=dev)
    K.prefill_varlen(d(qn), d(qp), d(kn), d(kp), d(v), ti([0, q_len]), ti([0, q_len]), q_len, scale, True, out)
    got = out.cpu()
    assert torch.isfinite(got).all()
    mask = torch.ones_like(ref, dtype=torch.bool)
    mask[40:, 0, 3] = False                                   # the rows that see the outlier, in its column
    attn_close(got[mask].view(1, -1), ref[mask].view(1, -1), 2e-2, 4e-4)
    sat = got[40:, 0, 3]
    assert (sat > 0).all() and (sat <= 65504.0 * 1.001).all()
