"""The benchmark configurations at their FULL shapes, each checked against the oracle on a sample of its rows and through
properties that do not depend on size.

  * chunked prefill: 128 heads, 4 sequences, a 2048-token chunk each over a 16384-token paged prefix (gather of the
    latent prefix, K/V up-projection, context attention without a mask, causal attention over the chunk, merge);
    the up-projected K/V tensor of the prefix is 2^32 bytes.
  * DSA decode: batch 32, contexts uniform[32768, 65536], 64 fp8 index heads, top-2048, sparse MLA over the picks; the
    index keys and queries are N(0,1) values put through the per-token e4m3 quantiser.
  * fp8-cache decode: batch 256, MTP pairs, contexts uniform[16384, 32768], the step (cache write + decode) replayed from
    a captured HIP graph.

Tolerances: attention outputs max-abs 2e-2 / mean-rel 2e-3 (6e-2 / 6e-3 over the fp8 cache), indexer logits 1e-4 of the
row's largest |logit|, integer results bit-exact.
"""
import pytest
import torch

from oracle import mla_oracle as O
from tests.conftest import attn_close

pytestmark = pytest.mark.gpu


def _paged_tables(lens, g, page=128):
    nblk_seq = (lens + page - 1) // page
    nblk = int(nblk_seq.sum())
    perm = torch.randperm(nblk, generator=g).to(torch.int32)
    bt = torch.zeros(lens.numel(), int(nblk_seq.max()), dtype=torch.int32)
    o = 0
    for b in range(lens.numel()):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n]
        o += n
    return bt, nblk


def test_chunked_prefill_full_shape(dev):
    """The whole chunked-prefill flow at 128 heads, 4 x 2048 queries over 4 x 16384 cached tokens.  Four (sequence, head)
    pairs are recomputed by the oracle as ONE causal attention over prefix + chunk keys (all 2048 query rows each), so
    the context pass, the causal pass and the merge are all inside the comparison; the pairs of sequences 2 and 3 read
    K/V beyond byte offset 2^31."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(2)
    B, N, Q, C = 4, 128, 2048, 16384
    scale = 192 ** -0.5
    pages = B * C // 128
    nope = torch.randn(pages, 128, 512, generator=g).bfloat16()
    rope = torch.randn(pages, 128, 64, generator=g).bfloat16()
    bt = torch.randperm(pages, generator=g).to(torch.int32).view(B, C // 128)
    w = (torch.randn(512, N * 256, generator=g) * 512 ** -0.5).bfloat16()       # up-projected K/V of unit scale
    q = torch.randn(B * Q, N, 192, generator=g).bfloat16()
    kv_c_s = torch.randn(B * Q, 512, generator=g).bfloat16()
    k_pe_s = torch.randn(B * Q, 64, generator=g).bfloat16()

    d = lambda x: x.to(dev)
    nope_d, rope_d, w_d, q_d = d(nope), d(rope), d(w), d(q)
    cu_q = torch.arange(0, (B + 1) * Q, Q, dtype=torch.int32, device=dev)
    cu_c = torch.arange(0, (B + 1) * C, C, dtype=torch.int32, device=dev)
    gathered = torch.empty(B * C, 576, dtype=torch.bfloat16, device=dev)
    K.gather_paged(nope_d, rope_d, gathered, d(bt), cu_c, B)
    kv_c = torch.matmul(gathered[:, :512], w_d).view(B * C, N, 256)
    assert kv_c.numel() * 2 >= 2 ** 32
    kv_s = torch.matmul(d(kv_c_s), w_d).view(B * Q, N, 256)
    o_c = torch.empty(B * Q, N, 128, dtype=torch.float32, device=dev)       # fp32 partials, bf16 result, as the backend runs it
    o_s, o = torch.empty_like(o_c), torch.empty(B * Q, N, 128, dtype=torch.bfloat16, device=dev)
    l_c = torch.empty(B * Q, N, dtype=torch.float32, device=dev)
    l_s = torch.empty_like(l_c)
    K.prefill_varlen(q_d[..., :128], q_d[..., 128:], kv_c[..., :128], gathered[:, 512:], kv_c[..., 128:], cu_q, cu_c, Q,
                     scale, False, o_c, l_c)
    K.prefill_varlen(q_d[..., :128], q_d[..., 128:], kv_s[..., :128], d(k_pe_s), kv_s[..., 128:], cu_q, cu_q, Q, scale,
                     True, o_s, l_s)
    K.merge_states(o_c, l_c, o_s, l_s, o)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()

    for b, h in ((0, 0), (1, 37), (2, 127), (3, 64)):
        ctx_rows = O.slots_for(bt, b, 0, C)
        lat = torch.cat([nope.view(-1, 512)[ctx_rows], kv_c_s[b * Q:(b + 1) * Q]]).float()
        pe = torch.cat([rope.view(-1, 64)[ctx_rows], k_pe_s[b * Q:(b + 1) * Q]])
        kv = (lat @ w[:, h * 256:(h + 1) * 256].float()).bfloat16().view(C + Q, 1, 256)     # the GEMM's output is bf16
        qh = q[b * Q:(b + 1) * Q, h:h + 1]
        ref, _ = O.attention_varlen(qh[..., :128], qh[..., 128:], kv[..., :128], pe, kv[..., 128:], [0, Q], [0, C + Q],
                                    scale, True)
        attn_close(o[b * Q:(b + 1) * Q, h:h + 1], ref, 2e-2, 2e-3)
        # the gathered latent is a bit-exact copy of the paged rows
        assert torch.equal(gathered[b * C:(b + 1) * C, :512].cpu(), nope.view(-1, 512)[ctx_rows])


def test_dsa_decode_full_shape(dev):
    """Indexer -> top-2048 -> rows -> sparse MLA at batch 32 over 32k-64k contexts on quantised N(0,1) keys and queries.
    Three tokens have their whole logit row recomputed by the oracle; every token's pick set is compared with the oracle's
    stable top-k of the SAME logits and with the single-workgroup variant of the kernel, bit for bit; rows are the picks
    mapped through the block table; the sparse attention of the sampled tokens equals the oracle's on the picked rows."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(3)
    B, H, N, k = 32, 64, 128, 2048
    lens = torch.randint(32768, 65537, (B,), generator=g).to(torch.int32)
    bt, nblk = _paged_tables(lens, g)
    sample = (0, 13, 31)
    # index keys: N(0,1) bf16 rows quantised per token by the product's kernel, a sequence at a time; the sampled
    # sequences keep their source rows for the oracle's quantiser
    k8 = torch.zeros(nblk, 128, 128, dtype=torch.uint8, device=dev)
    ks = torch.zeros(nblk, 128, dtype=torch.float32, device=dev)
    btd, lensd = bt.to(dev), lens.to(dev)
    src = {}
    torch.manual_seed(3)
    for b in range(B):
        L = int(lens[b])
        x = torch.randn(L, 128, device=dev).bfloat16()
        pos = torch.arange(L, device=dev)
        slots = btd[b, pos // 128].long() * 128 + pos % 128
        K.quant_rows_fp8(x, k8, ks, slot_mapping=slots)
        if b in sample:
            src[b] = x.cpu()
    qf = torch.randn(B, H, 128, generator=g)
    q8, qs = O.fp8_quant_token(qf)
    w = torch.randn(B, H, generator=g)
    max_len = int(lens.max())
    logits = torch.full((B, K.indexer_logits_stride(max_len)), float("nan"), device=dev)
    K.indexer_scores(q8.to(dev), w.to(dev), k8, ks, btd, lensd, logits, q_scale=qs.to(dev), max_seq_len=max_len)
    idx = torch.full((B, k), -7, dtype=torch.int32, device=dev)
    rows = torch.full((B, k), -7, dtype=torch.int32, device=dev)
    counts = torch.full((B,), -7, dtype=torch.int32, device=dev)
    K.topk(logits, lensd, k, idx, block_table=btd, page_size=128, num_pages=nblk, rows=rows, counts=counts)
    idx1 = torch.full((B, k), -7, dtype=torch.int32, device=dev)
    K.topk(logits, lensd, k, idx1, single_workgroup=True)
    torch.cuda.synchronize()
    assert torch.equal(idx, idx1)
    lg, idx_c, rows_c = logits.cpu(), idx.cpu(), rows.cpu()
    assert counts.cpu().tolist() == [k] * B
    for b in range(B):
        L = int(lens[b])
        want = O.topk_stable(lg[b], k, L)
        assert idx_c[b].tolist() == sorted(want.tolist()), f"token {b}: pick set differs from the stable top-k"
        pos = idx_c[b].long()
        assert torch.equal(rows_c[b].long(), bt[b, pos // 128].long() * 128 + pos % 128)
    for b in sample:
        L = int(lens[b])
        ref8, ref_s = O.fp8_quant_token(src[b])
        phys = O.slots_for(bt, b, 0, L).to(dev)
        assert torch.equal(k8.view(-1, 128)[phys].cpu(), ref8.view(torch.uint8))        # the quantiser, bit for bit
        assert torch.equal(ks.view(-1)[phys].cpu(), ref_s)
        ref = O.indexer_scores(q8[b], qs[b], ref8, ref_s, w[b])
        assert (lg[b, :L] - ref).abs().max().item() <= 1e-4 * ref.abs().max().item()
        # the picks are where the oracle's own logits are largest too: the k-th largest reference logit bounds them
        kth = torch.topk(ref, k).values[-1].item()
        assert (ref[idx_c[b].long()] >= kth - 2e-4 * ref.abs().max().item()).all()

    nope = torch.randn(nblk, 128, 512, device=dev).bfloat16()
    rope = torch.randn(nblk, 128, 64, device=dev).bfloat16()
    qn = torch.randn(B, N, 512, generator=g).bfloat16()
    qr = torch.randn(B, N, 64, generator=g).bfloat16()
    scale = 192 ** -0.5
    out = torch.empty(B, N, 512, dtype=torch.bfloat16, device=dev)
    K.sparse_decode(qn.to(dev), qr.to(dev), nope, rope, rows, counts, scale, out)
    out1 = torch.empty_like(out)
    K.sparse_decode(qn.to(dev), qr.to(dev), nope, rope, rows, counts, scale, out1, num_splits=1)
    torch.cuda.synchronize()
    assert (out.float() - out1.float()).abs().max().item() <= 8e-3            # invariance under the split count
    for b in sample:
        r = rows[b].long()
        small_n = nope.view(-1, 512)[r].cpu().view(k // 128, 128, 512)       # the picked rows as a 16-page cache
        small_r = rope.view(-1, 64)[r].cpu().view(k // 128, 128, 64)
        ref = O.sparse_decode(qn[b:b + 1], qr[b:b + 1], small_n, small_r, torch.arange(k // 128, dtype=torch.int32)[None],
                              torch.tensor([k], dtype=torch.int32), torch.arange(k, dtype=torch.int32)[None], scale)
        attn_close(out[b:b + 1], ref, 2e-2, 2e-3)


def test_fp8_decode_full_shape_under_graph_replay(dev):
    """Batch 256, MTP pairs, contexts 16k-32k over the fp8 cache: the step (quantising write of the 512 new tokens +
    decode) is captured once and replayed three times with eager work in between; every replay equals the eager step
    bit for bit, three sequences equal the oracle run on the oracle-quantised values of the same rows, and the result
    is invariant under the split count."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(4)
    B, N, QL = 256, 128, 2
    lens = torch.randint(16384, 32769, (B,), generator=g).to(torch.int32)
    bt, nblk = _paged_tables(lens, g)
    btd, lensd = bt.to(dev), lens.to(dev)
    sample = (0, 100, 255)
    cache = torch.zeros(nblk, 128, K.FP8_ROW_BYTES, dtype=torch.uint8, device=dev)
    src = {}
    torch.manual_seed(4)
    for b in range(B):
        L = int(lens[b])
        c, r = torch.randn(L, 512, device=dev).bfloat16(), torch.randn(L, 64, device=dev).bfloat16()
        pos = torch.arange(L, device=dev)
        K.cache_write_fp8(c, r, btd[b, pos // 128].long() * 128 + pos % 128, cache)
        if b in sample:
            src[b] = (c.cpu(), r.cpu())
    T = B * QL
    qn = torch.randn(T, N, 512, generator=g).bfloat16()
    qr = torch.randn(T, N, 64, generator=g).bfloat16()
    new_c = torch.randn(T, 512, generator=g).bfloat16()
    new_r = torch.randn(T, 64, generator=g).bfloat16()
    slots = torch.cat([O.slots_for(bt, b, int(lens[b]) - QL, int(lens[b])) for b in range(B)])
    qn_d, qr_d, nc_d, nr_d, slots_d = qn.to(dev), qr.to(dev), new_c.to(dev), new_r.to(dev), slots.to(dev)
    out = torch.empty(T, N, 512, dtype=torch.bfloat16, device=dev)
    max_len = bt.shape[1] * 128
    splits = K.default_num_splits(B, QL, N, max_len)
    scale = 192 ** -0.5

    def step(s=splits):
        K.cache_write_fp8(nc_d, nr_d, slots_d, cache)
        K.decode_fp8(qn_d, qr_d, cache, btd, lensd, scale, out, q_len=QL, num_splits=s, max_seq_len=max_len)

    step()
    torch.cuda.synchronize()
    eager = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for trial in range(3):
        out.zero_()
        scratch = torch.randn(1 << 20, device=dev).sum()           # eager work between the replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {trial} differs from the eager step"
        del scratch
    step(max(1, splits - 1) if splits > 1 else 2)
    torch.cuda.synchronize()
    assert (out.float() - eager.float()).abs().max().item() <= 8e-3
    for b in sample:
        L = int(lens[b])
        c, r = src[b]
        c, r = c.clone(), r.clone()
        c[L - QL:], r[L - QL:] = new_c[b * QL:(b + 1) * QL], new_r[b * QL:(b + 1) * QL]
        q8, sc = O.fp8_quant_block(c.float())
        npg = (L + 127) // 128
        deq = torch.zeros(npg * 128, 512)
        deq[:L] = O.fp8_dequant_block(q8, sc)
        rp = torch.zeros(npg * 128, 64, dtype=torch.bfloat16)
        rp[:L] = r
        ref = O.absorbed_decode(qn[b * QL:(b + 1) * QL], qr[b * QL:(b + 1) * QL], deq.view(npg, 128, 512),
                                rp.view(npg, 128, 64), torch.arange(npg, dtype=torch.int32)[None],
                                lens[b:b + 1], scale)
        attn_close(eager[b * QL:(b + 1) * QL], ref, 6e-2, 6e-3)
