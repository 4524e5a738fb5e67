"""Caches larger than 4 GiB: every kernel that takes a paged cache is run with the pages it touches spread over an
allocation whose byte offsets pass 2^32 (and whose element offsets pass 2^31), including the pages that straddle those
boundaries and the last page of the allocation.  A serving process on a 288 GB device holds caches of this size and
larger; an address computed in 32 bits would read or write somewhere else.

The inputs are the small seeded cases of the other tests; only the page numbers are mapped far apart, so the oracle
still runs on the small tensors.  The big allocations are never initialised as a whole (torch.empty) and never copied
to the host."""
import pytest
import torch

from oracle import mla_oracle as O
from tests.conftest import attn_close

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_REL = 2e-2, 2e-3


def _far_pages(n_small: int, n_big: int, page_bytes: int, seed: int) -> torch.Tensor:
    """n_small distinct page numbers in [0, n_big): the last two pages, the pages on either side of the 2^31- and
    2^32-byte offsets, page 0, and random ones, in random order."""
    g = torch.Generator().manual_seed(seed)
    must = {0, n_big - 1, n_big - 2}
    for boundary in (1 << 31, 1 << 32):
        pg = boundary // page_bytes
        must.update(x for x in (pg - 1, pg, pg + 1) if 0 <= x < n_big)
    must = sorted(must)[:n_small]
    rest = [int(x) for x in torch.randperm(n_big, generator=g)[:n_small + len(must)].tolist() if x not in set(must)]
    ids = torch.tensor((must + rest)[:n_small], dtype=torch.int64)
    assert ids.unique().numel() == n_small
    return ids[torch.randperm(n_small, generator=g)]


def _slots_of_all_rows(far: torch.Tensor, page: int = 128) -> torch.Tensor:
    return (far[:, None] * page + torch.arange(page)[None, :]).reshape(-1)


def test_bf16_cache_beyond_4gib_write_decode_sparse_gather(dev):
    from omni_npu_amd import kernels as K
    c = O.make_decode_case(4, 128, 200, 900, seed=11)
    n_small = c["nope"].shape[0]
    n_big = 40_000                                            # 40 000 x 128 x 512 x 2 B = 5.24 GB of nope pages
    far = _far_pages(n_small, n_big, 128 * 512 * 2, seed=1)
    nope = torch.empty(n_big, 128, 512, dtype=torch.bfloat16, device=dev)
    rope = torch.empty(n_big, 128, 64, dtype=torch.bfloat16, device=dev)
    assert nope.numel() * 2 > (1 << 32) and int(far.max()) * 128 * 512 > (1 << 31)

    # cache write to far slots, read back bit-exact
    slots = _slots_of_all_rows(far)
    K.cache_write(c["nope"].view(-1, 512).to(dev), c["rope"].view(-1, 64).to(dev), slots.to(dev), nope, rope)
    torch.cuda.synchronize()
    far_d = far.to(dev)
    assert torch.equal(nope[far_d].cpu(), c["nope"]) and torch.equal(rope[far_d].cpu(), c["rope"])

    # dense decode over the far pages
    bt_far = far[c["block_table"].long()].to(torch.int32)
    out = torch.full((4, 128, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode(c["q_nope"].to(dev), c["q_rope"].to(dev), nope, rope, bt_far.to(dev), c["seq_lens"].to(dev), c["scale"], out,
             q_len=1, num_splits=2)
    ref = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    attn_close(out, ref, MAX_ABS, MEAN_REL)

    # the same with a sliding window of 100 keys behind the first page taken as the sink (the blocks in between are skipped)
    out_w = torch.full((4, 128, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode(c["q_nope"].to(dev), c["q_rope"].to(dev), nope, rope, bt_far.to(dev), (c["seq_lens"] - 128).to(dev), c["scale"],
             out_w, q_len=1, num_splits=2, sink_len=128, window=100)
    ref_w = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"] - 128, 128, c["scale"], 100)
    attn_close(out_w, ref_w, MAX_ABS, MEAN_REL)

    # sparse decode: every third position of each sequence, named by flat cache rows of the big allocation
    k = 320
    idx = torch.full((4, k), -1, dtype=torch.int32)
    rows = torch.zeros(4, k, dtype=torch.int32)
    counts = torch.zeros(4, dtype=torch.int32)
    for b in range(4):
        pos = torch.arange(0, int(c["seq_lens"][b]), 3)[:k]
        idx[b, :pos.numel()] = pos.to(torch.int32)
        rows[b, :pos.numel()] = (bt_far[b, pos // 128].long() * 128 + pos % 128).to(torch.int32)
        counts[b] = pos.numel()
    assert int(rows.max()) * 1024 > (1 << 32)
    out_s = torch.full((4, 128, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.sparse_decode(c["q_nope"].to(dev), c["q_rope"].to(dev), nope, rope, rows.to(dev), counts.to(dev), c["scale"], out_s,
                    num_splits=2)
    ref_s = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx, c["scale"])
    attn_close(out_s, ref_s, MAX_ABS, MEAN_REL)

    # paged gather
    cu = torch.zeros(5, dtype=torch.int32)
    cu[1:] = torch.cumsum(c["seq_lens"], 0)
    total = int(cu[-1])
    dst = torch.zeros(total, 576, dtype=torch.bfloat16, device=dev)
    K.gather_paged(nope, rope, dst, bt_far.to(dev), cu.to(dev), 4)
    want = torch.zeros(total, 576, dtype=torch.bfloat16)
    O.gather_paged(c["nope"], c["rope"], want, c["block_table"], cu, 4)
    assert torch.equal(dst.cpu(), want)


def test_fused_norm_rope_cache_write_beyond_4gib(dev):
    from omni_npu_amd import kernels as K
    t, eps = 96, 1e-6
    g = torch.Generator().manual_seed(5)
    kv = (torch.randn(t, 576, generator=g) * 2).bfloat16()
    gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    cos, sin = O.rope_tables(torch.randint(0, 8192, (t,), generator=g), layout="half")
    n_big = 40_000
    far = _far_pages(8, n_big, 128 * 512 * 2, seed=2)        # the first eight: boundary pages, last pages, page 0
    slots = far[torch.arange(t) % 8] * 128 + torch.randperm(128, generator=g)[:t]
    nope = torch.empty(n_big, 128, 512, dtype=torch.bfloat16, device=dev)
    rope = torch.empty(n_big, 128, 64, dtype=torch.bfloat16, device=dev)
    kv_a_out = torch.empty(t, 512, dtype=torch.bfloat16, device=dev)
    k_pe_out = torch.empty(t, 64, dtype=torch.bfloat16, device=dev)
    K.kv_rmsnorm_rope_cache(kv.to(dev), gamma.to(dev), cos.to(dev), sin.to(dev), slots.to(dev), nope, rope, eps=eps,
                            table="half", interleaved_out=False, kv_a_out=kv_a_out, k_pe_out=k_pe_out)
    torch.cuda.synchronize()
    # the rows written at the far slots are the plain outputs (whose values the other tests pin against the oracle)
    sl = slots.to(dev)
    assert torch.equal(nope.view(-1, 512)[sl], kv_a_out) and torch.equal(rope.view(-1, 64)[sl], k_pe_out)
    k_pe_ref, kv_a_ref = O.kv_rmsnorm_rope_cache(kv, gamma, cos, sin, torch.full((t,), -1), torch.zeros(1, 128, 512).bfloat16(),
                                                 torch.zeros(1, 128, 64).bfloat16(), eps, table="half", interleaved_out=False)
    assert (kv_a_out.cpu().view(torch.int16).int() - kv_a_ref.view(torch.int16).int()).abs().max() <= 1
    assert (k_pe_out.cpu().view(torch.int16).int() - k_pe_ref.view(torch.int16).int()).abs().max() <= 1


def test_fp8_cache_beyond_4gib_write_and_decode(dev):
    from omni_npu_amd import kernels as K
    c = O.make_decode_case(3, 128, 300, 800, seed=13, q_len=2)
    q8, sc = O.fp8_quant_block(c["nope"].float())
    nope_deq = O.fp8_dequant_block(q8, sc)
    n_small = c["nope"].shape[0]
    n_big = 56_000                                            # 56 000 x 128 x 656 B = 4.70 GB
    far = _far_pages(n_small, n_big, 128 * 656, seed=3)
    cache = torch.empty(n_big, 128, 656, dtype=torch.uint8, device=dev)
    assert cache.numel() > (1 << 32)
    K.cache_write_fp8(c["nope"].view(-1, 512).to(dev), c["rope"].view(-1, 64).to(dev), _slots_of_all_rows(far).to(dev), cache)
    bt_far = far[c["block_table"].long()].to(torch.int32)
    out = torch.full((6, 128, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode_fp8(c["q_nope"].to(dev), c["q_rope"].to(dev), cache, bt_far.to(dev), c["seq_lens"].to(dev), c["scale"], out,
                 q_len=2, num_splits=2)
    ref = O.absorbed_decode(c["q_nope"], c["q_rope"], nope_deq, c["rope"], c["block_table"], c["seq_lens"], c["scale"])
    attn_close(out, ref, 6e-2, 6e-3)


def test_indexer_key_cache_beyond_4gib(dev):
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(17)
    batch, heads, page = 3, 64, 128
    lens = torch.tensor([700, 1500, 129], dtype=torch.int32)
    nblk_seq = (lens + page - 1) // page
    n_small = int(nblk_seq.sum())
    bt = torch.zeros(batch, int(nblk_seq.max()), dtype=torch.int32)
    perm = torch.randperm(n_small, generator=g)
    o = 0
    for b in range(batch):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n].to(torch.int32)
        o += n
    k8, ks = O.fp8_quant_token(torch.randn(n_small, page, 128, generator=g))
    q8, qs = O.fp8_quant_token(torch.randn(batch, heads, 128, generator=g))
    w = torch.randn(batch, heads, generator=g)
    n_big = 270_000                                           # 270 000 x 128 x 128 B = 4.42 GB of fp8 keys
    far = _far_pages(n_small, n_big, page * 128, seed=4)
    k8_big = torch.empty(n_big, page, 128, dtype=torch.uint8, device=dev)
    ks_big = torch.empty(n_big, page, dtype=torch.float32, device=dev)
    assert k8_big.numel() > (1 << 32)
    far_d = far.to(dev)
    k8_big[far_d] = k8.view(torch.uint8).to(dev)
    ks_big[far_d] = ks.to(dev)
    bt_far = far[bt.long()].to(torch.int32)
    max_len = int(lens.max())
    logits = torch.full((batch, K.indexer_logits_stride(max_len)), float("nan"), device=dev)
    K.indexer_scores(q8.to(dev), w.to(dev), k8_big, ks_big, bt_far.to(dev), lens.to(dev), logits, q_len=1,
                     q_scale=qs.to(dev), max_seq_len=max_len)
    got = logits.cpu()
    for b in range(batch):
        L = int(lens[b])
        rows = O.slots_for(bt, b, 0, L)
        ref = O.indexer_scores(q8[b], qs[b], k8.view(-1, 128)[rows], ks.reshape(-1)[rows], w[b])
        tol = 1e-4 * float(ref.abs().max()) + 1e-6
        assert (got[b, :L] - ref).abs().max().item() <= tol
