"""DSA path on the GPU: lightning-indexer logits, exact top-k, row translation and sparse MLA vs the oracle.

The reference's own tests for these ops are mocks (tests/unit/layers/test_npu_dsa.py:122-138), so the oracle here is
pinned only against the mathematics (see tests/test_oracle.py); tolerances: logits rel 1e-4 of the row's max |logit|
(fp32 accumulation order differs), top-k sets bit-exact on identical logits, attention 2e-2 / 2e-3.
"""
import pytest
import torch

from oracle import mla_oracle as O
from tests.conftest import attn_close

pytestmark = pytest.mark.gpu


def make_indexer_case(batch, lo, hi, seed, q_len=1, heads=64, page=128):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (batch,), generator=g)
    nblk_seq = (lens + page - 1) // page
    nblk = int(nblk_seq.sum())
    perm = torch.randperm(nblk, generator=g)
    bt = torch.zeros(batch, int(nblk_seq.max()), dtype=torch.int32)
    o = 0
    for b in range(batch):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n].to(torch.int32)
        o += n
    k = torch.randn(nblk, page, 128, generator=g)
    k8, ks = O.fp8_quant_token(k)
    t = batch * q_len
    q = torch.randn(t, heads, 128, generator=g)
    q8, qs = O.fp8_quant_token(q)
    w = torch.randn(t, heads, generator=g)
    return dict(seq_lens=lens.to(torch.int32), block_table=bt, k8=k8, k_scale=ks, q8=q8, q_scale=qs, w=w, q_len=q_len)


def logits_tol(c, t, ref):
    """1e-4 of the row's largest logit, plus 1e-5 of the largest magnitude that went into a logit (the same sum with |w|):
    with one to three visible keys every logit of a row can come out near zero by cancellation between heads, and the
    fp32 summation error does not shrink with it."""
    abs_c = dict(c)
    abs_c["w"] = c["w"].abs()
    return 1e-4 * ref.abs().max().item() + 1e-5 * oracle_logits(abs_c, t).max().item() + 1e-6


def oracle_logits(c, t):
    q_len = c["q_len"]
    b, i = divmod(t, q_len)
    L = int(c["seq_lens"][b])
    vis = L - q_len + i + 1
    rows = O.slots_for(c["block_table"], b, 0, vis)
    k8 = c["k8"].view(-1, 128)[rows]
    ks = c["k_scale"].reshape(-1)[rows]
    return O.indexer_scores(c["q8"][t], c["q_scale"][t], k8, ks, c["w"][t])


@pytest.mark.parametrize("batch,lo,hi,q_len", [(3, 1, 200, 1), (4, 1000, 5000, 1), (2, 300, 700, 2)])
def test_indexer_logits(dev, batch, lo, hi, q_len):
    from omni_npu_amd import kernels as K
    c = make_indexer_case(batch, lo, hi, seed=batch, q_len=q_len)
    t = batch * q_len
    max_len = int(c["seq_lens"].max())
    logits = torch.full((t, K.indexer_logits_stride(max_len)), float("nan"), device=dev)
    K.indexer_scores(c["q8"].to(dev), c["w"].to(dev), c["k8"].to(dev), c["k_scale"].to(dev), c["block_table"].to(dev),
                     c["seq_lens"].to(dev), logits, q_len=q_len, q_scale=c["q_scale"].to(dev), max_seq_len=max_len)
    got = logits.cpu()
    for tt in range(t):
        ref = oracle_logits(c, tt)
        n = ref.numel()
        assert (got[tt, :n] - ref).abs().max().item() <= logits_tol(c, tt, ref)
        pad_end = min((n + 31) // 32 * 32, got.shape[1])
        assert torch.isinf(got[tt, n:pad_end]).all() and (got[tt, n:pad_end] < 0).all()


@pytest.mark.parametrize("single_workgroup", [False, True], ids=["multi-workgroup", "single-workgroup"])
@pytest.mark.parametrize("n,k", [(5000, 2048), (100, 2048), (2048, 2048), (2049, 2048), (70000, 2048), (3000, 7), (20000, 2048),
                                 (9001, 300), (131071, 2048)])
def test_topk_bit_exact_sets_and_ties(dev, n, k, single_workgroup):
    """Identical scores in, identical index set out; heavy ties (quantised scores) go to the lower index.  Rows 1-3
    are the degenerate inputs (few distinct values) that take the radix-select paths of both variants; row 4 carries
    infinities and a huge outlier, which the linear binning must survive."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(n)
    rows = 5
    x = torch.randn(rows, n, generator=g)
    x[4, 1::97] = float("inf")
    x[4, 2::89] = float("-inf")
    x[4, 3] = 1e30
    x[1] = torch.round(x[1] * 4) / 4                       # many exact ties, including +-0
    x[1, ::5] = -0.0
    x[2] = 1.0                                             # all equal: the first k positions win
    x[3, : n // 2] = x[3, n // 2: 2 * (n // 2)]            # every value twice
    lens = torch.tensor([n, n, n, max(1, n - 3), n], dtype=torch.int32)
    out = torch.full((rows, 1, k), -7, dtype=torch.int32, device=dev)
    K.topk(x.to(dev), lens.to(dev), k, out, single_workgroup=single_workgroup)
    got = out.cpu().view(rows, k)
    for r in range(rows):
        ref = O.topk_stable(x[r], k, int(lens[r]))
        ref_set = sorted(i for i in ref.tolist() if i >= 0)
        g_valid = [i for i in got[r].tolist() if i >= 0]
        assert g_valid == ref_set, f"row {r}: selection differs"
        assert (got[r, len(g_valid):] == -1).all()


@pytest.mark.parametrize("single_workgroup", [False, True], ids=["multi-workgroup", "single-workgroup"])
def test_topk_rows_equals_topk_then_build_rows(dev, single_workgroup):
    """The fused launch writes the same positions, the same flat cache rows and the same counts as dsa_topk followed
    by dsa_build_rows (bit-exact integer work)."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(11)
    lens = torch.tensor([20000, 150, 9000, 2048, 2049], dtype=torch.int32)
    k, page = 2048, 128
    nblk_seq = (lens + page - 1) // page
    nblk = int(nblk_seq.sum())
    perm = torch.randperm(nblk, generator=g).to(torch.int32)
    bt = torch.zeros(len(lens), int(nblk_seq.max()), dtype=torch.int32)
    o = 0
    for b in range(len(lens)):
        n = int(nblk_seq[b])
        bt[b, :n] = perm[o:o + n]
        o += n
    x = torch.randn(len(lens), 20000, generator=g).to(dev)
    btd, lensd = bt.to(dev), lens.to(dev)
    idx_a = torch.full((len(lens), k), -5, dtype=torch.int32, device=dev)
    rows_a = torch.full((len(lens), k), -5, dtype=torch.int32, device=dev)
    cnt_a = torch.full((len(lens),), -5, dtype=torch.int32, device=dev)
    K.topk(x, lensd, k, idx_a, single_workgroup=single_workgroup)
    K.build_sparse_rows(idx_a, btd, lensd, page, nblk, rows_a, cnt_a)
    idx_b, rows_b, cnt_b = torch.full_like(idx_a, -6), torch.full_like(rows_a, -6), torch.full_like(cnt_a, -6)
    K.topk(x, lensd, k, idx_b, single_workgroup=single_workgroup, block_table=btd, page_size=page, num_pages=nblk,
           rows=rows_b, counts=cnt_b)
    assert torch.equal(idx_a, idx_b) and torch.equal(cnt_a, cnt_b)
    for b in range(len(lens)):
        c = int(cnt_a[b])
        assert c == min(int(lens[b]), k) and torch.equal(rows_a[b, :c], rows_b[b, :c])


def test_topk_on_indexer_logits_then_sparse_decode(dev):
    """Whole DSA decode chain at small scale: logits -> top-k (set equals the oracle's on the SAME logits) ->
    rows -> sparse MLA equals the oracle's sparse attention on that index set."""
    from omni_npu_amd import kernels as K
    batch, k = 4, 256
    c = make_indexer_case(batch, 200, 3000, seed=77)
    dc = O.make_decode_case(batch, 128, 200, 3000, seed=77)
    dc["seq_lens"], dc["block_table"] = c["seq_lens"], c["block_table"]        # same paging for both caches
    nblk = c["k8"].shape[0]
    g = torch.Generator().manual_seed(5)
    dc["nope"] = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    dc["rope"] = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    max_len = int(c["seq_lens"].max())
    logits = torch.empty(batch, K.indexer_logits_stride(max_len), device=dev)
    K.indexer_scores(c["q8"].to(dev), (c["w"] * c["q_scale"]).to(dev), c["k8"].to(dev), c["k_scale"].to(dev),
                     c["block_table"].to(dev), c["seq_lens"].to(dev), logits, max_seq_len=max_len)
    idx = torch.empty(batch, 1, k, dtype=torch.int32, device=dev)
    K.topk(logits, c["seq_lens"].to(dev), k, idx)
    lg = logits.cpu()
    for b in range(batch):
        ref = O.topk_stable(lg[b], k, int(c["seq_lens"][b]))
        assert sorted(i for i in ref.tolist() if i >= 0) == [i for i in idx[b, 0].tolist() if i >= 0]
    rows = torch.empty(batch, k, dtype=torch.int32, device=dev)
    counts = torch.empty(batch, dtype=torch.int32, device=dev)
    K.build_sparse_rows(idx, c["block_table"].to(dev), c["seq_lens"].to(dev), 128, nblk, rows, counts)
    assert counts.cpu().tolist() == [min(k, int(l)) for l in c["seq_lens"]]
    out = torch.empty(batch, 128, 512, dtype=torch.bfloat16, device=dev)
    K.sparse_decode(dc["q_nope"].to(dev), dc["q_rope"].to(dev), dc["nope"].to(dev), dc["rope"].to(dev), rows, counts,
                    dc["scale"], out, num_splits=2)
    ref = O.sparse_decode(dc["q_nope"], dc["q_rope"], dc["nope"], dc["rope"], c["block_table"], c["seq_lens"], idx.cpu(),
                          dc["scale"])
    attn_close(out, ref, 2e-2, 2e-3)


def test_sparse_decode_with_padding_and_full_coverage(dev):
    """-1 padding and out-of-range positions are dropped; with k >= L the sparse result equals dense decode."""
    from omni_npu_amd import kernels as K
    dc = O.make_decode_case(3, 128, 50, 300, seed=13)
    k = 512
    idx = torch.full((3, 1, k), -1, dtype=torch.int32)
    for b in range(3):
        L = int(dc["seq_lens"][b])
        perm = torch.randperm(L, generator=torch.Generator().manual_seed(b)).to(torch.int32)
        idx[b, 0, 0:2 * L:2] = perm                          # interleaved with -1 holes
    idx[0, 0, 1] = 100000                                    # beyond the sequence: ignored
    dev_idx = idx.to(dev)
    rows = torch.empty(3, k, dtype=torch.int32, device=dev)
    counts = torch.empty(3, dtype=torch.int32, device=dev)
    K.build_sparse_rows(dev_idx, dc["block_table"].to(dev), dc["seq_lens"].to(dev), 128, dc["nope"].shape[0], rows, counts)
    assert counts.cpu().tolist() == dc["seq_lens"].tolist()
    out = torch.empty(3, 128, 512, dtype=torch.bfloat16, device=dev)
    K.sparse_decode(dc["q_nope"].to(dev), dc["q_rope"].to(dev), dc["nope"].to(dev), dc["rope"].to(dev), rows, counts,
                    dc["scale"], out)
    dense = O.absorbed_decode(dc["q_nope"], dc["q_rope"], dc["nope"], dc["rope"], dc["block_table"], dc["seq_lens"],
                              dc["scale"])
    attn_close(out, dense, 2e-2, 2e-3)


def _random_indexer_cases(n_cases, seed):
    import random
    rng = random.Random(seed)
    out = []
    for i in range(n_cases):
        q_len = rng.choice([1, 1, 2, 3])
        batch = rng.randint(1, 6)
        lo = rng.choice([q_len, 31, 32, 33, 127, 128, 129, 1000])
        hi = lo + rng.choice([0, 1, 100, 2500])
        k = rng.choice([1, 7, 64, 300, 2048])
        out.append((i, batch, lo, hi, q_len, k, rng.random() < 0.5))
    return out


@pytest.mark.parametrize("i,batch,lo,hi,q_len,k,single_workgroup", _random_indexer_cases(24, seed=99))
def test_indexer_topk_rows_random_shapes(dev, i, batch, lo, hi, q_len, k, single_workgroup):
    """Seeded sweep over the indexer chain: logits against the oracle, top-k sets (on the kernel's own logits) bit-exact
    with ties to the lower position, and the fused row translation equal to positions mapped through the block table;
    ragged lengths around the 32-key block and 128-token page edges, MTP queries, k from 1 to 2048."""
    from omni_npu_amd import kernels as K
    c = make_indexer_case(batch, lo, hi, seed=300 + i, q_len=q_len)
    t = batch * q_len
    max_len = int(c["seq_lens"].max())
    nblk = c["k8"].shape[0]
    logits = torch.full((t, K.indexer_logits_stride(max_len)), float("nan"), device=dev)
    K.indexer_scores(c["q8"].to(dev), c["w"].to(dev), c["k8"].to(dev), c["k_scale"].to(dev), c["block_table"].to(dev),
                     c["seq_lens"].to(dev), logits, q_len=q_len, q_scale=c["q_scale"].to(dev), max_seq_len=max_len)
    idx = torch.full((t, k), -7, dtype=torch.int32, device=dev)
    rows = torch.full((t, k), -7, dtype=torch.int32, device=dev)
    counts = torch.full((t,), -7, dtype=torch.int32, device=dev)
    K.topk(logits, c["seq_lens"].to(dev), k, idx, q_len=q_len, single_workgroup=single_workgroup,
           block_table=c["block_table"].to(dev), page_size=128, num_pages=nblk, rows=rows, counts=counts)
    lg, idx_c, rows_c, counts_c = logits.cpu(), idx.cpu(), rows.cpu(), counts.cpu()
    for tt in range(t):
        ref = oracle_logits(c, tt)
        n = ref.numel()
        assert (lg[tt, :n] - ref).abs().max().item() <= logits_tol(c, tt, ref)
        want = O.topk_stable(lg[tt], k, n)
        got = [v for v in idx_c[tt].tolist() if v >= 0]
        assert got == sorted(v for v in want.tolist() if v >= 0), (tt, n, k)
        assert idx_c[tt, len(got):].eq(-1).all() and int(counts_c[tt]) == len(got) == min(n, k)
        b = tt // q_len
        pos = torch.tensor(got, dtype=torch.long)
        assert torch.equal(rows_c[tt, :len(got)].long(), c["block_table"][b, pos // 128].long() * 128 + pos % 128)


def test_quant_qk_in_one_launch_equals_the_two_launches(dev):
    """The indexer's two quantisations of a step (queries into plain buffers, new keys into the paged cache with pad slots
    skipped) as one launch: the same bytes and scales as two dsa_quant_rows_fp8 launches."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(17)
    t, h, nblk = 37, 64, 5
    q = torch.randn(t * h, 128, generator=g).bfloat16().to(dev)
    k = (torch.randn(t, 128, generator=g) * 3).bfloat16().to(dev)
    k[3] = 0                                                  # an all-zero row: scale 1
    slots = torch.randperm(nblk * 128, generator=g)[:t]
    slots[5] = -1
    slots = slots.to(dev)
    def run(one):
        q8 = torch.zeros(t * h, 128, dtype=torch.uint8, device=dev)
        qs = torch.zeros(t * h, dtype=torch.float32, device=dev)
        k8 = torch.full((nblk, 128, 128), 7, dtype=torch.uint8, device=dev)
        ks = torch.full((nblk, 128), -1.0, dtype=torch.float32, device=dev)
        if one:
            K.quant_qk_fp8(q, q8, qs, k, k8, ks, slots)
        else:
            K.quant_rows_fp8(q, q8, qs)
            K.quant_rows_fp8(k, k8, ks, slot_mapping=slots)
        return q8, qs, k8, ks
    a, b = run(True), run(False)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    ref8, refs = O.fp8_quant_token(k.float().cpu())
    sm = slots.cpu()
    ok = sm >= 0
    assert torch.equal(a[2].cpu().view(-1, 128)[sm[ok]], ref8.view(torch.uint8)[ok]) and torch.equal(a[3].cpu().view(-1)[sm[ok]], refs[ok])


def _sparse_case(batch, heads, lens, counts, seed):
    """Row lists over a paged cache: token b attends to counts[b] distinct keys of its sequence (ascending positions)."""
    c = O.make_decode_case(batch, heads, min(lens), max(lens), seed=seed, q_len=1)
    k = max(max(counts), 1)
    g = torch.Generator().manual_seed(seed)
    idx = torch.full((batch, k), -1, dtype=torch.int32)
    rows = torch.zeros(batch, k, dtype=torch.int32)
    cnt = torch.zeros(batch, dtype=torch.int32)
    for b in range(batch):
        L = int(c["seq_lens"][b])
        n = min(counts[b], L)
        pos = torch.randperm(L, generator=g)[:n].sort().values
        idx[b, :n] = pos.to(torch.int32)
        rows[b, :n] = O.slots_for(c["block_table"], b, 0, L)[pos].to(torch.int32)
        cnt[b] = n
    return c, idx, rows, cnt


@pytest.mark.parametrize("batch,heads,counts", [
    (3, 128, [2048, 2048, 2048]), (8, 128, [1, 63, 64, 65, 128, 129, 700, 0]), (5, 16, [40, 7, 200, 64, 1]),
    (2, 32, [300, 17]), (16, 64, [100 + 13 * i for i in range(16)]),
])
def test_sparse_decode_split_over_heads_matches_the_oracle_and_the_split_over_keys(dev, batch, heads, counts):
    """dsa_sparse_decode_heads_bf16 (a workgroup per (token, 16 heads) over all of the token's rows, no partials, no merge)
    against the oracle and against the split-KV form: attention within the bf16 bar, and - every probability going through
    P.V as two bf16 numbers - within 1.6e-3 of mean relative error; log-sum-exps within 1e-4 of the other form's; an empty
    row list gives zeros and -inf."""
    from omni_npu_amd import kernels as K
    c, idx, rows, cnt = _sparse_case(batch, heads, [2100] * batch if max(counts) > 1000 else [800] * batch, counts, seed=61 + batch)
    ref, ref_lse = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx,
                                   c["scale"], return_lse=True)
    args = [c[x].to(dev) for x in ("q_nope", "q_rope", "nope", "rope")]
    got = {}
    for method in ("keys", "heads"):
        out = torch.full((batch, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device=dev)
        K.sparse_decode(*args, rows.to(dev), cnt.to(dev), c["scale"], out, lse_out=lse, method=method)
        torch.cuda.synchronize()
        got[method] = (out.cpu(), lse.cpu())
    ma, mr = attn_close(got["heads"][0], ref, 2e-2, 2e-3)
    assert mr <= 1.6e-3, mr
    attn_close(got["keys"][0], ref, 2e-2, 2e-3)
    fin = torch.isfinite(ref_lse)
    assert torch.equal(torch.isfinite(got["heads"][1]), fin)
    assert torch.allclose(got["heads"][1][fin], ref_lse[fin], atol=2e-3, rtol=0)
    assert torch.allclose(got["heads"][1][fin], got["keys"][1][fin], atol=1e-4, rtol=0)
    empty = cnt == 0
    assert (got["heads"][0][empty] == 0).all() and torch.isinf(got["heads"][1][empty]).all()


@pytest.mark.parametrize("batch,heads,counts,splits", [
    (3, 128, [2048, 2048, 2048], 1), (3, 128, [2048, 1500, 2048], 2), (8, 128, [1, 63, 64, 65, 128, 129, 700, 0], 2),
    (16, 128, [2048] * 16, 4), (32, 128, [2048] * 31 + [5], 2), (2, 96, [300, 17], 1), (4, 80, [900, 33, 0, 512], 3),
    (1, 256, [1024], 4),
])
def test_sparse_decode_with_few_chunks_cuts_the_rows_instead(dev, batch, heads, counts, splits):
    """When tokens x chunks would leave most CUs idle the row-list kernel gives every 32 or 64 query rows a workgroup of
    their own (the small-row forms over several row groups).  Against the oracle, at the margin those forms keep
    (two-term probabilities), log-sum-exps included; an empty row list gives zeros and -inf; heads that do not fill the
    last group of rows leave their neighbours' partials alone."""
    from omni_npu_amd import kernels as K
    c, idx, rows, cnt = _sparse_case(batch, heads, [2100] * batch if max(counts) > 1000 else [1000] * batch, counts, seed=17 + batch)
    ref, ref_lse = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx,
                                   c["scale"], return_lse=True)
    args = [c[x].to(dev) for x in ("q_nope", "q_rope", "nope", "rope")]
    out = torch.full((batch, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full((batch, heads), float("nan"), dtype=torch.float32, device=dev)
    K.sparse_decode(*args, rows.to(dev), cnt.to(dev), c["scale"], out, lse_out=lse, num_splits=splits, method="keys")
    torch.cuda.synchronize()
    ma, mr = attn_close(out.cpu(), ref, 2e-2, 2e-3)
    assert mr <= 1.8e-3, mr
    fin = torch.isfinite(ref_lse)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert torch.allclose(lse.cpu()[fin], ref_lse[fin], atol=2e-3, rtol=0)
    empty = cnt == 0
    assert (out.cpu()[empty] == 0).all()


def test_sparse_decode_over_heads_starts_over_when_a_score_outgrows_its_reference(dev):
    """The references are fixed on the first 64 keys; a key further on whose score lies more than 2^100 above them makes
    the workgroup run the token again with the maxima it has seen.  Planted: one key, scaled so that its score against
    every head exceeds the first tile's by several hundred (log2)."""
    from omni_npu_amd import kernels as K
    c, idx, rows, cnt = _sparse_case(2, 32, [900, 900], [600, 500], seed=91)
    q = c["q_nope"].float()
    big = int(idx[0, 400])                                    # a key position far behind the first tile of token 0
    slot = int(O.slots_for(c["block_table"], 0, big, big + 1)[0])
    # make the key point along every head's query at once: the sum of the heads' (sign-aligned) queries, large
    direction = q[0].sum(0)
    c["nope"].view(-1, 512)[slot] = (direction / direction.norm() * 60.0).bfloat16()
    c["q_nope"][0] = (q[0] + direction / direction.norm() * 40.0).bfloat16()     # every head sees it: score ~ 60 * 40 * scale
    ref = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx, c["scale"])
    args = [c[x].to(dev) for x in ("q_nope", "q_rope", "nope", "rope")]
    out = torch.full((2, 32, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.sparse_decode(*args, rows.to(dev), cnt.to(dev), c["scale"], out, method="heads")
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    # token 0 is (nearly) the planted key's latent vector; bf16 of values up to 60 -> looser absolute bar there
    err = (out.float().cpu() - ref).abs()
    assert err[1].max() <= 2e-2 and err[0].max() <= 60.0 * 2 ** -8 + 2e-2
    assert (err.sum() / ref.abs().sum()).item() <= 2e-3


def test_sparse_decode_method_choice_and_refusals(dev):
    from omni_npu_amd import kernels as K
    c, idx, rows, cnt = _sparse_case(2, 24, [300, 300], [100, 50], seed=5)     # 24 heads: no multiple of 16
    args = [c[x].to(dev) for x in ("q_nope", "q_rope", "nope", "rope")]
    out = torch.zeros(2, 24, 512, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError, match="multiple of 16"):
        K.sparse_decode(*args, rows.to(dev), cnt.to(dev), c["scale"], out, method="heads")
    with pytest.raises(ValueError, match="unknown method"):
        K.sparse_decode(*args, rows.to(dev), cnt.to(dev), c["scale"], out, method="rows")
    K.sparse_decode(*args, rows.to(dev), cnt.to(dev), c["scale"], out)          # auto -> the split form
    ref = O.sparse_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], c["block_table"], c["seq_lens"], idx, c["scale"])
    attn_close(out, ref, 2e-2, 2e-3)
