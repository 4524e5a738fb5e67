"""fp8 cache write, paged gather and two-way merge against the oracle (through the C-ABI)."""
import pytest
import torch

from oracle import mla_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("t,nblk", [(1, 1), (64, 30), (515, 9)])
def test_cache_write_fp8_bit_exact(dev, t, nblk):
    """Quantised bytes, scales and rope bytes equal the oracle's closed form bit for bit."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(100 + t)
    kv_c = (torch.randn(t, 512, generator=g) * torch.rand(t, 1, generator=g) * 4).bfloat16()
    kv_c[0, :128] = 0                                          # an all-zero block: scale 1, bytes 0
    k_pe = torch.randn(t, 64, generator=g).bfloat16()
    slots = torch.randperm(nblk * 128, generator=g)[:t].to(torch.int64)
    if t > 4:
        slots[3] = -1
    cache = torch.randint(0, 255, (nblk, 128, 656), dtype=torch.uint8, generator=g)
    ref = cache.clone()
    q, sc = O.fp8_quant_block(kv_c)
    flat = ref.view(-1, 656)
    keep = slots >= 0
    flat[slots[keep], :512] = q.view(torch.uint8)[keep]
    flat[slots[keep], 512:528] = sc.contiguous().view(torch.uint8).view(t, 16)[keep]
    flat[slots[keep], 528:] = k_pe.contiguous().view(torch.uint8).view(t, 128)[keep]
    dc = cache.to(dev)
    K.cache_write_fp8(kv_c.to(dev), k_pe.to(dev).unsqueeze(1), slots.to(dev), dc)
    torch.cuda.synchronize()
    got = dc.cpu()
    assert torch.equal(got.view(-1, 656)[:, 512:528], ref.view(-1, 656)[:, 512:528]), "scales differ"
    assert torch.equal(got.view(-1, 656)[:, 528:], ref.view(-1, 656)[:, 528:]), "rope bytes differ"
    assert torch.equal(got, ref), "quantised bytes differ"


def test_gather_paged_matches_oracle(dev):
    from omni_npu_amd import kernels as K
    case = O.make_decode_case(5, 16, 200, 900, seed=21)
    lens = case["seq_lens"]
    starts = torch.tensor([0, 17, 128, 5, 300], dtype=torch.int32)
    n = torch.minimum(lens - starts, torch.tensor([150, 0, 256, 64, 1], dtype=torch.int32))
    cu = torch.zeros(6, dtype=torch.int32)
    cu[1:] = torch.cumsum(n, 0)
    tot = int(cu[-1])
    ref = torch.zeros(tot + 3, 576, dtype=torch.bfloat16)
    O.gather_paged(case["nope"], case["rope"], ref, case["block_table"], cu, 5, starts)
    dst = torch.zeros(tot + 3, 576, dtype=torch.bfloat16, device=dev)
    K.gather_paged(case["nope"].to(dev), case["rope"].to(dev), dst, case["block_table"].to(dev), cu.to(dev), 5,
                   starts.to(dev))
    assert torch.equal(dst.cpu(), ref)
    # seq_starts=None gathers from position 0
    ref2 = torch.zeros(tot, 576, dtype=torch.bfloat16)
    O.gather_paged(case["nope"], case["rope"], ref2, case["block_table"], cu, 5, None)
    dst2 = torch.zeros(tot, 576, dtype=torch.bfloat16, device=dev)
    K.gather_paged(case["nope"].to(dev), case["rope"].to(dev), dst2, case["block_table"].to(dev), cu.to(dev), 5)
    assert torch.equal(dst2.cpu(), ref2)


def test_gather_paged_fp8_matches_oracle(dev):
    """The dequantising gather out of the fp8 cache: every row equals cat(bf16(e4m3 * block scale), rope) bit for bit."""
    from omni_npu_amd import kernels as K
    case = O.make_decode_case(5, 16, 200, 900, seed=22)
    nblk = case["nope"].shape[0]
    g = torch.Generator().manual_seed(5)
    lat = (case["nope"].float() * (torch.rand(nblk, 128, 1, generator=g) * 6)).bfloat16()    # block scales of many sizes
    lat[0, 3, 128:256] = 0                                                                   # an all-zero block (scale 1)
    cache = torch.zeros(nblk, 128, 656, dtype=torch.uint8, device=dev)
    K.cache_write_fp8(lat.view(-1, 512).to(dev), case["rope"].view(-1, 64).to(dev),
                      torch.arange(nblk * 128, dtype=torch.int64, device=dev), cache)
    q8, sc = O.fp8_quant_block(lat.float())                    # (the cache write is pinned bit-exact against this)
    lens = case["seq_lens"]
    starts = torch.tensor([0, 17, 128, 5, 300], dtype=torch.int32)
    n = torch.minimum(lens - starts, torch.tensor([150, 0, 256, 64, 1], dtype=torch.int32))
    cu = torch.zeros(6, dtype=torch.int32)
    cu[1:] = torch.cumsum(n, 0)
    tot = int(cu[-1])
    for st in (starts, None):
        ref = torch.zeros(tot + 3, 576, dtype=torch.bfloat16)
        O.gather_paged_fp8(q8, sc, case["rope"], ref, case["block_table"], cu, 5, st)
        dst = torch.zeros(tot + 3, 576, dtype=torch.bfloat16, device=dev)
        K.gather_paged_fp8(cache, dst, case["block_table"].to(dev), cu.to(dev), 5, None if st is None else st.to(dev))
        assert torch.equal(dst.cpu().view(torch.int16), ref.view(torch.int16))
    # the reference-named entry takes the one-tensor cache as well
    from omni_npu_amd.attention import ops
    dst = torch.zeros(tot, 576, dtype=torch.bfloat16, device=dev)
    ops.gather_and_maybe_dequant_cache((cache,), dst, case["block_table"].to(dev), cu.to(dev), 5, "fp8", None, starts.to(dev), tot)
    ref = torch.zeros(tot, 576, dtype=torch.bfloat16)
    O.gather_paged_fp8(q8, sc, case["rope"], ref, case["block_table"], cu, 5, starts)
    assert torch.equal(dst.cpu().view(torch.int16), ref.view(torch.int16))
    with pytest.raises(ValueError):
        K.gather_paged_fp8(cache.view(nblk, 128 * 656), dst, case["block_table"].to(dev), cu.to(dev), 5)


@pytest.mark.parametrize("in_dt,out_dt", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                          (torch.bfloat16, torch.bfloat16)])
def test_merge_states_matches_oracle(dev, in_dt, out_dt):
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(5)
    t, n, d = 37, 16, 128
    po, so = torch.randn(t, n, d, generator=g).to(in_dt), torch.randn(t, n, d, generator=g).to(in_dt)
    pl, sl = torch.randn(t, n, generator=g) * 3, torch.randn(t, n, generator=g) * 3
    pl[0, 0] = float("-inf")                     # one side empty
    sl[1, 1] = float("inf")                      # +inf is read as empty
    pl[2, 2] = sl[2, 2] = float("-inf")          # both empty -> zeros, -inf
    ref, ref_lse = O.merge_attn_states(po, pl.unsqueeze(-1), so, sl.unsqueeze(-1))
    out = torch.empty(t, n, d, dtype=out_dt, device=dev)
    lse = torch.empty(t, n, dtype=torch.float32, device=dev)
    K.merge_states(po.to(dev), pl.to(dev), so.to(dev), sl.to(dev), out, lse)
    tol = 1e-5 if out_dt == torch.float32 else 1e-2
    assert torch.allclose(out.float().cpu(), ref, atol=tol, rtol=tol)
    got_lse = lse.cpu()
    fin = torch.isfinite(ref_lse.squeeze(-1))
    assert torch.equal(torch.isfinite(got_lse), fin)
    assert torch.allclose(got_lse[fin], ref_lse.squeeze(-1)[fin], atol=1e-5, rtol=1e-5)
    assert (out[2, 2] == 0).all()
