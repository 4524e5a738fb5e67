"""Bit-exact parity of the HIP latent-KV cache write against the oracle's row scatter."""
import pytest
import torch

from oracle import mla_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("t,nblk", [(1, 2), (64, 40), (512, 300), (1000, 9)])
def test_cache_write_bit_exact(dev, t, nblk):
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(t)
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    kv_c = torch.randn(t, 512, generator=g).bfloat16()
    k_pe = torch.randn(t, 1, 64, generator=g).bfloat16()
    slots = torch.randperm(nblk * 128, generator=g)[:t].to(torch.int64)
    slots[::7] = -1                                           # padding slots are skipped
    ref_n, ref_r = nope.clone(), rope.clone()
    O.cache_write(ref_n, slots, kv_c)
    O.cache_write(ref_r, slots, k_pe.squeeze(1))
    dn, dr = nope.to(dev), rope.to(dev)
    K.cache_write(kv_c.to(dev), k_pe.to(dev), slots.to(dev), dn, dr)
    torch.cuda.synchronize()
    assert torch.equal(dn.cpu(), ref_n) and torch.equal(dr.cpu(), ref_r)


def test_cache_write_four_dim_cache_and_strided_source(dev):
    """DSA layout [nblk,128,1,D] (dsa.py:67) and kv_c / k_pe as column slices of one [T,576] projection."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(1)
    nope = torch.zeros(6, 128, 1, 512, dtype=torch.bfloat16)
    rope = torch.zeros(6, 128, 1, 64, dtype=torch.bfloat16)
    latent = torch.randn(33, 576, generator=g).bfloat16()
    slots = torch.randperm(6 * 128, generator=g)[:33]
    ref_n, ref_r = nope.clone(), rope.clone()
    O.cache_write(ref_n, slots, latent[:, :512])
    O.cache_write(ref_r, slots, latent[:, 512:])
    dl, dn, dr = latent.to(dev), nope.to(dev), rope.to(dev)
    K.cache_write(dl[:, :512], dl[:, 512:], slots.to(dev), dn, dr)
    assert torch.equal(dn.cpu(), ref_n) and torch.equal(dr.cpu(), ref_r)


def test_scatter_rows_indexer_k(dev):
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(2)
    cache = torch.randn(5, 128, 1, 128, generator=g).bfloat16()
    k = torch.randn(77, 128, generator=g).bfloat16()
    slots = torch.randperm(5 * 128, generator=g)[:77]
    slots[3] = -1
    slots[5] = 5 * 128 + 9                                   # past the end of the cache: skipped, not a fault
    ref = cache.clone()
    keep = (slots >= 0) & (slots < 5 * 128)
    ref.view(-1, 128)[slots[keep]] = k[keep]
    dc = cache.to(dev)
    K.scatter_rows(k.to(dev), slots.to(dev), dc)
    assert torch.equal(dc.cpu(), ref)
