"""Parity of the fused RMSNorm + rotary embedding + cache write (and the query-side rotary embedding) against the CPU
oracle, through the C-ABI.

Bar: the oracle computes in float64 and rounds once to bf16; the kernel computes in fp32 (every operation rounded on its
own) and rounds once, so results may differ by one bf16 unit in the last place where the fp32 value sits within ~1e-7 of
a rounding boundary: at most 1 ulp anywhere, and at least 99.9 % of the elements identical.  Scatter positions, skipped
pad slots and the fp8 bytes are bit-exact."""
import pytest
import torch

from oracle import mla_oracle as O

pytestmark = pytest.mark.gpu
EPS = 1e-6


def _ulp_close(got: torch.Tensor, want: torch.Tensor):
    got, want = got.cpu().contiguous(), want.cpu().contiguous()
    assert got.shape == want.shape and got.dtype == want.dtype == torch.bfloat16
    a, b = got.view(torch.int16).int(), want.view(torch.int16).int()
    d = (a - b).abs()
    assert int(d.max()) <= 1, f"max distance {int(d.max())} ulp"
    assert float((d == 0).float().mean()) >= 0.999, f"only {float((d == 0).float().mean()):.5f} identical"


def _case(t, seed, wide=False):
    g = torch.Generator().manual_seed(seed)
    kv = torch.randn(t, 576, generator=g) * (1 + torch.rand(t, 1, generator=g) * 3)
    kv = kv.bfloat16()
    if wide:                                                # a [T,576] view of a wider projection output
        buf = torch.zeros(t, 640).bfloat16()
        buf[:, 32:608] = kv
        kv_view = lambda dev: buf.to(dev)[:, 32:608]
    else:
        kv_view = lambda dev: kv.to(dev)
    gamma = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    pos = torch.randint(0, 8192, (t,), generator=g)
    nblk = (t + 127) // 128 + 2
    perm = torch.randperm(nblk * 128, generator=g)[:t]
    slots = perm.clone()
    if t > 3:
        slots[1] = -1
        slots[t - 1] = -1
    return kv, kv_view, gamma, pos, slots, nblk


@pytest.mark.parametrize("t,layout,interleaved,wide", [(1, "half", False, False), (4, "repeat", True, False),
                                                       (64, "half", False, True), (301, "repeat", False, False),
                                                       (2048, "half", True, False)])
def test_fused_norm_rope_cache_matches_oracle(dev, t, layout, interleaved, wide):
    from omni_npu_amd import kernels as K
    kv, kv_view, gamma, pos, slots, nblk = _case(t, seed=t, wide=wide)
    cos, sin = O.rope_tables(pos, layout=layout)
    g = torch.Generator().manual_seed(99)
    nope0 = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope0 = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    nope_ref, rope_ref = nope0.clone(), rope0.clone()
    k_pe_ref, kv_a_ref = O.kv_rmsnorm_rope_cache(kv, gamma, cos, sin, slots, nope_ref, rope_ref, EPS, table=layout,
                                                 interleaved_out=interleaved)
    nope, rope = nope0.to(dev), rope0.to(dev)
    kv_a_out = torch.full((t, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    k_pe_out = torch.full((t, 64), float("nan"), dtype=torch.bfloat16, device=dev)
    K.kv_rmsnorm_rope_cache(kv_view(dev), gamma.to(dev), cos.to(dev), sin.to(dev), slots.to(dev), nope, rope, eps=EPS,
                            table=layout, interleaved_out=interleaved, kv_a_out=kv_a_out, k_pe_out=k_pe_out)
    torch.cuda.synchronize()
    _ulp_close(kv_a_out, kv_a_ref)
    _ulp_close(k_pe_out, k_pe_ref)
    # the cache rows hold exactly what the plain outputs hold, at the right slots; every other row is untouched
    flat_n, flat_r = nope.cpu().view(-1, 512), rope.cpu().view(-1, 64)
    keep = slots >= 0
    assert torch.equal(flat_n[slots[keep]], kv_a_out.cpu()[keep])
    assert torch.equal(flat_r[slots[keep]], k_pe_out.cpu()[keep])
    untouched = torch.ones(nblk * 128, dtype=torch.bool)
    untouched[slots[keep]] = False
    assert torch.equal(flat_n[untouched], nope0.view(-1, 512)[untouched])
    assert torch.equal(flat_r[untouched], rope0.view(-1, 64)[untouched])


def test_fused_without_plain_outputs_writes_the_same_rows(dev):
    from omni_npu_amd import kernels as K
    t = 130
    kv, kv_view, gamma, pos, slots, nblk = _case(t, seed=5)
    cos, sin = O.rope_tables(pos)
    a = [torch.zeros(nblk, 128, w, dtype=torch.bfloat16, device=dev) for w in (512, 64)]
    b = [torch.zeros(nblk, 128, w, dtype=torch.bfloat16, device=dev) for w in (512, 64)]
    args = (kv_view(dev), gamma.to(dev), cos.to(dev), sin.to(dev), slots.to(dev))
    K.kv_rmsnorm_rope_cache(*args, a[0], a[1], eps=EPS)
    K.kv_rmsnorm_rope_cache(*args, b[0], b[1], eps=EPS, kv_a_out=torch.empty(t, 512, dtype=torch.bfloat16, device=dev),
                            k_pe_out=torch.empty(t, 64, dtype=torch.bfloat16, device=dev))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_fused_fp8_equals_norm_then_quantising_write(dev):
    """Bytes of the fp8 cache rows == mla_cache_write_fp8 applied to the bf16 results of the bf16 variant."""
    from omni_npu_amd import kernels as K
    t = 257
    kv, kv_view, gamma, pos, slots, nblk = _case(t, seed=11)
    cos, sin = O.rope_tables(pos)
    args = (kv_view(dev), gamma.to(dev), cos.to(dev), sin.to(dev), slots.to(dev))
    nope = torch.zeros(nblk, 128, 512, dtype=torch.bfloat16, device=dev)
    rope = torch.zeros(nblk, 128, 64, dtype=torch.bfloat16, device=dev)
    kv_a = torch.empty(t, 512, dtype=torch.bfloat16, device=dev)
    k_pe = torch.empty(t, 64, dtype=torch.bfloat16, device=dev)
    K.kv_rmsnorm_rope_cache(*args, nope, rope, eps=EPS, kv_a_out=kv_a, k_pe_out=k_pe)
    want = torch.zeros(nblk, 128, 656, dtype=torch.uint8, device=dev)
    K.cache_write_fp8(kv_a, k_pe, slots.to(dev), want)
    got = torch.zeros(nblk, 128, 656, dtype=torch.uint8, device=dev)
    kv_a2 = torch.empty_like(kv_a)
    K.kv_rmsnorm_rope_cache(*args, got, None, eps=EPS, kv_a_out=kv_a2)
    assert torch.equal(got, want) and torch.equal(kv_a2, kv_a)
    # and the quantised latent matches the oracle's quantiser on the oracle's normalised rows (where those agree bit for bit)
    kv_a_ref = O.rms_norm(kv[:, :512], gamma, EPS)
    q_ref, sc_ref = O.fp8_quant_block(kv_a_ref.float())
    same = (kv_a.cpu() == kv_a_ref).all(-1) & (slots >= 0)
    rows = got.cpu().view(-1, 656)[slots[same]]
    assert torch.equal(rows[:, :512], q_ref[same].view(torch.uint8))
    assert torch.equal(rows[:, 512:528].contiguous().view(torch.float32), sc_ref[same])


@pytest.mark.parametrize("layout,interleaved", [("half", False), ("repeat", True)])
def test_query_rope_strided_and_in_place(dev, layout, interleaved):
    from omni_npu_amd import kernels as K
    t, n = 37, 128
    g = torch.Generator().manual_seed(3)
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    pos = torch.randint(0, 8192, (t,), generator=g)
    cos, sin = O.rope_tables(pos, layout=layout)
    want = O.interleave_rope(q[..., 128:], cos, sin, table=layout, interleaved_out=interleaved)
    qd = q.to(dev)
    got = K.interleave_rope(qd[..., 128:], cos.to(dev), sin.to(dev), table=layout, interleaved_out=interleaved)
    _ulp_close(got, want)
    # in place, in either output layout: the rope part of the query is rotated where it lies
    K.interleave_rope(qd[..., 128:], cos.to(dev), sin.to(dev), out=qd[..., 128:], table=layout, interleaved_out=interleaved)
    assert torch.equal(qd[..., 128:], got) and torch.equal(qd[..., :128].cpu(), q[..., :128])


@pytest.mark.parametrize("fp8", [False, True])
def test_fused_prologue_with_query_equals_the_two_launches(dev, fp8):
    """One launch for the key side (norm, rope, cache write, plain outputs) and the query's rope part, in place on a strided
    view: the same bits as the two launches, in the caches, the plain outputs and the query."""
    from omni_npu_amd import kernels as K
    t, n = 67, 128
    kv, kv_view, gamma, pos, slots, nblk = _case(t, seed=12)
    g = torch.Generator().manual_seed(13)
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    cos, sin = O.rope_tables(pos)
    cd, sd, gd, sl = cos.to(dev), sin.to(dev), gamma.to(dev), slots.to(dev)

    def caches():
        if fp8:
            return torch.zeros(nblk, 128, 656, dtype=torch.uint8, device=dev), None
        return torch.zeros(nblk, 128, 512, dtype=torch.bfloat16, device=dev), torch.zeros(nblk, 128, 64, dtype=torch.bfloat16, device=dev)

    n1, r1 = caches()
    a1, p1 = torch.zeros(t, 512, dtype=torch.bfloat16, device=dev), torch.zeros(t, 64, dtype=torch.bfloat16, device=dev)
    q1 = q.to(dev)
    K.kv_rmsnorm_rope_cache(kv_view(dev), gd, cd, sd, sl, n1, r1, eps=EPS, kv_a_out=a1, k_pe_out=p1)
    K.interleave_rope(q1[..., 128:], cd, sd, out=q1[..., 128:])
    n2, r2 = caches()
    a2, p2 = torch.zeros_like(a1), torch.zeros_like(p1)
    q2 = q.to(dev)
    K.kv_rmsnorm_rope_cache(kv_view(dev), gd, cd, sd, sl, n2, r2, eps=EPS, kv_a_out=a2, k_pe_out=p2, q_rope=q2[..., 128:])
    assert torch.equal(n1, n2) and (fp8 or torch.equal(r1, r2)) and torch.equal(a1, a2) and torch.equal(p1, p2)
    assert torch.equal(q1, q2) and torch.equal(q2[..., :128].cpu(), q[..., :128])
    _ulp_close(q2[..., 128:], O.interleave_rope(q[..., 128:], cos, sin))
    # without a cache (profile run) and into a separate query tensor
    q3 = torch.zeros(t, n, 64, dtype=torch.bfloat16, device=dev)
    K.kv_rmsnorm_rope_cache(kv_view(dev), gd, cd, sd, None, None, None, eps=EPS, kv_a_out=a2, k_pe_out=p2,
                            q_rope=q.to(dev)[..., 128:], q_out=q3)
    assert torch.equal(q3, q1[..., 128:]) and torch.equal(a1, a2)


@pytest.mark.parametrize("layout", ["half", "repeat"])
def test_rotary_mul_strided_and_in_place(dev, layout):
    """The half-rotation pairing of the indexer's rope dims (npu_dsa.py:116-131) on a strided view, then in place."""
    from omni_npu_amd import kernels as K
    t, n = 41, 64
    g = torch.Generator().manual_seed(6)
    q = torch.randn(t, n, 128, generator=g).bfloat16()
    pos = torch.randint(0, 8192, (t,), generator=g)
    cos, sin = O.rope_tables(pos, layout=layout)
    want = O.rotary_mul(q[..., :64], cos, sin, table=layout)
    qd = q.to(dev)
    got = K.rotary_mul(qd[..., :64], cos.to(dev), sin.to(dev), table=layout)
    _ulp_close(got, want)
    K.rotary_mul(qd[..., :64], cos.to(dev), sin.to(dev), out=qd[..., :64], table=layout)
    assert torch.equal(qd[..., :64], got) and torch.equal(qd[..., 64:].cpu(), q[..., 64:])


def test_reference_named_ops(dev):
    """The call shapes of src/omni_npu/v1/layers/attention/npu_mla.py:296-316."""
    from omni_npu_amd import torch_npu_ops as T
    t, n = 9, 16
    kv, _, gamma, pos, slots, nblk = _case(t, seed=8)
    cos, sin = O.rope_tables(pos)
    nope = torch.zeros(nblk, 128, 512, dtype=torch.bfloat16, device=dev)
    rope = torch.zeros(nblk, 128, 64, dtype=torch.bfloat16, device=dev)
    k_c, ckv_c, k_pe, kv_a = T.npu_kv_rmsnorm_rope_cache(kv.to(dev).view(-1, 1, 1, 576), gamma.to(dev),
                                                         cos.to(dev).view(-1, 1, 1, 64), sin.to(dev).view(-1, 1, 1, 64),
                                                         slots.to(dev), rope.unsqueeze(2), nope.unsqueeze(2), epsilon=EPS,
                                                         cache_mode="PA", is_output_kv=True)
    assert k_pe.shape == (t, 1, 1, 64) and kv_a.shape == (t, 1, 1, 512) and k_c.data_ptr() == rope.data_ptr()
    _ulp_close(kv_a.view(t, 512), O.rms_norm(kv[:, :512], gamma, EPS))
    _ulp_close(k_pe.view(t, 64), O.interleave_rope(kv[:, 512:], cos, sin))
    with pytest.raises(NotImplementedError):
        T.npu_kv_rmsnorm_rope_cache(kv.to(dev).view(-1, 1, 1, 576), gamma.to(dev), cos.to(dev), sin.to(dev), slots.to(dev),
                                    rope, nope, cache_mode="PA_NZ")
    g = torch.Generator().manual_seed(4)
    q_pe = torch.randn(t, n, 1, 64, generator=g).bfloat16()
    got = T.npu_interleave_rope(q_pe.to(dev), cos.to(dev).view(-1, 1, 1, 64), sin.to(dev).view(-1, 1, 1, 64))
    assert got.shape == q_pe.shape
    _ulp_close(got.view(t, n, 64), O.interleave_rope(q_pe.view(t, n, 64), cos, sin))
    # the indexer's call (npu_dsa.py:116-131): [T, N, 1, 64] with full-width rows
    got = T.npu_rotary_mul(q_pe.to(dev), cos.to(dev).view(-1, 1, 1, 64), sin.to(dev).view(-1, 1, 1, 64))
    assert got.shape == q_pe.shape
    _ulp_close(got.view(t, n, 64), O.rotary_mul(q_pe.view(t, n, 64), cos, sin))
    # the merge of partial results under the vendor op's name and argument layout (mla.py:683-687)
    parts, rows, d = 3, 40, 512
    outs = [torch.randn(rows, d, generator=g) for _ in range(parts)]
    lses = [torch.randn(rows, generator=g) * 3 for _ in range(parts)]
    lses[1][5] = float("-inf")
    merged, lse = T.npu_attention_update(lse=[v.to(dev) for v in lses], local_out=[o.to(dev) for o in outs], update_type=0)
    want_o, want_l = O.attention_update(torch.stack(outs), torch.stack(lses))
    assert merged.shape == (rows, d) and lse.shape == (rows,)
    assert torch.allclose(merged.cpu(), want_o.float(), rtol=1e-5, atol=1e-5)
    assert torch.allclose(lse.cpu(), want_l.float(), rtol=1e-5, atol=1e-5)
    with pytest.raises(NotImplementedError):
        T.npu_attention_update(lse=[v.to(dev) for v in lses], local_out=[o.to(dev) for o in outs], update_type=1)
