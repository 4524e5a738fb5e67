"""Static sink tokens with and without a sliding window on the GPU (reference attention/backends/mla.py:463-560 and
:705-779) against the oracle: the window plan bit-exact, the attentions within the bf16 bar, at kernel level and through
NPUMLAImpl.forward."""
from types import SimpleNamespace

import pytest
import torch

from omni_npu_amd import _vllm_compat as V
from omni_npu_amd.attention.backends import mla
from omni_npu_amd.compilation.acl_graph import HIPGraphWrapper
from oracle import mla_oracle as O
from tests.conftest import attn_close
from tests.test_backend_gpu import _mk_impl, _to
from tests.test_boundary import _cfg, _common
from tests.test_sink_oracle import _sink_case

pytestmark = pytest.mark.gpu
MAX_ABS, MEAN_REL = 2e-2, 2e-3


# ---- decode at kernel level -------------------------------------------------------------------------------------
@pytest.mark.parametrize("batch,heads,lo,hi,sink_len,window,q_len,splits", [
    (4, 128, 200, 3000, 128, 512, 1, None), (3, 128, 1, 100, 128, 16, 1, 1), (3, 16, 300, 900, 256, 100, 2, 3),
    (2, 128, 2000, 5000, 128, 4096, 1, None), (2, 128, 600, 700, 128, 1, 3, 2), (5, 128, 1, 400, 0, 77, 2, None),
    (6, 128, 30, 2000, 128, 31, 4, 4), (3, 128, 500, 9000, 384, 1000, 1, 8), (4, 128, 100, 160, 128, 129, 2, 1)])
def test_dense_window_decode_matches_oracle(dev, batch, heads, lo, hi, sink_len, window, q_len, splits):
    """The dense kernel over the shortened sequences (sink blocks + window blocks): plain and fused with W_UV."""
    from omni_npu_amd import kernels as K
    c, bt = _sink_case(batch, heads, lo, hi, sink_len, q_len, seed=batch * 3 + heads + q_len + window)
    t = batch * q_len
    out = torch.full((t, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full((t, heads), float("nan"), dtype=torch.float32, device=dev)
    g = {k: c[k].to(dev) for k in ("q_nope", "q_rope", "nope", "rope", "seq_lens")}
    K.decode(g["q_nope"], g["q_rope"], g["nope"], g["rope"], bt.to(dev), g["seq_lens"], c["scale"], out, q_len=q_len,
             lse_out=lse, num_splits=splits, sink_len=sink_len, window=window)
    ref = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], sink_len, c["scale"], window)
    attn_close(out, ref, MAX_ABS, MEAN_REL)
    assert torch.isfinite(lse).all()
    if heads == 128:
        gw = torch.Generator().manual_seed(1)
        w_uv = (torch.randn(heads, 512, 128, generator=gw) * 0.05).bfloat16()
        out_v = torch.full((t, heads * 128), float("nan"), dtype=torch.bfloat16, device=dev)
        K.decode(g["q_nope"], g["q_rope"], g["nope"], g["rope"], bt.to(dev), g["seq_lens"], c["scale"], out_v, q_len=q_len,
                 num_splits=splits, sink_len=sink_len, window=window, w_uv=w_uv.to(dev))
        ref_v = torch.einsum("tnl,nlv->tnv", ref, w_uv.float()).reshape(t, -1)
        attn_close(out_v, ref_v, 3e-2, 8e-3)


def test_dense_window_decode_ragged_queries_and_argument_errors(dev):
    from omni_npu_amd import kernels as K
    c, bt = _sink_case(3, 128, 300, 1500, 128, 1, seed=8)
    q_lens = [1, 3, 2]
    qsl = [0, 1, 4, 6]
    g0 = torch.Generator().manual_seed(4)
    qn, qr = torch.randn(6, 128, 512, generator=g0).bfloat16(), torch.randn(6, 128, 64, generator=g0).bfloat16()
    out = torch.full((6, 128, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    args = (qn.to(dev), qr.to(dev), c["nope"].to(dev), c["rope"].to(dev), bt.to(dev), c["seq_lens"].to(dev), c["scale"], out)
    K.decode(*args, q_len=3, query_start_loc=torch.tensor(qsl, dtype=torch.int32, device=dev), sink_len=128, window=200)
    ref = O.sink_decode(qn, qr, c["nope"], c["rope"], bt, c["seq_lens"], 128, c["scale"], 200, query_start_loc=qsl)
    attn_close(out, ref, MAX_ABS, MEAN_REL)
    with pytest.raises(ValueError, match="whole number of pages"):
        K.decode(*args, q_len=2, sink_len=100, window=64)
    with pytest.raises(ValueError, match="sink_len goes with window"):
        K.decode(*args, q_len=2, sink_len=128)
    with pytest.raises(ValueError, match="both phases"):
        K.decode(*args, q_len=2, sink_len=128, window=64, phase="split")


def test_window_plan_bit_exact(dev):
    from omni_npu_amd import _lib
    lib = _lib.load()
    lens = torch.tensor([0, 1, 31, 32, 33, 100, 128, 129, 4096, 4097, 5000, 70000], dtype=torch.int32)
    for q_len, sink_len, window in [(1, 128, 64), (2, 128, 100), (4, 0, 1), (1, 256, 4096), (3, 128, 33)]:
        short = torch.full((12,), -1, dtype=torch.int32, device=dev)
        skip = torch.full((12,), -1, dtype=torch.int32, device=dev)
        rc = lib.mla_window_plan(lens.to(dev).data_ptr(), None, 12, q_len, sink_len, window, short.data_ptr(), skip.data_ptr(),
                                 torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        for i, L in enumerate(lens.tolist()):
            lo0 = max(0, max(0, L - q_len + 1) - window)
            assert int(skip[i]) == lo0 // 32
            assert int(short[i]) == (sink_len + L - 32 * (lo0 // 32) if L > 0 else 0)


def test_sink_decode_without_window_is_the_dense_kernel_over_the_longer_table(dev):
    from omni_npu_amd import kernels as K
    c, bt = _sink_case(5, 128, 100, 2500, 256, 2, seed=21)
    out = torch.full((10, 128, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode(c["q_nope"].to(dev), c["q_rope"].to(dev), c["nope"].to(dev), c["rope"].to(dev), bt.to(dev),
             (c["seq_lens"] + 256).to(dev), c["scale"], out, q_len=2)
    ref = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], 256, c["scale"], None)
    attn_close(out, ref, MAX_ABS, MEAN_REL)


# ---- prefill with a band ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("q_lens,k_extra,window,heads", [
    ([200], [0], 64, 4), ([37, 300, 1], [0, 0, 0], 7, 4), ([129, 64], [50, 300], 100, 8), ([500], [0], 1, 2),
    ([260, 131], [0, 17], 128, 16), ([70], [0], 1000, 4), ([1000], [24], 129, 2)])
def test_prefill_with_a_sliding_window_matches_oracle(dev, q_lens, k_extra, window, heads):
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(sum(q_lens) + window)
    k_lens = [a + b for a, b in zip(q_lens, k_extra)]
    cu_q = [0] + torch.tensor(q_lens).cumsum(0).tolist()
    cu_k = [0] + torch.tensor(k_lens).cumsum(0).tolist()
    t, tk = cu_q[-1], cu_k[-1]
    qn, qp = torch.randn(t, heads, 128, generator=g).bfloat16(), torch.randn(t, heads, 64, generator=g).bfloat16()
    kn, kp = torch.randn(tk, heads, 128, generator=g).bfloat16(), torch.randn(tk, 64, generator=g).bfloat16()
    v = torch.randn(tk, heads, 128, generator=g).bfloat16()
    scale = 192 ** -0.5
    out = torch.full((t, heads, 128), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((t, heads), float("nan"), dtype=torch.float32, device=dev)
    K.prefill_varlen(qn.to(dev), qp.to(dev), kn.to(dev), kp.to(dev), v.to(dev), torch.tensor(cu_q, dtype=torch.int32, device=dev),
                     torch.tensor(cu_k, dtype=torch.int32, device=dev), max(q_lens), scale, True, out, lse, window=window)
    ref, ref_lse = O.attention_varlen(qn, qp, kn, kp, v, cu_q, cu_k, scale, True, window=window)
    attn_close(out, ref, MAX_ABS, MEAN_REL)
    assert (lse.cpu() - ref_lse).abs().max() < 2e-2
    with pytest.raises(ValueError, match="window must be positive"):
        K.prefill_varlen(qn.to(dev), qp.to(dev), kn.to(dev), kp.to(dev), v.to(dev), torch.tensor(cu_q, dtype=torch.int32, device=dev),
                         torch.tensor(cu_k, dtype=torch.int32, device=dev), max(q_lens), scale, True, out, lse, window=0)


# ---- through NPUMLAImpl.forward ---------------------------------------------------------------------------------
def _with_sink_pages(common, nsb):
    """Block tables of _common moved up by nsb pages, with the shared sink pages 0..nsb-1 in front of every row."""
    bt = common.block_table_tensor + nsb
    sink = torch.arange(nsb, dtype=torch.int32).view(1, -1).expand(bt.shape[0], -1)
    common.block_table_tensor = torch.cat([sink, bt], 1).contiguous()
    return common


@pytest.mark.parametrize("window", [None, 48])
@pytest.mark.parametrize("q_lens,seq_lens,n", [([1] * 4, [160, 7, 300, 129], 4), ([2, 2, 2], [500, 129, 1000], 128)])
def test_impl_decode_with_sink_tokens(dev, q_lens, seq_lens, n, window):
    g = torch.Generator().manual_seed(len(q_lens) + (window or 0))
    sink_len, nsb = 128, 1
    common = _with_sink_pages(_common(q_lens, seq_lens), nsb)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    own = common.block_table_tensor[:, nsb:]
    common.slot_mapping = torch.cat([O.slots_for(own, b, s - ql, s) for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev, sliding_window=window)
    impl.update_sink_kv(rope[0].to(dev), nope[0].to(dev))                       # the sink latents are what page 0 holds
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    spec.sink_len = sink_len
    builder = mla.NPUMLAMetadataBuilder(spec, ["l"], _cfg(cap=2), dev)
    # oracle: write the new rows, absorb q, sink decode, up-project
    O.cache_write(nope, common.slot_mapping, kvc)
    O.cache_write(rope, common.slot_mapping, kpe.view(-1, 64))
    kvw = w.float().view(512, n, 256)
    ql = torch.einsum("tnp,lnp->tnl", q[..., :128].float(), kvw[..., :128]).bfloat16()    # the absorb GEMM stores bf16
    qsl = common.query_start_loc_cpu.tolist()
    o = O.sink_decode(ql, q[..., 128:].float(), nope, rope, common.block_table_tensor, common.seq_lens_cpu, sink_len,
                      impl.scale, window, query_start_loc=qsl)
    ref = torch.einsum("tnl,lnv->tnv", o, kvw[..., 128:]).reshape(t, -1)
    meta = builder.build(0, _to(common, dev))
    assert meta.decode.seq_sink_len == [sink_len] * len(q_lens)
    # the cache before the write: the oracle's copy minus the new rows is not needed, the write puts the same rows
    raw = torch.cat([nope.reshape(-1), rope.reshape(-1)]).to(dev).view(torch.uint8)
    kv_cache = mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 576, dtype=torch.bfloat16)
    out = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    impl.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out)
    attn_close(out, ref, 3e-2, 8e-3)


@pytest.mark.parametrize("window", [None, 20])
def test_impl_prefill_with_sink_tokens(dev, window):
    g = torch.Generator().manual_seed(31 + (window or 0))
    n, sink_len, nsb = 4, 128, 1
    q_lens = [16, 200, 37]
    common = _with_sink_pages(_common(q_lens, q_lens), nsb)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    sink_c, sink_pe = torch.randn(sink_len, 512, generator=g).bfloat16(), torch.randn(sink_len, 64, generator=g).bfloat16()
    own = common.block_table_tensor[:, nsb:]
    common.slot_mapping = torch.cat([O.slots_for(own, b, 0, s) for b, s in enumerate(q_lens)])
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev, sliding_window=window)
    impl.update_sink_kv(sink_pe.to(dev), sink_c.to(dev))
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    spec.sink_len = sink_len
    builder = mla.NPUMLAMetadataBuilder(spec, ["l"], _cfg(cap=2), dev)
    ref = O.sink_prefill(q.float(), kvc, kpe.view(-1, 64), w, sink_c, sink_pe, common.query_start_loc_cpu.tolist(),
                         impl.scale, window)
    meta = builder.build(0, _to(common, dev))
    raw = torch.zeros(nblk * 128 * 576, dtype=torch.bfloat16, device=dev).view(torch.uint8)
    kv_cache = mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 576, dtype=torch.bfloat16)
    out = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    impl.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out)
    attn_close(out, ref, 3e-2, 8e-3)
    # the new latents went into the pages behind the sink page
    sm = common.slot_mapping.cpu()
    assert torch.equal(kv_cache[0].view(-1, 512)[sm.to(dev)].cpu(), kvc)


def test_impl_decode_with_sink_tokens_over_the_fp8_cache(dev):
    """Sink tokens over the fp8 cache, without and with a window; the oracle reads the dequantised cache."""
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(77)
    n, sink_len, nsb = 128, 128, 1
    q_lens, seq_lens = [2, 2, 2], [300, 129, 700]
    common = _with_sink_pages(_common(q_lens, seq_lens), nsb)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    own = common.block_table_tensor[:, nsb:]
    common.slot_mapping = torch.cat([O.slots_for(own, b, s - ql, s) for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    O.cache_write(nope, common.slot_mapping, kvc)
    O.cache_write(rope, common.slot_mapping, kpe.view(-1, 64))
    cache = torch.zeros(nblk, 128, K.FP8_ROW_BYTES, dtype=torch.uint8, device=dev)
    K.cache_write_fp8(nope.view(-1, 512).to(dev), rope.view(-1, 64).to(dev), torch.arange(nblk * 128, device=dev), cache)
    q8, sc = O.fp8_quant_block(nope.float())
    nope_deq = O.fp8_dequant_block(q8, sc)
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev, kv_cache_dtype="fp8")
    impl.update_sink_kv(rope[0].to(dev), nope[0].to(dev))
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    spec.sink_len = sink_len
    meta = mla.NPUMLAMetadataBuilder(spec, ["l"], _cfg(cap=2), dev).build(0, _to(common, dev))
    kvw = w.float().view(512, n, 256)
    ql = torch.einsum("tnp,lnp->tnl", q[..., :128].float(), kvw[..., :128]).bfloat16()
    o = O.sink_decode(ql, q[..., 128:].float(), nope_deq, rope, common.block_table_tensor.cpu(), common.seq_lens_cpu, sink_len,
                      impl.scale, None, query_start_loc=common.query_start_loc_cpu.tolist())
    ref = torch.einsum("tnl,lnv->tnv", o, kvw[..., 128:]).reshape(t, -1)
    out = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    impl.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), (cache,), meta, output=out)
    attn_close(out, ref, 6e-2, 1.2e-2)
    # ... and with a window
    impl_w, _ = _mk_impl(mla.NPUMLAImpl, n, dev, kv_cache_dtype="fp8", sliding_window=64)
    impl_w.update_sink_kv(rope[0].to(dev), nope[0].to(dev))
    o_w = O.sink_decode(ql, q[..., 128:].float(), nope_deq, rope, common.block_table_tensor.cpu(), common.seq_lens_cpu, sink_len,
                        impl.scale, 64, query_start_loc=common.query_start_loc_cpu.tolist())
    ref_w = torch.einsum("tnl,lnv->tnv", o_w, kvw[..., 128:]).reshape(t, -1)
    out_w = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    impl_w.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), (cache,), meta, output=out_w)
    attn_close(out_w, ref_w, 6e-2, 1.2e-2)


@pytest.mark.parametrize("batch,heads,lo,hi,sink_len,window,q_len,splits", [
    (4, 128, 200, 3000, 128, 512, 1, None), (3, 128, 1, 100, 128, 16, 1, 1), (3, 16, 300, 900, 256, 100, 2, 3),
    (2, 128, 600, 700, 128, 1, 3, 2), (5, 128, 1, 400, 0, 77, 2, None), (6, 64, 30, 2000, 128, 31, 4, 4),
    (3, 128, 500, 9000, 384, 1000, 1, 8), (4, 128, 100, 160, 128, 129, 2, 1)])
def test_fp8_window_decode_matches_oracle(dev, batch, heads, lo, hi, sink_len, window, q_len, splits):
    from omni_npu_amd import kernels as K
    c, bt = _sink_case(batch, heads, lo, hi, sink_len, q_len, seed=batch * 5 + heads + q_len + window)
    t = batch * q_len
    q8, sc = O.fp8_quant_block(c["nope"].float())
    deq = O.fp8_dequant_block(q8, sc)
    nblk = c["nope"].shape[0]
    cache = torch.zeros(nblk, 128, K.FP8_ROW_BYTES, dtype=torch.uint8, device=dev)
    K.cache_write_fp8(c["nope"].view(-1, 512).to(dev), c["rope"].view(-1, 64).to(dev), torch.arange(nblk * 128, device=dev), cache)
    out = torch.full((t, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    K.decode_fp8(c["q_nope"].to(dev), c["q_rope"].to(dev), cache, bt.to(dev), c["seq_lens"].to(dev), c["scale"], out, q_len=q_len,
                 num_splits=splits, sink_len=sink_len, window=window)
    if sink_len:
        ref = O.sink_decode(c["q_nope"], c["q_rope"], deq, c["rope"], bt, c["seq_lens"], sink_len, c["scale"], window)
    else:
        ref = O.absorbed_decode(c["q_nope"], c["q_rope"], deq, c["rope"], bt, c["seq_lens"], c["scale"], window=window)
    attn_close(out, ref, 6e-2, 6e-3)


@pytest.mark.parametrize("window", [None, 200])
def test_graph_replay_of_the_sink_decode_sees_new_lengths(dev, window):
    """The sink paths add work in front of the attention kernel (a length add, or the row list); captured in a HIP graph
    they must read the device tensors' new contents on every replay."""
    n, sink_len, nsb = 128, 128, 1
    q_lens, seq_lens = [1] * 5, [900, 130, 257, 64, 1000]
    common = _with_sink_pages(_common(q_lens, seq_lens), nsb)
    nblk = int(common.block_table_tensor.max()) + 1
    g = torch.Generator().manual_seed(19)
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16().to(dev)
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16().to(dev)
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev, sliding_window=window)
    impl.update_sink_kv(rope[0], nope[0])
    spec = V.AttentionSpec(128, 1, 576, torch.bfloat16)
    spec.sink_len = sink_len
    builder = mla.NPUMLAMetadataBuilder(spec, ["l"], _cfg(cap=1), dev)
    own = common.block_table_tensor[:, nsb:].clone()
    common.slot_mapping = torch.cat([O.slots_for(own, b, s - 1, s) for b, s in enumerate(seq_lens)])
    meta = builder.build(0, _to(common, dev))
    q = torch.randn(5, n, 192, generator=g).bfloat16().to(dev)
    kvc, kpe = torch.randn(5, 512, generator=g).bfloat16().to(dev), torch.randn(5, 1, 64, generator=g).bfloat16().to(dev)
    out = torch.zeros(5, n * 128, dtype=torch.bfloat16, device=dev)

    def model(qq):
        return impl.forward(None, qq, kvc, kpe, (nope, rope), meta, output=out)

    model(q)
    torch.cuda.synchronize()
    wrapper = HIPGraphWrapper(model, _cfg(), V.CUDAGraphMode.FULL)
    desc = V.BatchDescriptor(num_tokens=5, num_reqs=5, uniform=True)
    seen = []
    with V.set_forward_context({"l": meta}, desc, V.CUDAGraphMode.FULL):
        wrapper(q)
        for trial in range(3):
            q.copy_(torch.randn(5, n, 192, generator=g).bfloat16())
            new_lens = torch.tensor([s - 20 * (trial + 1) for s in seq_lens], dtype=torch.int32)
            meta.decode.seq_lens.copy_(new_lens.to(dev))
            meta.slot_mapping.copy_(torch.cat([O.slots_for(own, b, int(s) - 1, int(s)) for b, s in enumerate(new_lens)]).to(dev))
            got = wrapper(q).clone()
            torch.cuda.synchronize()
            out.zero_()
            eager = model(q).clone()
            assert torch.equal(got, eager), f"replay {trial} differs from eager"
            seen.append(got)
    assert not torch.equal(seen[0], seen[1])


# ---- seeded sweeps --------------------------------------------------------------------------------------------------
def _window_cases(n, seed):
    import random
    rng = random.Random(seed)
    out = []
    for i in range(n):
        q_len = rng.choice([1, 1, 2, 3, 4])
        heads = rng.choice([8, 16, 64, 128, 128])
        batch = rng.randint(1, 7)
        sink_len = rng.choice([0, 128, 128, 256])
        window = rng.choice([1, 2, 31, 32, 33, 63, 64, 100, 128, 129, 500, 1000])
        lo = rng.choice([q_len, q_len, 31, 32, 33, 64, 100, 129, 700])
        hi = lo + rng.choice([0, 1, 35, 300, 1500])
        splits = rng.choice([None, 1, 2, 3, 7, 30])
        out.append((i, batch, heads, q_len, sink_len, window, lo, hi, splits))
    return out


@pytest.mark.parametrize("i,batch,heads,q_len,sink_len,window,lo,hi,splits", _window_cases(48, seed=77))
def test_dense_window_decode_random_shapes(dev, i, batch, heads, q_len, sink_len, window, lo, hi, splits):
    """Window starts at every offset inside a 32-key block, windows shorter and longer than the sequences, sequences no
    longer than their query tokens, with and without a sink, split counts from one to more chunks than there is work."""
    from omni_npu_amd import kernels as K
    c, bt = _sink_case(batch, heads, lo, hi, sink_len, q_len, seed=3000 + i)
    t = batch * q_len
    out = torch.full((t, heads, 512), float("nan"), dtype=torch.bfloat16, device=dev)
    lse = torch.full((t, heads), float("nan"), dtype=torch.float32, device=dev)
    K.decode(c["q_nope"].to(dev), c["q_rope"].to(dev), c["nope"].to(dev), c["rope"].to(dev), bt.to(dev), c["seq_lens"].to(dev),
             c["scale"], out, q_len=q_len, lse_out=lse, num_splits=splits, sink_len=sink_len, window=window)
    if sink_len:
        ref = O.sink_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], sink_len, c["scale"], window)
    else:
        ref = O.absorbed_decode(c["q_nope"], c["q_rope"], c["nope"], c["rope"], bt, c["seq_lens"], c["scale"], window=window)
    attn_close(out, ref, MAX_ABS, MEAN_REL)
    assert torch.isfinite(lse).all()


def _prefill_window_cases(n, seed):
    import random
    rng = random.Random(seed)
    out = []
    for i in range(n):
        nseq = rng.randint(1, 3)
        q_lens = [rng.choice([1, 5, 31, 32, 33, 127, 128, 129, 300, 700]) for _ in range(nseq)]
        k_extra = [rng.choice([0, 0, 1, 40, 200]) for _ in range(nseq)]
        window = rng.choice([1, 2, 31, 32, 33, 64, 65, 127, 128, 129, 400, 5000])
        heads = rng.choice([1, 2, 8])
        out.append((i, q_lens, k_extra, window, heads))
    return out


@pytest.mark.parametrize("i,q_lens,k_extra,window,heads", _prefill_window_cases(24, seed=5))
def test_prefill_window_random_shapes(dev, i, q_lens, k_extra, window, heads):
    from omni_npu_amd import kernels as K
    g = torch.Generator().manual_seed(4000 + i)
    k_lens = [a + b for a, b in zip(q_lens, k_extra)]
    cu_q = [0] + torch.tensor(q_lens).cumsum(0).tolist()
    cu_k = [0] + torch.tensor(k_lens).cumsum(0).tolist()
    t, tk = cu_q[-1], cu_k[-1]
    qn, qp = torch.randn(t, heads, 128, generator=g).bfloat16(), torch.randn(t, heads, 64, generator=g).bfloat16()
    kn, kp = torch.randn(tk, heads, 128, generator=g).bfloat16(), torch.randn(tk, 64, generator=g).bfloat16()
    v = torch.randn(tk, heads, 128, generator=g).bfloat16()
    scale = 192 ** -0.5
    out = torch.full((t, heads, 128), float("nan"), dtype=torch.float32, device=dev)
    lse = torch.full((t, heads), float("nan"), dtype=torch.float32, device=dev)
    K.prefill_varlen(qn.to(dev), qp.to(dev), kn.to(dev), kp.to(dev), v.to(dev), torch.tensor(cu_q, dtype=torch.int32, device=dev),
                     torch.tensor(cu_k, dtype=torch.int32, device=dev), max(q_lens), scale, True, out, lse, window=window)
    ref, ref_lse = O.attention_varlen(qn, qp, kn, kp, v, cu_q, cu_k, scale, True, window=window)
    attn_close(out, ref, MAX_ABS, MEAN_REL)
    assert (lse.cpu() - ref_lse).abs().max() < 2e-2
