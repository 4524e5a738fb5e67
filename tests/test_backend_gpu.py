"""Impl.forward of both backends end to end on the GPU (cache write -> attention -> up-projection) against the
oracle, driven through the metadata builders, plus HIP-graph capture/replay through the graph wrapper.
Shapes follow the reference's numeric tests (tests/integration/attention/test_npu_mla_math.py: 4 heads, (B,S) in
{(1,16),(8,160)}; test_mla_chunked_prefill.py: context 48 = [32,16], suffix 16) and the benchmark head count."""
from types import SimpleNamespace

import pytest
import torch

from omni_npu_amd import _vllm_compat as V
from omni_npu_amd.attention.backends import dsa, mla
from omni_npu_amd.compilation.acl_graph import HIPGraphWrapper
from oracle import mla_oracle as O
from tests.conftest import attn_close
from tests.test_boundary import _cfg, _common

pytestmark = pytest.mark.gpu


def _mk_impl(cls, n, dev, seed=0, **over):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(512, n * 256, generator=g) * 0.05).bfloat16()
    proj = lambda x: (x @ w.to(x.device),)
    kw = dict(num_heads=n, head_size=576, scale=192 ** -0.5, num_kv_heads=1, alibi_slopes=None, sliding_window=None,
              kv_cache_dtype="auto", logits_soft_cap=None, attn_type=V.AttentionType.DECODER,
              kv_sharing_target_layer_name=None, q_lora_rank=None, kv_lora_rank=512, qk_nope_head_dim=128,
              qk_rope_head_dim=64, qk_head_dim=192, v_head_dim=128, kv_b_proj=proj)
    kw.update(over)
    impl = cls(**kw)
    kv = w.view(512, n, 256)
    impl.W_UK_T = kv[..., :128].permute(1, 2, 0).contiguous().to(dev)
    impl.W_UV = kv[..., 128:].transpose(0, 1).contiguous().to(dev)
    return impl, w


def _to(c, dev):
    for f in ("query_start_loc", "seq_lens", "block_table_tensor", "slot_mapping"):
        setattr(c, f, getattr(c, f).to(dev))
    return c


def _oracle_mla(q, kvc, kpe, w, nope, rope, common, n, scale):
    """Reference semantics of NPUMLAImpl.forward in fp32 on the CPU."""
    O.cache_write(nope, common.slot_mapping, kvc)
    O.cache_write(rope, common.slot_mapping, kpe.view(-1, 64))
    qsl = common.query_start_loc_cpu.tolist()
    out = torch.zeros(q.shape[0], n * 128)
    kvw = w.float().view(512, n, 256)
    for b in range(common.num_reqs):
        L, q0, q1 = int(common.seq_lens_cpu[b]), qsl[b], qsl[b + 1]
        rows = O.slots_for(common.block_table_tensor.cpu(), b, 0, L)
        lat, pe = nope.view(-1, 512)[rows].float(), rope.view(-1, 64)[rows].float()
        kn, vv = O.kv_up_proj(lat, w.float(), n, 128, 128)
        o, _ = O.attention_varlen(q[q0:q1, :, :128], q[q0:q1, :, 128:], kn, pe, vv, [0, q1 - q0], [0, L], scale, True)
        out[q0:q1] = o.reshape(q1 - q0, -1)
    return out


@pytest.mark.parametrize("q_lens,seq_lens,n", [
    ([1] * 8, [160] * 8, 4),                 # pure decode
    ([16], [16], 4),                         # pure prefill, no context
    ([1, 1, 16, 16], [300, 77, 64, 64], 4),  # mixed: 2 decodes, then 2 prefills with 48 tokens of chunked context
    ([2, 2, 2], [500, 129, 1000], 128),      # MTP pairs at the benchmark head count
])
def test_mla_impl_forward_matches_reference_semantics(dev, q_lens, seq_lens, n):
    g = torch.Generator().manual_seed(len(q_lens))
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    # slots of the new tokens: the last q_len positions of each sequence
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev)
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l"], _cfg(cap=2), dev)
    builder.chunked_prefill_workspace_size = 64
    ref = _oracle_mla(q.float(), kvc, kpe, w, nope.clone(), rope.clone(), common, n, impl.scale)
    meta = builder.build(0, _to(common, dev))
    raw = torch.cat([nope.reshape(-1), rope.reshape(-1)]).to(dev).view(torch.uint8)
    kv_cache = mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 576, dtype=torch.bfloat16)
    out = torch.full((t + 3, n * 128), 7.0, dtype=torch.bfloat16, device=dev)          # padded output buffer
    res = impl.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out)
    assert res is out and (out[t:] == 7).all()                                          # padding rows untouched
    attn_close(out[:t], ref, 3e-2, 8e-3)                                                # the reference's 3e-2 bar


class _PlainLinear:
    """An up-projection as the model owns it when nothing is quantised: a weight [out, in] and a call that returns a tuple."""

    def __init__(self, w_in_out, dev):
        self.weight = w_in_out.t().contiguous().to(dev)
        self.bias = None
        self.calls = 0

    def __call__(self, x):
        self.calls += 1
        return (x @ self.weight.t(),)


@pytest.mark.parametrize("fp16_path", [True, False])
def test_mla_prefill_with_a_plain_up_projection_makes_keys_and_values_in_fp16(dev, fp16_path):
    """Where kv_b_proj is a plain weight the prefill makes k_nope and v with an fp16 GEMM (the kernel then converts no value
    tile) instead of calling the module; prefill_kv_fp16 = False keeps the module's bf16 call.  Both against the oracle,
    mixed batch with a chunked context, and against each other."""
    q_lens, seq_lens, n = [1, 1, 16, 16], [300, 77, 64, 64], 4
    g = torch.Generator().manual_seed(11)
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev)
    impl.kv_b_proj = _PlainLinear(w, dev)
    impl.prefill_kv_fp16 = fp16_path
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l"], _cfg(cap=2), dev)
    builder.chunked_prefill_workspace_size = 64
    ref = _oracle_mla(q.float(), kvc, kpe, w, nope.clone(), rope.clone(), common, n, impl.scale)
    meta = builder.build(0, _to(common, dev))
    raw = torch.cat([nope.reshape(-1), rope.reshape(-1)]).to(dev).view(torch.uint8)
    kv_cache = mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 576, dtype=torch.bfloat16)
    out = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    impl.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out)
    attn_close(out, ref, 3e-2, 8e-3)
    # the module is called only where the fp16 path is off (prefill: the suffix and one context chunk)
    assert (impl.kv_b_proj.calls == 0) == fp16_path


def test_mla_impl_forward_fp8_cache_with_chunked_context(dev):
    """NPUMLAImpl.forward over the fp8 block-scaled cache, mixed batch: decodes read the quantised cache (the new token
    included), prefills attend over their own un-quantised suffix plus a chunked context gathered and dequantised from
    the cache (two chunks of the 64-row workspace).  The oracle sees exactly those values."""
    from omni_npu_amd import kernels as K
    q_lens, seq_lens, n = [1, 1, 16, 16], [300, 77, 112, 64], 4
    g = torch.Generator().manual_seed(11)
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev, kv_cache_dtype="fp8")
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l"], _cfg(cap=2), dev)
    builder.chunked_prefill_workspace_size = 64
    deq = lambda x: O.fp8_dequant_block(*O.fp8_quant_block(x.float()))
    # oracle: what the cache holds after the write, dequantised; prefill suffixes use the raw new latents
    nope_q, rope_c = deq(nope), rope.clone().float()
    O.cache_write(nope_q, common.slot_mapping, deq(kvc))
    O.cache_write(rope_c, common.slot_mapping, kpe.view(-1, 64).float())
    qsl = common.query_start_loc_cpu.tolist()
    ref = torch.zeros(t, n * 128)
    for b in range(common.num_reqs):
        L, q0, q1 = seq_lens[b], qsl[b], qsl[b + 1]
        rows = O.slots_for(common.block_table_tensor.cpu(), b, 0, L)
        lat, pe = nope_q.view(-1, 512)[rows].clone(), rope_c.view(-1, 64)[rows]
        if q_lens[b] > 1:
            lat[L - q_lens[b]:] = kvc[q0:q1].float()            # the suffix is attended before it is quantised
        kn, vv = O.kv_up_proj(lat, w.float(), n, 128, 128)
        o, _ = O.attention_varlen(q[q0:q1, :, :128].float(), q[q0:q1, :, 128:].float(), kn, pe, vv, [0, q1 - q0], [0, L],
                                  impl.scale, True)
        ref[q0:q1] = o.reshape(q1 - q0, -1)
    meta = builder.build(0, _to(common, dev))
    assert meta.prefill.chunked_context is not None and len(meta.prefill.chunked_context.seq_tot) >= 2
    raw = torch.zeros(nblk * 128 * 656, dtype=torch.uint8, device=dev)
    kv_cache = mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 656, dtype=torch.uint8)
    K.cache_write_fp8(nope.view(-1, 512).to(dev), rope.view(-1, 64).to(dev),
                      torch.arange(nblk * 128, dtype=torch.int64, device=dev), kv_cache[0])
    out = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    impl.forward(SimpleNamespace(_k_scale=None), q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out)
    attn_close(out, ref, 3e-2, 8e-3)


def test_dsa_impl_forward_with_indexer(dev):
    """Indexer (quantise, cache K, fp8 logits, top-k) -> NPUDSAImpl.forward; checked against the oracle's sparse
    attention on the index set the GPU selected, and the set against the oracle's selection on the GPU's logits."""
    g = torch.Generator().manual_seed(3)
    n, topk = 128, 64
    q_lens, seq_lens = [1, 1, 1, 40], [700, 90, 300, 40]      # three decodes and one prefill without context
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    raw = torch.zeros(nblk * 128 * 704, dtype=torch.bfloat16, device=dev).view(torch.uint8)
    kv_cache = dsa.NPUDSABackend.reshape_kv_cache(raw, nblk, 128, 1, 704, dtype=torch.bfloat16)
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    idx_k = torch.randn(nblk, 128, 128, generator=g).bfloat16()
    kv_cache[0].copy_(nope.view(nblk, 128, 1, 512)); kv_cache[1].copy_(rope.view(nblk, 128, 1, 64))
    k8_ref, ks_ref = O.fp8_quant_token(idx_k.float())
    k8v, ksv = dsa.indexer_cache_views(kv_cache[2])
    k8v.copy_(k8_ref.view(torch.uint8)); ksv.copy_(ks_ref)

    impl, w = _mk_impl(dsa.NPUDSAImpl, n, dev)
    indexer = dsa.LightningIndexer(topk, max_tokens=t + 2, device=dev)
    impl.indexer = indexer
    builder = dsa.NPUDSAMetadataBuilder(V.AttentionSpec(128, 1, 704, torch.bfloat16), ["l"], _cfg(cap=1), dev)
    meta = builder.build(0, _to(common, dev))
    q = torch.randn(t, n, 192, generator=g).bfloat16()
    kvc, kpe = torch.randn(t, 512, generator=g).bfloat16(), torch.randn(t, 1, 64, generator=g).bfloat16()
    iq, ik, iw = torch.randn(t, 64, 128, generator=g).bfloat16(), torch.randn(t, 128, generator=g).bfloat16(), torch.randn(t, 64, generator=g)
    sel = indexer(iq.to(dev), ik.to(dev), iw.to(dev), kv_cache, meta)
    assert sel.shape == (t, 1, topk) and indexer.topk_indices_buffer[:t].data_ptr() == sel.data_ptr()
    # the new keys were quantised into the cache exactly as the oracle quantises them
    k8_new, ks_new = O.fp8_quant_token(ik.float())
    sm = common.slot_mapping.cpu()
    assert torch.equal(k8v.cpu()[sm // 128, sm % 128], k8_new.view(torch.uint8))
    assert torch.equal(ksv.cpu()[sm // 128, sm % 128], ks_new)
    out = torch.zeros(t, n * 128, dtype=torch.bfloat16, device=dev)
    assert indexer.rows_for(meta) is not None and indexer.rows_for(object()) is None
    impl.forward(None, q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out)
    # the same forward when the picks come without their cache rows (an indexer that only fills the index buffer): the
    # positions are translated by a launch of their own, same result bit for bit
    indexer._rows_meta = None
    out2 = torch.zeros_like(out)
    impl.forward(None, q.to(dev), kvc.to(dev), kpe.to(dev), kv_cache, meta, output=out2)
    assert torch.equal(out, out2)

    # oracle: caches after the write, per-token visible length, sparse attention on the selected positions
    O.cache_write(nope, common.slot_mapping.cpu(), kvc); O.cache_write(rope, common.slot_mapping.cpu(), kpe.view(-1, 64))
    sel_cpu = sel.cpu()
    qsl = [0, 1, 2, 3, 43]
    ref = torch.zeros(t, n * 128)
    ql = O.q_absorb(q[..., :128], impl.W_UK_T.cpu())
    for b in range(4):
        for i in range(qsl[b + 1] - qsl[b]):
            tok = qsl[b] + i
            vis = seq_lens[b] - q_lens[b] + i + 1
            valid = sel_cpu[tok, 0][sel_cpu[tok, 0] >= 0]
            assert valid.numel() == min(topk, vis) and int(valid.max()) < vis
            o = O.sparse_decode(ql[tok:tok + 1].bfloat16(), q[tok:tok + 1, :, 128:], nope, rope,
                                common.block_table_tensor[b:b + 1].cpu(), [vis], sel_cpu[tok:tok + 1], impl.scale)
            ref[tok] = O.v_up_proj(o.transpose(0, 1).contiguous().bfloat16(), impl.W_UV.cpu()).view(-1)
    attn_close(out, ref, 3e-2, 8e-3)


def test_graph_wrapper_captures_and_replays_the_decode_forward(dev):
    """FULL mode: first call captures a HIP graph for the batch descriptor, later calls replay it and see the device
    tensors' new contents; a second descriptor gets its own graph; NONE runs eagerly."""
    n = 128
    q_lens, seq_lens = [1] * 6, [900, 130, 257, 64, 511, 1000]
    common = _common(q_lens, seq_lens)
    nblk = int(common.block_table_tensor.max()) + 1
    g = torch.Generator().manual_seed(9)
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16().to(dev)
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16().to(dev)
    impl, w = _mk_impl(mla.NPUMLAImpl, n, dev)
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l"], _cfg(cap=1), dev)
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - 1, s) for b, s in enumerate(seq_lens)])
    meta = builder.build(0, _to(common, dev))
    q = torch.randn(6, n, 192, generator=g).bfloat16().to(dev)
    kvc, kpe = torch.randn(6, 512, generator=g).bfloat16().to(dev), torch.randn(6, 1, 64, generator=g).bfloat16().to(dev)
    out = torch.zeros(6, n * 128, dtype=torch.bfloat16, device=dev)

    def model(qq):
        return impl.forward(None, qq, kvc, kpe, (nope, rope), meta, output=out)

    model(q)                                                  # warm-up (allocations, LDS attribute) outside capture
    torch.cuda.synchronize()
    wrapper = HIPGraphWrapper(model, _cfg(), V.CUDAGraphMode.FULL)
    desc = V.BatchDescriptor(num_tokens=6, num_reqs=6, uniform=True)
    with V.set_forward_context({"l": meta}, desc, V.CUDAGraphMode.FULL):
        wrapper(q)                                            # capture
        assert desc in wrapper.concrete_graph_entries and wrapper.concrete_graph_entries[desc].graph is not None
        for trial in range(3):
            q.copy_(torch.randn(6, n, 192, generator=g).bfloat16())
            new_lens = torch.tensor([s - 10 * (trial + 1) for s in seq_lens], dtype=torch.int32)
            meta.decode.seq_lens.copy_(new_lens.to(dev))
            meta.slot_mapping.copy_(torch.cat([O.slots_for(common.block_table_tensor.cpu(), b, int(s) - 1, int(s))
                                               for b, s in enumerate(new_lens)]).to(dev))
            got = wrapper(q).clone()                          # replay
            torch.cuda.synchronize()
            out.zero_()
            eager = model(q).clone()
            assert torch.equal(got, eager), f"replay {trial} differs from eager"
    with V.set_forward_context({"l": meta}, desc, V.CUDAGraphMode.NONE):
        assert wrapper(q) is out and len(wrapper.concrete_graph_entries) == 1


def test_graph_wrapper_options_act_on_the_capture(dev):
    """``gc_disable`` silences gc.collect / empty_cache for the duration of a capture only, ``weak_ref_output`` hands back an
    alias that owns nothing (the graph's pool keeps the bytes), and replays still see new input contents
    (reference acl_graph.py:190-222)."""
    import gc
    from omni_npu_amd.compilation.acl_graph import HIPGraphOptions
    real_collect, real_empty = gc.collect, torch.cuda.empty_cache
    seen = {}

    def runnable(x):
        seen["collect"], seen["empty"] = gc.collect, torch.cuda.empty_cache
        return x * 2 + 1, x.float().sum(dim=-1)

    x = torch.arange(24, dtype=torch.bfloat16, device=dev).view(4, 6)
    runnable(x)
    torch.cuda.synchronize()
    for gc_disable, weak in ((True, True), (False, False)):
        w = HIPGraphWrapper(runnable, _cfg(), V.CUDAGraphMode.FULL,
                            cudagraph_options=HIPGraphOptions(debug_log_enable=False, gc_disable=gc_disable,
                                                              weak_ref_output=weak))
        desc = V.BatchDescriptor(num_tokens=4, num_reqs=4, uniform=True)
        with V.set_forward_context(None, desc, V.CUDAGraphMode.FULL):
            first = w(x)
            assert (seen["collect"] is not real_collect) == gc_disable and (seen["empty"] is not real_empty) == gc_disable
            assert gc.collect is real_collect and torch.cuda.empty_cache is real_empty     # restored after the capture
            held = w.concrete_graph_entries[desc].output
            assert isinstance(first, tuple) and isinstance(held, tuple)
            for a, b in zip(first, held):
                assert a.data_ptr() == b.data_ptr() and a.shape == b.shape and a.dtype == b.dtype
                # the entry's copy never owns the bytes: its storage is a bare span, not the allocator's block
                assert b.untyped_storage().data_ptr() == b.data_ptr()
            for k in range(3):
                x.copy_(torch.arange(24, dtype=torch.bfloat16).view(4, 6) + k)
                y, ssum = w(x)
                torch.cuda.synchronize()
                assert torch.equal(y, x * 2 + 1) and torch.equal(ssum, x.float().sum(dim=-1))
