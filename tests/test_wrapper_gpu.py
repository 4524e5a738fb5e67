"""The caller of the backends end to end on the GPU: hidden states -> forward_oot (projections, norms, rotary embedding,
cache write, attention, output projection) against an fp32 torch restatement of the same chain on the CPU, and the
indexer module (projections, LayerNorm, rotary embedding, selection) against the oracle's selection.

Bar: the reference's end-to-end 3e-2 (tests/integration/attention/test_npu_mla_math.py:147-156), taken relative to the
output scale because the chain here ends in an output projection of arbitrary gain."""
from types import SimpleNamespace

import pytest
import torch

from omni_npu_amd import _vllm_compat as V
from omni_npu_amd.attention.backends import dsa, mla
from oracle import mla_oracle as O
from tests.test_backend_gpu import _mk_impl, _oracle_mla, _to
from tests.test_boundary import _cfg, _common

pytestmark = pytest.mark.gpu
EPS = 1e-6


class _Lin(torch.nn.Module):                     # same call shape as vLLM's linear layers: returns (out, bias)
    def __init__(self, w):
        super().__init__()
        self.w = w

    def forward(self, x):
        return x @ self.w, None


class _Norm(torch.nn.Module):                    # RMSNorm with the attribute names of vLLM's
    def __init__(self, weight, eps=EPS):
        super().__init__()
        self.weight, self.variance_epsilon = weight, eps

    def forward(self, x):
        return torch.nn.functional.rms_norm(x.float(), (x.shape[-1],), self.weight.float(), self.variance_epsilon).to(x.dtype)


def _weights(g, hidden, n, q_lora):
    s = lambda *shape, gain: (torch.randn(*shape, generator=g) * gain).bfloat16()
    return dict(qkv_a=s(hidden, q_lora + 576, gain=hidden ** -0.5), q_b=s(q_lora, n * 192, gain=q_lora ** -0.5),
                q_norm=(1 + 0.1 * torch.randn(q_lora, generator=g)).bfloat16(),
                kv_norm=(1 + 0.1 * torch.randn(512, generator=g)).bfloat16(), o=s(n * 128, hidden, gain=(n * 128) ** -0.5))


@pytest.mark.parametrize("q_lens,seq_lens,fused", [([1] * 6, [200, 31, 129, 500, 64, 1000], True),
                                                   ([1, 1, 24], [300, 77, 24], True),
                                                   ([2, 2], [150, 400], False)])
def test_forward_oot_matches_fp32_chain(dev, monkeypatch, q_lens, seq_lens, fused):
    from omni_npu_amd.layers.attention.npu_mla_wrapper import MLAAttention, NPUMultiHeadLatentAttentionWrapper
    from omni_npu_amd.layers.rotary_embedding import HIPRotaryEmbedding
    g = torch.Generator().manual_seed(sum(seq_lens))
    hidden, n, q_lora = 256, 16, 128
    w = _weights(g, hidden, n, q_lora)
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    positions = torch.cat([torch.arange(s - ql, s) for ql, s in zip(q_lens, seq_lens)])
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    x = torch.randn(t, hidden, generator=g).bfloat16()

    impl, w_kv_b = _mk_impl(mla.NPUMLAImpl, n, dev, seed=5)
    attn = MLAAttention(impl)
    raw = torch.cat([nope.reshape(-1), rope.reshape(-1)]).to(dev).view(torch.uint8)
    attn.kv_cache = [mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 576, dtype=torch.bfloat16)]
    attn._k_scale = None
    rotary = HIPRotaryEmbedding(max_position=2048, device=dev)
    kv_norm = _Norm(w["kv_norm"].to(dev))
    if not fused:                                             # a norm without exposed parameters: the two-module path
        inner = kv_norm
        kv_norm = lambda v: inner(v)
    wrap = NPUMultiHeadLatentAttentionWrapper(hidden, n, 128, 64, 128, q_lora, 512, attn, kv_norm, _Lin(w["o"].to(dev)),
                                              rotary_emb=rotary, fused_qkv_a_proj=_Lin(w["qkv_a"].to(dev)),
                                              q_a_layernorm=_Norm(w["q_norm"].to(dev)), q_b_proj=_Lin(w["q_b"].to(dev)))
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l"], _cfg(cap=2), dev)
    builder.chunked_prefill_workspace_size = 64

    # ---- fp32 chain on the CPU (bf16 rounding only where the GPU chain stores bf16 tensors) ----
    qkv = (x.float() @ w["qkv_a"].float()).bfloat16()
    q_c = torch.nn.functional.rms_norm(qkv[:, :q_lora].float(), (q_lora,), w["q_norm"].float(), EPS).bfloat16()
    q = (q_c.float() @ w["q_b"].float()).bfloat16().view(t, n, 192)
    cos, sin = O.rope_tables(positions)
    kv_a = O.rms_norm(qkv[:, q_lora:q_lora + 512], w["kv_norm"], EPS)
    k_pe = O.interleave_rope(qkv[:, q_lora + 512:], cos, sin)
    q = torch.cat([q[..., :128], O.interleave_rope(q[..., 128:], cos, sin)], -1)
    attn_ref = _oracle_mla(q.float(), kv_a, k_pe.view(t, 1, 64), w_kv_b, nope.clone(), rope.clone(), common, n, impl.scale)
    ref = attn_ref.bfloat16().float() @ w["o"].float()

    meta = builder.build(0, _to(common, dev))
    from omni_npu_amd import kernels as K
    writes = []
    real_write = K.cache_write
    monkeypatch.setattr(K, "cache_write", lambda *a, **k: writes.append(1) or real_write(*a, **k))
    with V.set_forward_context(attn_metadata={attn.layer_name: meta}):
        out = wrap.forward_oot(positions.to(dev), x.to(dev))
    assert out.shape == (t, hidden)
    # fused path: the norm + rope launch wrote the cache rows and the impl skipped its own write; two-module path: the impl's
    assert len(writes) == (0 if fused else 1) and impl.cache_written_for is None
    err = (out.float().cpu() - ref).abs().max().item()
    assert err <= 3e-2 * ref.abs().max().item(), f"max err {err:.4g} vs scale {ref.abs().max().item():.4g}"
    # the cache rows of the new tokens hold the normalised latent and the rotated key (to the last bf16 bit but one)
    sm = common.slot_mapping.cpu()
    got_n = attn.kv_cache[0][0].cpu().view(-1, 512)[sm]
    got_r = attn.kv_cache[0][1].cpu().view(-1, 64)[sm]
    assert ((got_n.view(torch.int16).int() - kv_a.view(torch.int16).int()).abs() <= 1).all()
    assert ((got_r.view(torch.int16).int() - k_pe.view(torch.int16).int()).abs() <= 1).all()


@pytest.mark.parametrize("q_lens,seq_lens", [([1] * 5, [200, 31, 129, 500, 1000]), ([2, 2, 2], [150, 400, 77]),
                                             ([40, 7, 130], [40, 7, 130])])
def test_custom_model_module_matches_fp32_chain(dev, q_lens, seq_lens):
    """``NPUDeepseekMLAAttention.forward(hidden_states, cos, sin)`` (src/omni_npu/v1/layers/attention/npu_mla.py:152-348):
    all-decode batches (MTP too) and all-prefill batches without cached context, against the fp32 chain on the CPU."""
    from omni_npu_amd.layers.attention.npu_mla_wrapper import MLAAttention
    from omni_npu_amd.v1.layers.attention import NPUDeepseekMLAAttention
    g = torch.Generator().manual_seed(sum(seq_lens) + len(q_lens))
    hidden, n, q_lora = 256, 16, 128
    w = _weights(g, hidden, n, q_lora)
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    positions = torch.cat([torch.arange(s - ql, s) for ql, s in zip(q_lens, seq_lens)])
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    x = torch.randn(t, hidden, generator=g).bfloat16()

    impl, w_kv_b = _mk_impl(mla.NPUMLAImpl, n, dev, seed=5)
    attn = MLAAttention(impl)
    raw = torch.cat([nope.reshape(-1), rope.reshape(-1)]).to(dev).view(torch.uint8)
    attn.kv_cache = [mla.NPUMLABackend.reshape_kv_cache(raw, nblk, 128, 1, 576, dtype=torch.bfloat16)]
    wq_a, wkv_a = w["qkv_a"][:, :q_lora].contiguous(), w["qkv_a"][:, q_lora:].contiguous()
    mod = NPUDeepseekMLAAttention(hidden, n, 128, 64, 128, q_lora, 512, attn, _Lin(wq_a.to(dev)), _Norm(w["q_norm"].to(dev)),
                                  _Lin(w["q_b"].to(dev)), _Lin(wkv_a.to(dev)), _Norm(w["kv_norm"].to(dev)), _Lin(w["o"].to(dev)))
    builder = mla.NPUMLAMetadataBuilder(V.AttentionSpec(128, 1, 576, torch.bfloat16), ["l"], _cfg(cap=2), dev)

    # ---- fp32 chain on the CPU (bf16 rounding only where the GPU chain stores bf16 tensors) ----
    q_c = torch.nn.functional.rms_norm((x.float() @ wq_a.float()).bfloat16().float(), (q_lora,), w["q_norm"].float(),
                                       EPS).bfloat16()
    q = (q_c.float() @ w["q_b"].float()).bfloat16().view(t, n, 192)
    kv = (x.float() @ wkv_a.float()).bfloat16()
    cos, sin = O.rope_tables(positions)
    kv_a = O.rms_norm(kv[:, :512], w["kv_norm"], EPS)
    k_pe = O.interleave_rope(kv[:, 512:], cos, sin)
    q = torch.cat([q[..., :128], O.interleave_rope(q[..., 128:], cos, sin)], -1)
    attn_ref = _oracle_mla(q.float(), kv_a, k_pe.view(t, 1, 64), w_kv_b, nope.clone(), rope.clone(), common, n, impl.scale)
    ref = attn_ref.bfloat16().float() @ w["o"].float()

    meta = builder.build(0, _to(common, dev))
    assert (meta.prefill is None) != (meta.decode is None)
    cd, sd = cos.to(dev).view(-1, 1, 1, 64), sin.to(dev).view(-1, 1, 1, 64)
    with V.set_forward_context(attn_metadata={attn.layer_name: meta}):
        out = mod(x.to(dev), cd, sd)
    assert out.shape == (t, hidden)
    err = (out.float().cpu() - ref).abs().max().item()
    assert err <= 3e-2 * ref.abs().max().item(), f"max err {err:.4g} vs scale {ref.abs().max().item():.4g}"
    sm = common.slot_mapping.cpu()
    got_n = attn.kv_cache[0][0].cpu().view(-1, 512)[sm]
    got_r = attn.kv_cache[0][1].cpu().view(-1, 64)[sm]
    # (the kv projection is a bf16 GEMM on the GPU and an fp32 product rounded once here, so a projected value can land on
    # the other side of a rounding boundary: the bar is one bf16 step of the value, or of 1/16 for values that are
    # differences of larger terms, and almost all of them identical to the last bit but one)
    for got, want in ((got_n, kv_a), (got_r, k_pe)):
        step = 2.0 ** -7 * want.float().abs().clamp(min=1 / 16)
        assert ((got.float() - want.float()).abs() <= step).all()
        d = (got.view(torch.int16).int() - want.view(torch.int16).int()).abs()
        assert float((d <= 1).float().mean()) >= 0.999
    # memory-profiling run: no metadata, no cache access, the projections still run
    with V.set_forward_context(attn_metadata=None):
        dry = mod(x.to(dev), cd, sd)
    assert dry.shape == (t, hidden) and float(dry.abs().max()) == 0.0


@pytest.mark.parametrize("q_lens,seq_lens", [([1, 1, 1], [700, 90, 300]), ([40, 9], [40, 9])])
def test_custom_model_sparse_module(dev, q_lens, seq_lens):
    """``NPUDeepseekSparseAttention.forward(hidden_states, cos, sin)`` (src/omni_npu/v1/layers/attention/npu_dsa.py:296-586):
    the output against the oracle's sparse attention over the positions the module's own indexer selected (the selection
    itself is covered by test_indexer_module_selects_what_the_oracle_selects), wrapped in the fp32 chain of projections."""
    from omni_npu_amd.layers.attention.indexer import DSV32Indexer
    from omni_npu_amd.layers.attention.npu_mla_wrapper import MLAAttention
    from omni_npu_amd.v1.layers.attention import NPUDeepseekSparseAttention
    torch.manual_seed(1)
    g = torch.Generator().manual_seed(sum(seq_lens))
    hidden, n, q_lora, topk = 256, 128, 128, 64
    w = _weights(g, hidden, n, q_lora)
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    positions = torch.cat([torch.arange(s - ql, s) for ql, s in zip(q_lens, seq_lens)])
    raw = torch.zeros(nblk * 128 * 704, dtype=torch.bfloat16, device=dev).view(torch.uint8)
    kv_cache = dsa.NPUDSABackend.reshape_kv_cache(raw, nblk, 128, 1, 704, dtype=torch.bfloat16)
    nope = torch.randn(nblk, 128, 512, generator=g).bfloat16()
    rope = torch.randn(nblk, 128, 64, generator=g).bfloat16()
    kv_cache[0].copy_(nope.view(nblk, 128, 1, 512)); kv_cache[1].copy_(rope.view(nblk, 128, 1, 64))
    k8_ref, ks_ref = O.fp8_quant_token(torch.randn(nblk, 128, 128, generator=g).bfloat16().float())
    k8v, ksv = dsa.indexer_cache_views(kv_cache[2])
    k8v.copy_(k8_ref.view(torch.uint8)); ksv.copy_(ks_ref)
    x = torch.randn(t, hidden, generator=g).bfloat16()

    impl, w_kv_b = _mk_impl(dsa.NPUDSAImpl, n, dev, seed=5)
    attn = MLAAttention(impl)
    attn.kv_cache = [kv_cache]
    idx = DSV32Indexer(hidden, q_lora, topk, max_tokens=t, device=dev)
    wq_a, wkv_a = w["qkv_a"][:, :q_lora].contiguous(), w["qkv_a"][:, q_lora:].contiguous()
    mod = NPUDeepseekSparseAttention(hidden, n, 128, 64, 128, q_lora, 512, attn, idx, _Lin(wq_a.to(dev)),
                                     _Norm(w["q_norm"].to(dev)), _Lin(w["q_b"].to(dev)), _Lin(wkv_a.to(dev)),
                                     _Norm(w["kv_norm"].to(dev)), _Lin(w["o"].to(dev)))
    builder = dsa.NPUDSAMetadataBuilder(V.AttentionSpec(128, 1, 704, torch.bfloat16), ["l"], _cfg(cap=1), dev)
    meta = builder.build(0, _to(common, dev))
    cos, sin = O.rope_tables(positions)
    cd, sd = cos.to(dev).view(-1, 1, 1, 64), sin.to(dev).view(-1, 1, 1, 64)
    with V.set_forward_context(attn_metadata={attn.layer_name: meta}):
        out = mod(x.to(dev), cd, sd)
    assert out.shape == (t, hidden)
    sel = idx.topk_indices_buffer[:t].view(t, 1, topk).cpu()

    q_c = torch.nn.functional.rms_norm((x.float() @ wq_a.float()).bfloat16().float(), (q_lora,), w["q_norm"].float(),
                                       EPS).bfloat16()
    q = (q_c.float() @ w["q_b"].float()).bfloat16().view(t, n, 192)
    kv = (x.float() @ wkv_a.float()).bfloat16()
    kv_a = O.rms_norm(kv[:, :512], w["kv_norm"], EPS)
    k_pe = O.interleave_rope(kv[:, 512:], cos, sin)
    q_pe = O.interleave_rope(q[..., 128:], cos, sin)
    sm = common.slot_mapping.cpu()
    O.cache_write(nope, sm, kv_a); O.cache_write(rope, sm, k_pe)
    ql = O.q_absorb(q[..., :128], impl.W_UK_T.cpu())
    attn_ref = torch.zeros(t, n * 128)
    tok = 0
    for b, (qlen, L) in enumerate(zip(q_lens, seq_lens)):
        for i in range(qlen):
            vis = L - qlen + i + 1
            valid = sel[tok, 0][sel[tok, 0] >= 0]
            assert valid.numel() == min(topk, vis) and int(valid.max()) < vis
            o = O.sparse_decode(ql[tok:tok + 1].bfloat16(), q_pe[tok:tok + 1], nope, rope,
                                common.block_table_tensor[b:b + 1].cpu(), [vis], sel[tok:tok + 1], impl.scale)
            attn_ref[tok] = O.v_up_proj(o.transpose(0, 1).contiguous().bfloat16(), impl.W_UV.cpu()).view(-1)
            tok += 1
    ref = attn_ref.bfloat16().float() @ w["o"].float()
    err = (out.float().cpu() - ref).abs().max().item()
    assert err <= 3e-2 * ref.abs().max().item(), f"max err {err:.4g} vs scale {ref.abs().max().item():.4g}"
    with V.set_forward_context(attn_metadata=None):
        dry = mod(x.to(dev), cd, sd)
    assert dry.shape == (t, hidden) and float(dry.abs().max()) == 0.0


@pytest.mark.parametrize("variant", ["positions", "tables"])
def test_indexer_module_selects_what_the_oracle_selects(dev, variant):
    """``positions``: the patched module (patch_dsv32_indexer.py:77-146, rotary module, interleaved pairs); ``tables``:
    the custom-model module (npu_dsa.py:105-142, cos / sin rows, half-rotation pairing)."""
    from omni_npu_amd.layers.attention.indexer import DSV32Indexer
    from omni_npu_amd.layers.rotary_embedding import HIPRotaryEmbedding
    torch.manual_seed(0)
    hidden, q_lora, topk = 256, 128, 32
    q_lens, seq_lens = [1, 1, 1], [400, 90, 257]
    common = _common(q_lens, seq_lens)
    t = common.num_actual_tokens
    nblk = int(common.block_table_tensor.max()) + 1
    common.slot_mapping = torch.cat([O.slots_for(common.block_table_tensor, b, s - ql, s)
                                     for b, (ql, s) in enumerate(zip(q_lens, seq_lens))])
    positions = torch.tensor([s - 1 for s in seq_lens])
    raw = torch.zeros(nblk * 128 * 704, dtype=torch.bfloat16, device=dev).view(torch.uint8)
    kv_cache = dsa.NPUDSABackend.reshape_kv_cache(raw, nblk, 128, 1, 704, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(1)
    idx_k = torch.randn(nblk, 128, 128, generator=g).bfloat16()
    k8_ref, ks_ref = O.fp8_quant_token(idx_k.float())
    k8v, ksv = dsa.indexer_cache_views(kv_cache[2])
    k8v.copy_(k8_ref.view(torch.uint8)); ksv.copy_(ks_ref)

    idx = DSV32Indexer(hidden, q_lora, topk, max_tokens=t, device=dev)
    rotary = HIPRotaryEmbedding(max_position=1024, device=dev)
    builder = dsa.NPUDSAMetadataBuilder(V.AttentionSpec(128, 1, 704, torch.bfloat16), ["l"], _cfg(cap=1), dev)
    meta = builder.build(0, _to(common, dev))
    x = torch.randn(t, hidden, generator=g).bfloat16()
    qr = torch.randn(t, q_lora, generator=g).bfloat16()
    cos, sin = O.rope_tables(positions)
    if variant == "positions":
        sel = idx(x.to(dev), qr.to(dev), positions.to(dev), rotary, kv_cache, meta)
        rotate = O.interleave_rope
    else:
        sel, k_out = idx.forward_tables(x.to(dev), qr.to(dev), cos.to(dev).view(-1, 1, 1, 64), sin.to(dev).view(-1, 1, 1, 64),
                                        meta, kv_cache)
        assert k_out.shape == (t, 1, 128)
        rotate = O.rotary_mul
    assert sel.shape == (t, 1, topk) and idx.topk_indices_buffer.data_ptr() == sel.data_ptr()

    # the module's q, k, weights restated on the CPU from its own parameters; selection by the oracle on those
    cpu = lambda m: {k_: v.detach().float().cpu() for k_, v in m.state_dict().items()}
    q = (qr.float() @ cpu(idx.wq_b)["weight"].T).bfloat16().view(t, 64, 128)
    kk = torch.nn.functional.layer_norm((x.float() @ cpu(idx.wk)["weight"].T).bfloat16().float(), (128,),
                                        cpu(idx.k_norm)["weight"], cpu(idx.k_norm)["bias"], 1e-6).bfloat16()
    q = torch.cat([rotate(q[..., :64], cos, sin), q[..., 64:]], -1)
    kk = torch.cat([rotate(kk[:, :64], cos, sin), kk[:, 64:]], -1)
    if variant == "tables":
        assert ((k_out.cpu().view(t, 128).view(torch.int16).int() - kk.view(torch.int16).int()).abs() <= 2).all()
    wts = (x.float() @ cpu(idx.weights_proj)["weight"].T).bfloat16().float()
    sm = common.slot_mapping.cpu()
    # the new key rows in the cache: quantised like the oracle quantises them (GEMM / LayerNorm rounding may move a bf16
    # value by an ulp, so compare the dequantised rows)
    k8_new, ks_new = O.fp8_quant_token(kk.float())
    got = k8v.cpu()[sm // 128, sm % 128].view(torch.float8_e4m3fn).float() * ksv.cpu()[sm // 128, sm % 128].unsqueeze(-1)
    want = k8_new.float() * ks_new.unsqueeze(-1)
    assert (got - want).abs().max().item() <= 0.13 * want.abs().max().item()
    # selection: every position the GPU picked must score (by the oracle, on the cache as the GPU left it) at least as
    # high as the oracle's k-th best, up to the fp8 / bf16 noise of the scores
    q8, qs = O.fp8_quant_token(q.float())
    for b, L in enumerate(seq_lens):
        rows = O.slots_for(common.block_table_tensor.cpu(), b, 0, L)
        k8 = k8v.cpu().view(-1, 128)[rows].view(torch.float8_e4m3fn)
        ks = ksv.cpu().view(-1)[rows]
        sc = O.indexer_scores(q8[b], qs[b], k8, ks, wts[b])
        picked = sel[b, 0].cpu()
        picked = picked[picked >= 0].long()
        assert picked.numel() == min(topk, L) and int(picked.max()) < L and picked.unique().numel() == picked.numel()
        kth = torch.sort(sc, descending=True).values[picked.numel() - 1]
        assert (sc[picked] >= kth - 2e-2 * sc.abs().max()).all()
