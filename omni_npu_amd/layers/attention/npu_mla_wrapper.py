"""The caller of the MLA backends: projections -> norms -> rotary embedding -> (indexer) -> attention -> output projection.

Mirrors ``NPUMultiHeadLatentAttentionWrapper.forward_oot`` (src/omni_npu/layers/attention/npu_mla_wrapper.py:10-80) and the
attention layer it calls (``self.mla_attn``: the kv cache is ``kv_cache[forward_context.virtual_engine]``, the metadata
``forward_context.attn_metadata[layer_name]``, src/omni_npu/v1/layers/attention/npu_mla.py:159-162, 176).  The projection
modules are the caller's (any callable returning ``(tensor, bias)`` like vLLM's linear layers: library GEMMs, as in the
reference); what this file adds on the GPU side is that the RMSNorm of the compressed KV, the rotary embedding of the
shared rope key and the write of both into the paged cache run as ONE kernel when the norm and the rotary module expose
their parameters (the backend impl is told, through ``cache_written_for``, that the rows of this step are in place)."""
from __future__ import annotations

from typing import Any, Optional

import torch

from ... import _vllm_compat as V
from ... import kernels as K
from ..rotary_embedding import HIPRotaryEmbedding


class MLAAttention(torch.nn.Module):
    """Stand-in for vLLM's attention layer object: owns the backend impl and the per-engine kv caches, allocates the output
    and calls ``impl.forward(layer, q, kv_c_normed, k_pe, kv_cache, attn_metadata, output=...)``."""

    def __init__(self, impl: Any, layer_name: str = "model.layers.0.self_attn.attn"):
        super().__init__()
        self.impl, self.layer_name = impl, layer_name
        self.kv_cache: list = [None]

    def forward(self, q: torch.Tensor, kv_c_normed: torch.Tensor, k_pe: torch.Tensor, output_shape=None) -> torch.Tensor:
        ctx = V.get_forward_context()
        meta = ctx.attn_metadata
        if isinstance(meta, dict):
            meta = meta[self.layer_name]
        shape = output_shape if output_shape is not None else (q.shape[0], self.impl.num_heads * self.impl.v_head_dim)
        out = torch.zeros(shape, dtype=q.dtype, device=q.device)
        return self.impl.forward(self, q, kv_c_normed, k_pe, self.kv_cache[ctx.virtual_engine], meta, output=out)


class NPUMultiHeadLatentAttentionWrapper(torch.nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, qk_nope_head_dim: int, qk_rope_head_dim: int, v_head_dim: int,
                 q_lora_rank: Optional[int], kv_lora_rank: int, mla_attn: MLAAttention, kv_a_layernorm, o_proj,
                 rotary_emb=None, fused_qkv_a_proj=None, q_a_layernorm=None, q_b_proj=None, kv_a_proj_with_mqa=None,
                 q_proj=None, indexer=None, is_sparse: bool = False, indexer_rope_emb=None):
        super().__init__()
        self.hidden_size, self.num_heads = hidden_size, num_heads
        self.qk_nope_head_dim, self.qk_rope_head_dim, self.v_head_dim = qk_nope_head_dim, qk_rope_head_dim, v_head_dim
        self.qk_head_dim = qk_nope_head_dim + qk_rope_head_dim
        self.q_lora_rank, self.kv_lora_rank = q_lora_rank, kv_lora_rank
        self.mla_attn, self.kv_a_layernorm, self.o_proj, self.rotary_emb = mla_attn, kv_a_layernorm, o_proj, rotary_emb
        self.fused_qkv_a_proj, self.q_a_layernorm, self.q_b_proj = fused_qkv_a_proj, q_a_layernorm, q_b_proj
        self.kv_a_proj_with_mqa, self.q_proj = kv_a_proj_with_mqa, q_proj
        self.indexer, self.is_sparse, self.indexer_rope_emb = indexer, is_sparse, indexer_rope_emb

    def _kv_norm_rope(self, positions: torch.Tensor, kv_lora: torch.Tensor, q: Optional[torch.Tensor] = None):
        """kv_a_layernorm(kv_c) and rotary(k_pe): one fused launch when possible (which then also rotates the rope part
        of ``q`` in place and writes the cache rows), the two modules otherwise."""
        norm, rope = self.kv_a_layernorm, self.rotary_emb
        eps = getattr(norm, "variance_epsilon", getattr(norm, "eps", None))
        if isinstance(rope, HIPRotaryEmbedding) and hasattr(norm, "weight") and eps is not None and kv_lora.is_cuda \
                and kv_lora.dtype == torch.bfloat16 and kv_lora.shape[-1] == K.D_NOPE + K.D_ROPE:
            t = kv_lora.shape[0]
            cos, sin = rope.get_cos_sin(positions)
            kv_c_normed = torch.zeros(t, K.D_NOPE, dtype=kv_lora.dtype, device=kv_lora.device)
            k_pe = torch.zeros(t, K.D_ROPE, dtype=kv_lora.dtype, device=kv_lora.device)
            impl, meta, slots, nope_c, rope_c = self._cache_target()
            q_rope = None
            if q is not None and q.dtype == torch.bfloat16 and q.stride(-1) == 1 and q.shape[0] == t:
                q_rope = q[..., self.qk_nope_head_dim:]
            if impl is not None:
                impl.cache_written_for = None                  # a launch that raises must leave no mark behind
            K.kv_rmsnorm_rope_cache(kv_lora, norm.weight, cos, sin, slots, nope_c, rope_c, eps=eps, kv_a_out=kv_c_normed,
                                    k_pe_out=k_pe, q_rope=q_rope)
            if impl is not None and slots is not None:
                # the rows of this step are in place: the impl skips its own write for this metadata object, provided
                # the launch covered every token it would have written
                impl.cache_written_for = (meta, min(int(slots.numel()), t))
            return kv_c_normed, k_pe.unsqueeze(1), (cos, sin, q_rope is not None)
        kv_c, k_pe = kv_lora.split([self.kv_lora_rank, self.qk_rope_head_dim], dim=-1)
        return norm(kv_c), k_pe.unsqueeze(1), None

    def _cache_target(self):
        """Where the fused launch may also write the new tokens' cache rows: (impl, metadata, slot_mapping, latent cache,
        rope cache or None for the fp8 cache) when the step has metadata, the layer a cache, every token a slot, and the
        backend impl can skip its own write for a marked metadata object; five times None otherwise.  The mark itself
        is set by the caller once the launch has been issued."""
        none = (None, None, None, None, None)
        impl = getattr(self.mla_attn, "impl", None)
        if impl is None or not hasattr(impl, "cache_written_for"):
            return none
        ctx = V.get_forward_context()
        meta = ctx.attn_metadata
        if isinstance(meta, dict):
            meta = meta.get(self.mla_attn.layer_name)
        kv_cache = self.mla_attn.kv_cache[ctx.virtual_engine]
        if meta is None or kv_cache is None or getattr(meta, "slot_mapping", None) is None:
            return none
        if meta.slot_mapping.numel() < meta.num_actual_tokens:
            return none
        if getattr(impl, "fp8_cache", False):
            return impl, meta, meta.slot_mapping, kv_cache[0], None
        return impl, meta, meta.slot_mapping, kv_cache[0], kv_cache[1]

    def forward_oot(self, positions: torch.Tensor, hidden_states: torch.Tensor,
                    llama_4_scaling: Optional[torch.Tensor] = None) -> torch.Tensor:
        q_c = None
        if self.q_lora_rank is not None:
            assert self.fused_qkv_a_proj is not None, "fused_qkv_a_proj is required when q_lora_rank is not None"
            assert self.q_a_layernorm is not None, "q_a_layernorm is required when q_lora_rank is not None"
            assert self.q_b_proj is not None, "q_b_proj is required when q_lora_rank is not None"
            qkv_lora = self.fused_qkv_a_proj(hidden_states)[0]
            q_c, kv_lora = qkv_lora.split([self.q_lora_rank, self.kv_lora_rank + self.qk_rope_head_dim], dim=-1)
            q_c = self.q_a_layernorm(q_c)
            q = self.q_b_proj(q_c)[0]
        else:
            assert self.kv_a_proj_with_mqa is not None, "kv_a_proj_with_mqa is required when q_lora_rank is None"
            assert self.q_proj is not None, "q_proj is required when q_lora_rank is None"
            kv_lora = self.kv_a_proj_with_mqa(hidden_states)[0]
            q = self.q_proj(hidden_states)[0]

        q = q.view(-1, self.num_heads, self.qk_head_dim)
        kv_c_normed, k_pe, cos_sin = self._kv_norm_rope(positions, kv_lora, q if self.rotary_emb is not None else None)
        if self.rotary_emb is not None:
            if cos_sin is not None:                            # k_pe is rotated already, and q too unless it did not qualify
                if not cos_sin[2]:
                    K.interleave_rope(q[..., self.qk_nope_head_dim:], cos_sin[0], cos_sin[1],
                                      out=q[..., self.qk_nope_head_dim:], table="half")
            else:
                q[..., self.qk_nope_head_dim:], k_pe = self.rotary_emb(positions, q[..., self.qk_nope_head_dim:], k_pe)

        if self.indexer and self.is_sparse:
            ctx = V.get_forward_context()
            attn_metadata = ctx.attn_metadata
            if isinstance(attn_metadata, dict):
                attn_metadata = attn_metadata[self.mla_attn.layer_name]
            self_kv_cache = self.mla_attn.kv_cache[ctx.virtual_engine]
            self.indexer(hidden_states, q_c, positions, self.indexer_rope_emb, self_kv_cache, attn_metadata)

        if llama_4_scaling is not None:
            q *= llama_4_scaling

        attn_out = self.mla_attn(q, kv_c_normed, k_pe,
                                 output_shape=(hidden_states.shape[0], self.num_heads * self.v_head_dim))
        return self.o_proj(attn_out)[0]

    forward = forward_oot
