"""The custom-model MLA attention module: the second caller of the kernels, which does not go through ``Impl.forward``.

Mirrors ``NPUDeepseekMLAAttention.forward(hidden_states, cos, sin)`` of
src/omni_npu/v1/layers/attention/npu_mla.py:152-348: the model hands the layer the cos / sin rows of its tokens; a batch is
either all decode (:169-242) or all prefill without cached context (:244-348, the route the reference serves with chunked
prefill disabled).  The projection modules are the caller's (callables returning ``(tensor, bias)`` like vLLM's linear
layers: library GEMMs, as in the reference).  On this side of the boundary:

* decode: RMSNorm + rotary embedding + cache write (``npu_kv_rmsnorm_rope_cache``, :196-206) and the query's rotary
  embedding (``npu_interleave_rope``, :210) are one launch, the attention call (:213-232) is the split-KV kernel, and the
  ``W_UV`` product (:235-240) is fused into the merge of its partials;
* prefill: the same fused launch also returns the normalised latent and the rotated key (``is_output_kv``, :296-309), the
  varlen kernel runs causally over the step's own tokens (:329-344).

The reference overlaps the kv projections with the q projections on a second stream (:280-323); here everything stays on
the current stream: the GEMMs on either side are matrix-pipe work at the part's power limit and gain nothing side by side.
"""
from __future__ import annotations

from typing import Any, Optional

import torch

from .... import _vllm_compat as V
from .... import kernels as K


class NPUDeepseekMLAAttention(torch.nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, qk_nope_head_dim: int, qk_rope_head_dim: int, v_head_dim: int,
                 q_lora_rank: int, kv_lora_rank: int, attn: Any, q_a_proj, q_a_layernorm, q_b_proj, kv_a_proj_with_mqa,
                 kv_a_layernorm, o_proj, prefix: str = "model.layers.0.self_attn"):
        super().__init__()
        self.hidden_size, self.num_local_heads = hidden_size, num_heads
        self.qk_nope_head_dim, self.qk_rope_head_dim, self.v_head_dim = qk_nope_head_dim, qk_rope_head_dim, v_head_dim
        self.qk_head_dim = qk_nope_head_dim + qk_rope_head_dim
        self.q_lora_rank, self.kv_lora_rank = q_lora_rank, kv_lora_rank
        self.attn, self.prefix = attn, prefix
        self.q_a_proj, self.q_a_layernorm, self.q_b_proj = q_a_proj, q_a_layernorm, q_b_proj
        self.kv_a_proj_with_mqa, self.kv_a_layernorm, self.o_proj = kv_a_proj_with_mqa, kv_a_layernorm, o_proj
        if not hasattr(kv_a_layernorm, "weight") or self._eps() is None:
            raise TypeError("kv_a_layernorm must expose weight and variance_epsilon (or eps): it runs inside the fused kernel")

    def _eps(self) -> Optional[float]:
        n = self.kv_a_layernorm
        return getattr(n, "variance_epsilon", getattr(n, "eps", None))

    def _metadata(self):
        ctx = V.get_forward_context()
        meta = ctx.attn_metadata
        if isinstance(meta, dict):
            meta = meta[getattr(self.attn, "layer_name", f"{self.prefix}.attn")]
        return ctx, meta

    def forward(self, hidden_states: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
        ctx, meta = self._metadata()
        if meta is None or meta.prefill is not None:
            if meta is not None and meta.decode is not None:
                raise NotImplementedError("NPUDeepseekMLAAttention: a batch is all decode or all prefill on this route "
                                          "(the reference picks one branch for the whole batch, npu_mla.py:164-167)")
            return self._forward_prefill(hidden_states, cos, sin, ctx, meta)
        return self._forward_decode(hidden_states, cos, sin, ctx, meta)

    def _caches(self, ctx):
        kv_cache = self.attn.kv_cache[ctx.virtual_engine]
        fp8 = bool(getattr(self.attn.impl, "fp8_cache", False))
        return kv_cache, kv_cache[0], (None if fp8 else kv_cache[1])

    def _q(self, hidden_states: torch.Tensor) -> torch.Tensor:
        q_lora = self.q_a_proj(hidden_states)[0]
        return self.q_b_proj(self.q_a_layernorm(q_lora))[0].view(-1, self.num_local_heads, self.qk_head_dim)

    def _forward_decode(self, hidden_states, cos, sin, ctx, meta) -> torch.Tensor:
        impl = self.attn.impl
        kv_cache, nope_c, rope_c = self._caches(ctx)
        q = self._q(hidden_states)
        kv = self.kv_a_proj_with_mqa(hidden_states)[0]
        t = q.shape[0]
        # (N, T, P) @ W_UK_T (N, P, L) -> token-major [T, N, L]
        ql_nope = torch.bmm(q[..., :self.qk_nope_head_dim].transpose(0, 1), impl.W_UK_T).transpose(0, 1)
        q_pe = q[..., self.qk_nope_head_dim:]                   # rotated in place by the launch that writes the cache
        K.kv_rmsnorm_rope_cache(kv, self.kv_a_layernorm.weight, cos, sin, meta.slot_mapping, nope_c, rope_c, eps=self._eps(),
                                q_rope=q_pe)
        out = torch.empty(t, self.num_local_heads * self.v_head_dim, dtype=q.dtype, device=q.device)
        impl._forward_decode(ql_nope, q_pe, kv_cache, meta, proj_out=out)
        return self.o_proj(out)[0]

    def _forward_prefill(self, hidden_states, cos, sin, ctx, meta) -> torch.Tensor:
        impl = self.attn.impl
        q = self._q(hidden_states)
        kv = self.kv_a_proj_with_mqa(hidden_states)[0]
        t, dev = q.shape[0], q.device
        kv_a = torch.empty(t, self.kv_lora_rank, dtype=q.dtype, device=dev)
        k_pe = torch.empty(t, self.qk_rope_head_dim, dtype=q.dtype, device=dev)
        attn_output = torch.empty(t, self.num_local_heads, self.v_head_dim, dtype=q.dtype, device=dev)
        if meta is None:                                     # memory-profiling run: same projections, no attention, no cache
            K.kv_rmsnorm_rope_cache(kv, self.kv_a_layernorm.weight, cos, sin, None, None, None, eps=self._eps(),
                                    kv_a_out=kv_a, k_pe_out=k_pe)
            attn_output.fill_(0)
            return self.o_proj(attn_output.view(t, -1))[0]
        _, nope_c, rope_c = self._caches(ctx)
        q_pe = q[..., self.qk_nope_head_dim:]
        K.kv_rmsnorm_rope_cache(kv, self.kv_a_layernorm.weight, cos, sin, meta.slot_mapping, nope_c, rope_c,
                                eps=self._eps(), kv_a_out=kv_a, k_pe_out=k_pe, q_rope=q_pe)
        k_nope, v = impl._kv_up(kv_a, allow_fp16=True)
        cu = meta.prefill.query_start_loc.to(torch.int32).contiguous()
        K.prefill_varlen(q[..., :self.qk_nope_head_dim], q_pe, k_nope, k_pe.to(k_nope.dtype), v, cu, cu,
                         meta.prefill.max_query_len, impl.scale, True, attn_output)
        return self.o_proj(attn_output.view(t, -1))[0]
