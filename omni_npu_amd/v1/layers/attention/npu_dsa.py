"""The custom-model sparse (DSA) attention module: projections, fused norm + rope + cache write, the indexer, sparse MLA.

Mirrors ``NPUDeepseekSparseAttention.forward(hidden_states, cos, sin)`` of
src/omni_npu/v1/layers/attention/npu_dsa.py:296-586 (prefill :369-443, decode :490-586, attention call :310-355, epilogue
:357-367): the module owns its indexer (``Indexer.forward`` of :105-142, here ``DSV32Indexer.forward_tables``), hands it the
normalised ``q_lora`` and the cos / sin rows, and feeds the indices it returns straight into the sparse attention.  A batch
is all decode or all prefill.  Not here: the MLA-prolog fusion flag and the omni-cache branches of the reference (:395-400,
:445-488, :520-552), which are off by default and tied to components outside this path.

The projections are the caller's modules (callables returning ``(tensor, bias)``); the value up-projection of the
epilogue is fused into the merge of the split-KV partials where W_UV allows it."""
from __future__ import annotations

from typing import Any, Optional

import torch

from .... import _vllm_compat as V
from .... import kernels as K


class NPUDeepseekSparseAttention(torch.nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, qk_nope_head_dim: int, qk_rope_head_dim: int, v_head_dim: int,
                 q_lora_rank: int, kv_lora_rank: int, attn: Any, indexer: Any, q_a_proj, q_a_layernorm, q_b_proj,
                 kv_a_proj_with_mqa, kv_a_layernorm, o_proj, prefix: str = "model.layers.0.self_attn"):
        super().__init__()
        self.hidden_size, self.num_local_heads = hidden_size, num_heads
        self.qk_nope_head_dim, self.qk_rope_head_dim, self.v_head_dim = qk_nope_head_dim, qk_rope_head_dim, v_head_dim
        self.qk_head_dim = qk_nope_head_dim + qk_rope_head_dim
        self.q_lora_rank, self.kv_lora_rank = q_lora_rank, kv_lora_rank
        self.attn, self.indexer, self.prefix = attn, indexer, prefix
        self.q_a_proj, self.q_a_layernorm, self.q_b_proj = q_a_proj, q_a_layernorm, q_b_proj
        self.kv_a_proj_with_mqa, self.kv_a_layernorm, self.o_proj = kv_a_proj_with_mqa, kv_a_layernorm, o_proj
        if not hasattr(kv_a_layernorm, "weight") or self._eps() is None:
            raise TypeError("kv_a_layernorm must expose weight and variance_epsilon (or eps): it runs inside the fused kernel")

    def _eps(self) -> Optional[float]:
        n = self.kv_a_layernorm
        return getattr(n, "variance_epsilon", getattr(n, "eps", None))

    def forward(self, hidden_states: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
        ctx = V.get_forward_context()
        meta = ctx.attn_metadata
        if isinstance(meta, dict):
            meta = meta[getattr(self.attn, "layer_name", f"{self.prefix}.attn")]
        if meta is not None and meta.prefill is not None and meta.decode is not None:
            raise NotImplementedError("NPUDeepseekSparseAttention: a batch is all decode or all prefill on this route "
                                      "(the reference picks one branch for the whole batch, npu_dsa.py:306-309)")
        impl = self.attn.impl
        q_lora = self.q_a_layernorm(self.q_a_proj(hidden_states)[0])
        latent = self.kv_a_proj_with_mqa(hidden_states)[0]
        q = self.q_b_proj(q_lora)[0].view(-1, self.num_local_heads, self.qk_head_dim)
        t, dev = q.shape[0], q.device
        ql_nope = torch.bmm(q[..., :self.qk_nope_head_dim].transpose(0, 1), impl.W_UK_T).transpose(0, 1)
        q_pe = q[..., self.qk_nope_head_dim:]                   # rotated in place by the fused launches below
        out = torch.empty(t, self.num_local_heads * self.v_head_dim, dtype=q.dtype, device=dev)
        if meta is None:
            # memory-profiling run (:401-407, :317-324): norm and rope without a cache, zero attention output
            kv_a = torch.empty(t, self.kv_lora_rank, dtype=q.dtype, device=dev)
            k_pe = torch.empty(t, self.qk_rope_head_dim, dtype=q.dtype, device=dev)
            K.kv_rmsnorm_rope_cache(latent, self.kv_a_layernorm.weight, cos, sin, None, None, None, eps=self._eps(),
                                    kv_a_out=kv_a, k_pe_out=k_pe, q_rope=q_pe)
            return self.o_proj(out.fill_(0))[0]
        kv_cache = self.attn.kv_cache[ctx.virtual_engine]
        assert len(kv_cache) == 3, f"{len(kv_cache)=}."
        K.kv_rmsnorm_rope_cache(latent, self.kv_a_layernorm.weight, cos, sin, meta.slot_mapping, kv_cache[0], kv_cache[1],
                                eps=self._eps(), q_rope=q_pe)
        topk_indices = self.indexer.forward_tables(hidden_states, q_lora, cos, sin, meta, kv_cache)[0]
        if meta.prefill is not None:
            p = meta.prefill
            part, lens, q_len, qsl = p, p.kv_lens, p.max_query_len, p.query_start_loc.to(torch.int32).contiguous()
        else:
            d = meta.decode
            part, lens, q_len, qsl = d, d.seq_lens, d.q_len, d.query_start_loc
        fused = out if impl._fusable_w_uv(out) else None
        select = getattr(self.indexer, "select", self.indexer)
        rc = select.rows_for(meta) if hasattr(select, "rows_for") else None
        attn_out = impl._apply_sparse_attention(ql_nope, q_pe, kv_cache, part, lens, q_len, qsl, topk_indices[:t],
                                                proj_out=fused, rows_counts=None if rc is None else (rc[0][:t], rc[1][:t]))
        if fused is None:
            impl._v_up_proj(attn_out, out=out)
        return self.o_proj(out)[0]
