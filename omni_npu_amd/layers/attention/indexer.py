"""The DeepSeek-V3.2 indexer module: projections, key LayerNorm, rotary embedding of the first 64 dims, then the HIP
selection (fp8 quantisation, key cache write, score GEMM, exact top-k).

Mirrors the patched ``Indexer.__init__`` / ``forward`` of
src/omni_npu/vllm_patches/patches/models/deepseek/patch_dsv32_indexer.py:24-146; the linear layers are plain
``torch.nn.Linear`` (library GEMMs; the reference uses replicated, i.e. unsharded, linears too, :50-67).
``forward_tables`` is the custom-model variant of src/omni_npu/v1/layers/attention/npu_dsa.py:105-142, which gets the
cos / sin rows of its tokens instead of positions and rotates with the half-rotation pairing (``npu_rotary_mul``)."""
from __future__ import annotations

from typing import Optional

import torch

from ... import kernels as K
from ...attention.backends.dsa import LightningIndexer


class DSV32Indexer(torch.nn.Module):
    def __init__(self, hidden_size: int, q_lora_rank: int, index_topk: int, index_n_heads: int = 64,
                 index_head_dim: int = 128, qk_rope_head_dim: int = 64, max_tokens: int = 1,
                 dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        self.topk_tokens, self.n_head, self.head_dim, self.rope_dim = index_topk, index_n_heads, index_head_dim, qk_rope_head_dim
        self.q_lora_rank = q_lora_rank
        self.wq_b = torch.nn.Linear(q_lora_rank, index_head_dim * index_n_heads, bias=False, dtype=dtype, device=device)
        self.wk = torch.nn.Linear(hidden_size, index_head_dim, bias=False, dtype=dtype, device=device)
        self.k_norm = torch.nn.LayerNorm(index_head_dim, eps=1e-6, dtype=dtype, device=device)
        self.weights_proj = torch.nn.Linear(hidden_size, index_n_heads, bias=False, dtype=dtype, device=device)
        self.select = LightningIndexer(index_topk, index_n_heads, index_head_dim, max_tokens=max_tokens, device=device)

    @property
    def topk_indices_buffer(self) -> torch.Tensor:
        return self.select.topk_indices_buffer

    def forward(self, hidden_states: torch.Tensor, qr: torch.Tensor, positions: torch.Tensor, rotary_emb,
                kv_cache=None, attn_metadata=None) -> torch.Tensor:
        q = self.wq_b(qr).view(-1, self.n_head, self.head_dim)
        q_pe, q_nope = torch.split(q, [self.rope_dim, self.head_dim - self.rope_dim], dim=-1)
        k = self.k_norm(self.wk(hidden_states))
        k_pe, k_nope = torch.split(k, [self.rope_dim, self.head_dim - self.rope_dim], dim=-1)
        q_pe, k_pe = rotary_emb(positions, q_pe, k_pe.unsqueeze(1))
        q = torch.cat([q_pe, q_nope], dim=-1)
        k = torch.cat([k_pe.squeeze(1), k_nope], dim=-1)
        weights = self.weights_proj(hidden_states)
        return self.select(q, k, weights, kv_cache, attn_metadata)

    def forward_tables(self, hidden_states: torch.Tensor, qr: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                       attn_metadata=None, kv_cache=None):
        """Argument order and return value of npu_dsa.py:105-142: (top-k indices, the rotated index key [T, 1, 128]).
        The rope dims sit in front of the others in q and k already, so the rotation runs in place on strided views and
        no concatenation is needed."""
        q = self.wq_b(qr).view(-1, self.n_head, self.head_dim)
        k = self.k_norm(self.wk(hidden_states)).unsqueeze(1)
        K.rotary_mul(q[..., :self.rope_dim], cos, sin, out=q[..., :self.rope_dim])
        K.rotary_mul(k[..., :self.rope_dim], cos, sin, out=k[..., :self.rope_dim])
        weights = self.weights_proj(hidden_states)
        return self.select(q, k.squeeze(1), weights, kv_cache, attn_metadata), k
