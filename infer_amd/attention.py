"""``Attention`` module with the interface of ``infer/ops/attention.py:47-122``.

``forward(Q, K, V)`` appends the new K/V rows to the layer's paged cache at
``context.slot_mapping`` and then attends: decode steps run the paged decode kernel, prefill steps
the varlen causal kernel (over the paged cache when ``context.block_tables`` is set, i.e. when a
prefix was already cached).  ``k_cache`` / ``v_cache`` are assigned by the runner
(``infer/engine/model_runner.py:58-64``) and start empty, in which case the append is skipped
exactly as in the reference (``attention.py:108``)."""
from __future__ import annotations

import torch

from . import ops
from .context import get_context


class Attention(torch.nn.Module):

    def __init__(self, num_heads: int, head_dim: int, scale: float, num_kv_heads: int):
        super().__init__()
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.scale = scale
        # one layer's view of the paged caches, [blocks, block_size, num_kv_heads, head_dim]; the runner
        # replaces the empty placeholders once the pool is sized
        self.k_cache = self.v_cache = torch.tensor([])

    def has_cache(self) -> bool:
        return self.k_cache.numel() > 0 and self.v_cache.numel() > 0

    def forward(self, Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, kv_stored: bool = False) -> torch.Tensor:
        """``Q`` [tokens, num_heads * head_dim], ``K``/``V`` [tokens, num_kv_heads * head_dim] of the step's
        new tokens.  ``kv_stored`` says that the caller has already written ``K``/``V`` to the caches (the
        fused norm + rotary + append kernel does), so the append of ``attention.py:108-109`` is skipped."""
        meta = get_context()
        q = Q.view(-1, self.num_heads, self.head_dim)
        k_new = K.view(-1, self.num_kv_heads, self.head_dim)
        v_new = V.view(-1, self.num_kv_heads, self.head_dim)
        if self.has_cache() and not kv_stored:
            ops.store_kvcache(k_new, v_new, self.k_cache, self.v_cache, meta.slot_mapping)
        out = self._prefill(q, k_new, v_new, meta) if meta.is_prefill else self._decode(q, meta)
        return out.view(-1, self.num_heads * self.head_dim)

    def _prefill(self, q, k_new, v_new, meta) -> torch.Tensor:
        # with a block table some prefix is already cached, and every key (cached and new, the new ones were
        # appended above) is read from the paged cache; without one the keys are the packed new rows
        paged = meta.block_tables is not None
        keys, values = (self.k_cache, self.v_cache) if paged else (k_new, v_new)
        return ops.flash_attn_varlen_func(
            q, keys, values, cu_seqlens_q=meta.cu_seqlens_q, cu_seqlens_k=meta.cu_seqlens_k,
            max_seqlen_q=meta.max_seqlen_q, max_seqlen_k=meta.max_seqlen_k, softmax_scale=self.scale,
            causal=True, block_table=meta.block_tables)

    def _decode(self, q, meta) -> torch.Tensor:
        # one query token per sequence: [batch, 1, heads, head_dim]
        return ops.flash_attn_with_kvcache(
            q.unsqueeze(1), self.k_cache, self.v_cache, cache_seqlens=meta.context_lens,
            block_table=meta.block_tables, softmax_scale=self.scale, causal=True)
