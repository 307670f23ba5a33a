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
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])

    def forward(self, Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, kv_stored: bool = False) -> torch.Tensor:
        """``kv_stored`` says that the caller has already written ``K``/``V`` to the caches (the fused
        norm + rotary + append kernel does), so the append of ``attention.py:108-109`` is skipped."""
        Q = Q.view(-1, self.num_heads, self.head_dim)
        K = K.view(-1, self.num_kv_heads, self.head_dim)
        V = V.view(-1, self.num_kv_heads, self.head_dim)
        context = get_context()
        k_cache, v_cache = self.k_cache, self.v_cache
        if k_cache.numel() and v_cache.numel() and not kv_stored:
            ops.store_kvcache(K, V, k_cache, v_cache, context.slot_mapping)
        if context.is_prefill:
            if context.block_tables is not None:   # prefix cache: keys come from the paged cache
                K, V = k_cache, v_cache
            O = ops.flash_attn_varlen_func(Q, K, V,
                                           max_seqlen_q=context.max_seqlen_q, cu_seqlens_q=context.cu_seqlens_q,
                                           max_seqlen_k=context.max_seqlen_k, cu_seqlens_k=context.cu_seqlens_k,
                                           softmax_scale=self.scale, causal=True, block_table=context.block_tables)
        else:
            O = ops.flash_attn_with_kvcache(Q.unsqueeze(1), k_cache, v_cache,
                                            cache_seqlens=context.context_lens, block_table=context.block_tables,
                                            softmax_scale=self.scale, causal=True)
        return O.view(-1, self.num_heads * self.head_dim)
