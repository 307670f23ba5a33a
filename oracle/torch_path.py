"""The reference's own torch attention applied to the paged path, on the CPU.  TEST INFRASTRUCTURE
ONLY (see ``oracle/paged_ref.py`` for who may import this).

The one attention the reference implements in torch is ``Attention.forward_native`` =
``torch.nn.functional.scaled_dot_product_attention(Q, K, V, is_causal=False)``
(``infer/ops/attention.py:64-71``); its append is ``cache.flat[slot*D:+D] = row``
(``infer/ops/attention.py:16-35``).  Here the paged gather that ``flash_attn`` does internally is
written out (block_table lookup, truncate to the context length, expand KV heads for GQA) and the
result handed to that same SDPA call, bf16 storage with float32 math.  Used (a) as a second,
independently formulated check of ``paged_ref.paged_decode_ref`` and (b) as the CPU baseline that
``bench.py`` times on the host cores.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F


def append_torch(key, value, k_cache, v_cache, slot_mapping) -> None:
    n, hkv, d = key.shape
    width = hkv * d
    valid = slot_mapping >= 0
    rows = slot_mapping[valid].long()
    k_cache.view(-1, width).index_copy_(0, rows, key.reshape(n, width)[valid])
    v_cache.view(-1, width).index_copy_(0, rows, value.reshape(n, width)[valid])


def paged_decode_torch(q, k_cache, v_cache, block_table, context_lens, scale) -> torch.Tensor:
    """``q`` [B, Hq, D] bf16 -> float32 [B, Hq, D]."""
    b, hq, d = q.shape
    _, bs, hkv, _ = k_cache.shape
    g = hq // hkv
    out = torch.zeros((b, hq, d), dtype=torch.float32)
    lens = context_lens.tolist()
    for i in range(b):
        n = lens[i]
        if n <= 0:
            continue
        blocks = block_table[i, : (n + bs - 1) // bs].long()
        k = k_cache[blocks].reshape(-1, hkv, d)[:n].float()      # [L, Hkv, D]
        v = v_cache[blocks].reshape(-1, hkv, d)[:n].float()
        k = k.permute(1, 0, 2).repeat_interleave(g, dim=0)       # [Hq, L, D]
        v = v.permute(1, 0, 2).repeat_interleave(g, dim=0)
        qi = q[i].float().unsqueeze(1)                            # [Hq, 1, D]
        out[i] = F.scaled_dot_product_attention(qi, k, v, is_causal=False, scale=scale)[:, 0]
    return out
