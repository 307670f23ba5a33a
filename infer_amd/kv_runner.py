"""Host side of a step: cache sizing and the per-step metadata the kernels consume.

Mirrors the parts of ``infer/engine/model_runner.py`` that sit on the KV-cache path:
``allocate_kv_cache`` (``:47-64``), ``prepare_block_tables`` (``:66-70``), ``prepare_prefill``
(``:72-108``) and ``prepare_decode`` (``:110-126``).  Metadata is built in host lists, staged in
pinned tensors and copied asynchronously, as the reference does."""
from __future__ import annotations

import torch

from .context import set_context
from .sequence import Sequence


def kv_block_bytes(num_layers: int, block_size: int, num_kv_heads: int, head_dim: int, itemsize: int = 2) -> int:
    """Bytes of one pool block across all layers, K and V (``model_runner.py:54``)."""
    return 2 * num_layers * block_size * num_kv_heads * head_dim * itemsize


def num_kvcache_blocks(total: int, used: int, peak: int, current: int, utilization: float, block_bytes: int) -> int:
    """Pool size from the memory numbers the reference reads (``model_runner.py:50-55``)."""
    return int(total * utilization - used - peak + current) // block_bytes


def allocate_kv_cache(num_blocks: int, num_layers: int, block_size: int, num_kv_heads: int, head_dim: int,
                      device, dtype=torch.bfloat16) -> torch.Tensor:
    """One zeroed tensor ``[2, layers, nblk, bs, Hkv, D]``; layer ``l`` uses ``kv[0, l]`` and ``kv[1, l]``."""
    assert num_blocks > 0
    return torch.zeros(2, num_layers, num_blocks, block_size, num_kv_heads, head_dim, dtype=dtype, device=device)


def bind_kv_cache(model: torch.nn.Module, kv_cache: torch.Tensor) -> int:
    """Hands every module that has ``k_cache``/``v_cache`` its layer view (``model_runner.py:59-64``)."""
    layer_id = 0
    for module in model.modules():
        if hasattr(module, "k_cache") and hasattr(module, "v_cache"):
            module.k_cache = kv_cache[0, layer_id]
            module.v_cache = kv_cache[1, layer_id]
            layer_id += 1
    return layer_id


def _to_device(values, dtype, device):
    t = torch.tensor(values, dtype=dtype, pin_memory=torch.device(device).type == "cuda")
    return t.to(device, non_blocking=True)


def prepare_block_tables(seqs: list[Sequence], device="cuda") -> torch.Tensor:
    max_len = max(len(seq.block_table) for seq in seqs)
    rows = [seq.block_table + [-1] * (max_len - len(seq.block_table)) for seq in seqs]
    return _to_device(rows, torch.int32, device)


def prepare_prefill(seqs: list[Sequence], device="cuda"):
    block_size = Sequence.block_size
    input_ids, positions, slot_mapping = [], [], []
    cu_seqlens_q, cu_seqlens_k = [0], [0]
    max_seqlen_q = max_seqlen_k = 0
    for seq in seqs:
        seqlen = len(seq)
        input_ids.extend(seq[seq.num_cached_tokens:])
        positions.extend(range(seq.num_cached_tokens, seqlen))
        seqlen_q = seqlen - seq.num_cached_tokens
        cu_seqlens_q.append(cu_seqlens_q[-1] + seqlen_q)
        cu_seqlens_k.append(cu_seqlens_k[-1] + seqlen)
        max_seqlen_q = max(max_seqlen_q, seqlen_q)
        max_seqlen_k = max(max_seqlen_k, seqlen)
        if not seq.block_table:
            continue
        for i in range(seq.num_cached_blocks, seq.num_blocks):
            start = seq.block_table[i] * block_size
            fill = block_size if i != seq.num_blocks - 1 else seq.last_block_num_tokens
            slot_mapping.extend(range(start, start + fill))
    block_tables = prepare_block_tables(seqs, device) if cu_seqlens_k[-1] > cu_seqlens_q[-1] else None
    input_ids = _to_device(input_ids, torch.int64, device)
    positions = _to_device(positions, torch.int64, device)
    set_context(True, _to_device(cu_seqlens_q, torch.int32, device), _to_device(cu_seqlens_k, torch.int32, device),
                max_seqlen_q, max_seqlen_k, _to_device(slot_mapping, torch.int32, device), None, block_tables)
    return input_ids, positions


def prepare_decode(seqs: list[Sequence], device="cuda"):
    block_size = Sequence.block_size
    input_ids, positions, slot_mapping, context_lens = [], [], [], []
    for seq in seqs:
        input_ids.append(seq.last_token)
        positions.append(len(seq))
        context_lens.append(len(seq))
        slot_mapping.append(seq.block_table[-1] * block_size + seq.last_block_num_tokens - 1)
    set_context(False, slot_mapping=_to_device(slot_mapping, torch.int32, device),
                context_lens=_to_device(context_lens, torch.int32, device),
                block_tables=prepare_block_tables(seqs, device))
    return _to_device(input_ids, torch.int64, device), _to_device(positions, torch.int64, device)
