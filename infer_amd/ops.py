"""Python entry points of the paged KV-cache path, argument-compatible with the reference.

* ``store_kvcache``            - same signature and asserts as ``infer/ops/attention.py:38-45``.
* ``flash_attn_with_kvcache``  - keyword set used at ``infer/ops/attention.py:118-120``.
* ``flash_attn_decode``        - the signature the stub ``src/operators/flashattn/flashattn_decode.cu:11-12``
  intended: ``(Q, K, V, is_causal, block_table, O)`` with an out-parameter, plus the context lengths
  it forgot.

All of them launch hand-written HIP kernels through the C ABI of ``libinfer_kv.so`` on torch's
current stream.  Tensors must live on the GPU; there is no CPU path.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib

_workspaces: dict = {}
_retired_workspaces: list = []      # outgrown workspaces stay alive: captured graphs may still point at them


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(*tensors):
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("infer_amd ops need GPU tensors: the HIP kernels are the only implementation")


def store_kvcache(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  slot_mapping: torch.Tensor) -> None:
    """Scatter ``key``/``value`` rows ``[N, Hkv, D]`` into the paged caches at ``slot_mapping``.

    Rows with a negative slot are skipped.  Bit-exact copy."""
    n, num_heads, head_dim = key.shape
    d = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == d and v_cache.stride(1) == d
    assert slot_mapping.numel() == n
    assert key.dtype == torch.bfloat16 and value.dtype == torch.bfloat16
    assert k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
    assert slot_mapping.dtype == torch.int32 and slot_mapping.is_contiguous()
    assert value.shape == key.shape
    _require_gpu(key, value, k_cache, v_cache, slot_mapping)
    assert k_cache.stride(0) == k_cache.shape[1] * d and v_cache.stride(0) == v_cache.shape[1] * d
    if n == 0:
        return
    num_slots = k_cache.shape[0] * k_cache.shape[1]
    lib = _lib.load()
    rc = lib.infer_kv_append_bf16(key.data_ptr(), key.stride(0), value.data_ptr(), value.stride(0),
                                  k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(),
                                  n, d, num_slots, _stream_ptr(key))
    _lib.check(rc, "store_kvcache")


def gather_kvcache(cache: torch.Tensor, block_table_row: torch.Tensor, length: int) -> torch.Tensor:
    """The first ``length`` tokens of one sequence as a dense ``[length, Hkv, D]`` tensor, gathered from the
    paged ``cache`` ``[nblk, bs, Hkv, D]`` through the sequence's block-table row (int32, on the device): the
    per-sequence tensor the getters of the reference's cache pool hand out (``include/kvcache.hpp:47-48``)."""
    assert cache.dim() == 4 and cache.dtype == torch.bfloat16 and cache.is_contiguous()
    nblk, bs, hkv, d = cache.shape
    assert block_table_row.dtype == torch.int32 and block_table_row.dim() == 1 and block_table_row.is_contiguous()
    assert 0 <= length <= block_table_row.numel() * bs
    _require_gpu(cache, block_table_row)
    out = torch.empty((length, hkv, d), dtype=cache.dtype, device=cache.device)
    rc = _lib.load().infer_kv_gather_bf16(cache.data_ptr(), block_table_row.data_ptr(), length, hkv * d, bs, nblk,
                                          out.data_ptr(), _stream_ptr(cache))
    _lib.check(rc, "gather_kvcache")
    return out


def qk_norm_rope_store_kvcache(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, positions: torch.Tensor,
                               q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor, eps: float,
                               cos_sin_cache: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                               slot_mapping: torch.Tensor, write_key: bool = True) -> None:
    """One launch for ``q_norm``, ``k_norm``, the in-place neox rotary embedding and ``store_kvcache``
    (the sequence at ``infer/models/Qwen3.py:113-131``).  ``q`` ``[N, Hq, D]`` and ``k`` ``[N, Hkv, D]``
    are updated in place (``k`` only if ``write_key``), the rotated ``k`` and ``v`` land in the caches
    at ``slot_mapping``; rows with a negative slot skip the caches."""
    n, hq, d = q.shape
    hkv = k.shape[1]
    assert k.shape == (n, hkv, d) and v.shape == (n, hkv, d)
    for t in (q, k, v, q_norm_weight, k_norm_weight, cos_sin_cache, k_cache, v_cache):
        assert t.dtype == torch.bfloat16
    for t in (q, k, v):
        assert t.stride(2) == 1 and t.stride(1) == d
    assert q_norm_weight.shape == (d,) and k_norm_weight.shape == (d,)
    assert q_norm_weight.is_contiguous() and k_norm_weight.is_contiguous()
    assert cos_sin_cache.dim() == 2 and cos_sin_cache.shape[1] == d and cos_sin_cache.is_contiguous()
    assert positions.dtype == torch.int64 and positions.numel() == n and positions.is_contiguous()
    assert slot_mapping.dtype == torch.int32 and slot_mapping.numel() == n and slot_mapping.is_contiguous()
    assert k_cache.stride(1) == hkv * d and v_cache.stride(1) == hkv * d
    assert k_cache.stride(0) == k_cache.shape[1] * hkv * d and v_cache.stride(0) == v_cache.shape[1] * hkv * d
    _require_gpu(q, k, v, positions, q_norm_weight, k_norm_weight, cos_sin_cache, k_cache, v_cache, slot_mapping)
    if n == 0:
        return
    rc = _lib.load().infer_kv_qk_norm_rope_append_bf16(
        q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), positions.data_ptr(),
        q_norm_weight.data_ptr(), k_norm_weight.data_ptr(), float(eps), cos_sin_cache.data_ptr(),
        cos_sin_cache.shape[0], k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(), n, hq, hkv, d,
        k_cache.shape[0] * k_cache.shape[1], int(bool(write_key)), _stream_ptr(q))
    _lib.check(rc, "qk_norm_rope_store_kvcache")


def decode_workspace(device, max_batch: int, num_q_heads: int, num_kv_heads: int, head_dim: int) -> torch.Tensor:
    """Workspace for the split-KV partial results, cached per (device, shape): allocated once so that
    steady-state decode steps (and HIP graph replays) never allocate."""
    key = (str(device), num_q_heads, num_kv_heads, head_dim)
    ws = _workspaces.get(key)
    if ws is None or ws[0] < max_batch:
        cap = max(max_batch, 64 if ws is None else 2 * ws[0])
        with torch.cuda.device(device):      # the library's per-device set-up, before any graph capture
            _lib.check(_lib.load().infer_kv_init(), "infer_kv_init")
        nbytes = _lib.load().infer_paged_decode_workspace_bytes(cap, num_q_heads, num_kv_heads, head_dim)
        if nbytes == 0:
            raise RuntimeError("paged decode: unsupported shape "
                               f"(Hq={num_q_heads}, Hkv={num_kv_heads}, D={head_dim})")
        if ws is not None:
            _retired_workspaces.append(ws[1])
        ws = (cap, torch.empty(nbytes, dtype=torch.uint8, device=device))
        _workspaces[key] = ws
    return ws[1]


_workspace_streams: dict = {}      # data_ptr of a shared workspace -> the stream that used it last


def _claim_shared_workspace(workspace: torch.Tensor, device) -> None:
    """The shared workspace holds the partial results of a call until its merge kernel has run, so calls
    that use it must be ordered on one stream.  A call on another stream while the last one still has work
    pending is refused (a host-side check on a change of stream only; streams under capture are not
    queried): pass ``workspace=`` of its own to such a call."""
    cur = torch.cuda.current_stream(device)
    last = _workspace_streams.get(workspace.data_ptr())
    if last is not None and last != cur and not torch.cuda.is_current_stream_capturing() and not last.query():
        raise RuntimeError("paged decode: the shared workspace is still in use on another stream; "
                           "order the calls on one stream or pass a workspace of their own")
    _workspace_streams[workspace.data_ptr()] = cur


def _decode_args(q3, k_cache, v_cache, cache_seqlens, block_table):
    assert q3.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16
    uniform = isinstance(cache_seqlens, int)      # one length for the whole batch, known on the host
    assert block_table.dtype == torch.int32 and (uniform or cache_seqlens.dtype == torch.int32)
    assert k_cache.dim() == 4 and k_cache.shape == v_cache.shape
    assert k_cache.stride() == v_cache.stride()
    b, hq, d = q3.shape
    nblk, bs, hkv, dk = k_cache.shape
    assert dk == d and q3.stride(2) == 1 and q3.stride(1) == d
    assert k_cache.stride(3) == 1 and k_cache.stride(2) == d
    assert cache_seqlens >= 0 if uniform else (cache_seqlens.numel() == b and cache_seqlens.is_contiguous())
    assert block_table.dim() == 2 and block_table.shape[0] == b and block_table.shape[1] >= 1
    assert block_table.stride(1) == 1
    _require_gpu(q3, k_cache, v_cache, block_table, *(() if uniform else (cache_seqlens,)))
    return b, hq, d, nblk, bs, hkv


def paged_attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      context_lens: torch.Tensor, scale: float, out: torch.Tensor, workspace=None,
                      split_workgroups: int = 0) -> None:
    """Out-parameter form: ``q``/``out`` are ``[B, Hq, D]``.  ``split_workgroups`` = workgroups along
    the KV-split axis of this call (0: the library's choice for the device).  The default workspace is
    shared by every call for the shape on the device, so such calls must be ordered on one stream;
    pass a ``workspace`` of its own to a call that runs on another stream.

    ``context_lens`` is the int32 tensor of the reference's call, or a Python int when every sequence
    of the batch has that many tokens (``cache_seqlens: int`` of ``flash_attn_with_kvcache``): the
    library then plans the launch on the host and, for batches that fill the chip, runs one kernel
    without a merge launch (``split_workgroups`` does not apply)."""
    b, hq, d, nblk, bs, hkv = _decode_args(q, k_cache, v_cache, context_lens, block_table)
    assert out.shape == q.shape and out.dtype == torch.bfloat16 and out.stride(2) == 1 and out.stride(1) == d
    if workspace is None:
        workspace = decode_workspace(q.device, b, hq, hkv, d)
        _claim_shared_workspace(workspace, q.device)
    lib = _lib.load()
    if isinstance(context_lens, int):
        rc = lib.infer_paged_decode_uniform_bf16(
            q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1),
            out.data_ptr(), out.stride(0), block_table.data_ptr(), block_table.stride(0), block_table.shape[1],
            context_lens, b, hq, hkv, d, bs, nblk, float(scale), workspace.data_ptr(), workspace.numel(),
            _stream_ptr(q))
        _lib.check(rc, "paged_attn_decode")
        return
    rc = lib.infer_paged_decode_bf16(
        q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1),
        out.data_ptr(), out.stride(0), block_table.data_ptr(), block_table.stride(0), block_table.shape[1],
        context_lens.data_ptr(), b, hq, hkv, d, bs, nblk, float(scale), int(split_workgroups),
        workspace.data_ptr(), workspace.numel(), _stream_ptr(q))
    _lib.check(rc, "paged_attn_decode")


def paged_attn_decode_split(q, k_cache, v_cache, block_table, context_lens, scale, workspace,
                            split_workgroups: int = 0) -> None:
    """Bandwidth-bound phase alone (partials stay in ``workspace``); for profiling."""
    assert isinstance(context_lens, torch.Tensor), "the split phase takes the lengths as a tensor"
    b, hq, d, nblk, bs, hkv = _decode_args(q, k_cache, v_cache, context_lens, block_table)
    rc = _lib.load().infer_paged_decode_split_bf16(
        q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), k_cache.stride(0), k_cache.stride(1),
        block_table.data_ptr(), block_table.stride(0), block_table.shape[1], context_lens.data_ptr(),
        b, hq, hkv, d, bs, nblk, float(scale), int(split_workgroups), workspace.data_ptr(), workspace.numel(),
        _stream_ptr(q))
    _lib.check(rc, "paged_attn_decode_split")


def paged_attn_decode_merge(out, context_lens, num_kv_heads, workspace) -> None:
    b, hq, d = out.shape
    rc = _lib.load().infer_paged_decode_merge_bf16(
        out.data_ptr(), out.stride(0), context_lens.data_ptr(), b, hq, num_kv_heads, d,
        workspace.data_ptr(), workspace.numel(), _stream_ptr(out))
    _lib.check(rc, "paged_attn_decode_merge")


def flash_attn_with_kvcache(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, *,
                            cache_seqlens: "torch.Tensor | int", block_table: torch.Tensor,
                            softmax_scale: float | None = None, causal: bool = True) -> torch.Tensor:
    """``q`` is ``[B, 1, Hq, D]``; returns ``[B, 1, Hq, D]``.  With a single query token the causal
    mask hides nothing, so ``causal`` only has to be accepted.  ``cache_seqlens`` is an int32 tensor
    ``[B]`` or one int for the whole batch, as in flash-attn."""
    assert q.dim() == 4 and q.shape[1] == 1, "decode takes one query token per sequence"
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** -0.5
    q3 = q[:, 0]
    out = torch.empty((q.shape[0], q.shape[2], q.shape[3]), dtype=q.dtype, device=q.device)
    paged_attn_decode(q3, k_cache, v_cache, block_table, cache_seqlens, softmax_scale, out)
    return out.unsqueeze(1)


def flash_attn_decode(Q: torch.Tensor, K: torch.Tensor, V: torch.Tensor, is_causal: bool,
                      block_table: torch.Tensor, O: torch.Tensor, context_lens: torch.Tensor,
                      softmax_scale: float | None = None) -> None:
    """``Q``/``O`` ``[B, Hq, D]``, ``K``/``V`` the paged caches."""
    if softmax_scale is None:
        softmax_scale = Q.shape[-1] ** -0.5
    paged_attn_decode(Q, K, V, block_table, context_lens, softmax_scale, O)


def flash_attn_varlen_func(q, k, v, *, max_seqlen_q, cu_seqlens_q, max_seqlen_k, cu_seqlens_k,
                           softmax_scale=None, causal=True, block_table=None):
    """Packed variable-length attention (keyword set of ``infer/ops/attention.py:113-116``).

    ``q`` is ``[total_q, Hq, D]``.  With ``block_table`` the keys come from the paged caches
    ``k``/``v`` ``[nblk, bs, Hkv, D]`` (prefix-cache case); without it ``k``/``v`` are the packed rows
    ``[total_k, Hkv, D]``.  Returns ``[total_q, Hq, D]``.  ``max_seqlen_k`` is accepted for
    signature compatibility; the kernel reads the lengths from ``cu_seqlens_k``."""
    assert q.dim() == 3 and q.dtype == torch.bfloat16 and k.dtype == torch.bfloat16 and v.dtype == torch.bfloat16
    tq, hq, d = q.shape
    assert q.stride(2) == 1 and q.stride(1) == d
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    assert cu_seqlens_q.is_contiguous() and cu_seqlens_k.is_contiguous()
    nseq = cu_seqlens_q.numel() - 1
    assert cu_seqlens_k.numel() == nseq + 1
    _require_gpu(q, k, v, cu_seqlens_q, cu_seqlens_k)
    if softmax_scale is None:
        softmax_scale = d ** -0.5
    out = torch.empty((tq, hq, d), dtype=q.dtype, device=q.device)
    if tq == 0 or nseq == 0:
        return out
    if block_table is not None:
        assert k.dim() == 4 and k.shape == v.shape and k.stride() == v.stride()
        nblk, bs, hkv, dk = k.shape
        assert dk == d and k.stride(3) == 1 and k.stride(2) == d
        assert block_table.dtype == torch.int32 and block_table.shape[0] == nseq and block_table.stride(1) == 1
        _require_gpu(block_table)
        blk_stride, tok_stride, rows = k.stride(0), k.stride(1), nblk * bs
        bt_ptr, bt_stride, bt_cols = block_table.data_ptr(), block_table.stride(0), block_table.shape[1]
    else:
        assert k.dim() == 3 and k.shape == v.shape and k.stride() == v.stride()
        rows, hkv, dk = k.shape
        assert dk == d and k.stride(2) == 1 and k.stride(1) == d
        blk_stride, tok_stride, bs, nblk = 0, k.stride(0), 0, 0
        bt_ptr, bt_stride, bt_cols = None, 0, 0
    rc = _lib.load().infer_paged_prefill_bf16(
        q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), blk_stride, tok_stride, rows,
        out.data_ptr(), out.stride(0), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), bt_ptr, bt_stride, bt_cols,
        nseq, int(max_seqlen_q), hq, hkv, d, bs, nblk, float(softmax_scale), int(bool(causal)), _stream_ptr(q))
    _lib.check(rc, "flash_attn_varlen_func")
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
             out: torch.Tensor | None = None):
    """``RMSNorm.forward`` of ``infer/ops/norm.py:63-98``: returns ``out`` or, with ``residual``,
    ``(out, residual)`` where ``residual`` has been updated in place to ``x + residual``."""
    if isinstance(x, SplitKSum):
        return _rms_norm_splitk(x, weight, eps, residual, out)
    hidden = x.shape[-1]
    x2 = x.reshape(-1, hidden)
    assert x2.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x2.stride(1) == 1
    assert weight.shape == (hidden,) and weight.is_contiguous()
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    o2 = out.view(-1, hidden)
    assert o2.shape == x2.shape and o2.dtype == torch.bfloat16 and o2.stride(1) == 1
    r2 = None
    if residual is not None:
        r2 = residual.view(-1, hidden)
        assert r2.shape == x2.shape and r2.dtype == torch.bfloat16 and r2.stride(1) == 1
    _require_gpu(x2, weight, o2, *([r2] if r2 is not None else []))
    rc = _lib.load().infer_rms_norm_bf16(
        x2.data_ptr(), x2.stride(0), r2.data_ptr() if r2 is not None else None,
        r2.stride(0) if r2 is not None else 0, weight.data_ptr(), o2.data_ptr(), o2.stride(0),
        x2.shape[0], hidden, float(eps), _stream_ptr(x))
    _lib.check(rc, "rms_norm")
    return out if residual is None else (out, residual)


def _rms_norm_splitk(x: "SplitKSum", weight, eps, residual, out):
    """RMSNorm over a split-K GEMM result that is still in pieces: the kernel adds the partial sums
    (in split order, rounded to bf16 once: the same bits as reducing first) and normalises."""
    x.check_alive()
    p = x.partial
    splits, m, hidden = p.shape
    assert p.dtype == torch.float32 and p.is_contiguous()
    assert weight.dtype == torch.bfloat16 and weight.shape == (hidden,) and weight.is_contiguous()
    if out is None:
        out = torch.empty((m, hidden), dtype=x.dtype, device=p.device)
    assert out.shape == (m, hidden) and out.dtype == torch.bfloat16 and out.stride(1) == 1
    r2 = None
    if residual is not None:
        r2 = residual.view(-1, hidden)
        assert r2.shape == (m, hidden) and r2.dtype == torch.bfloat16 and r2.stride(1) == 1
    rc = _lib.load().infer_rms_norm_splitk_bf16(
        p.data_ptr(), splits, m * hidden, hidden, r2.data_ptr() if r2 is not None else None,
        r2.stride(0) if r2 is not None else 0, weight.data_ptr(), out.data_ptr(), out.stride(0), m, hidden,
        float(eps), _stream_ptr(p))
    _lib.check(rc, "rms_norm (split-K input)")
    return out if residual is None else (out, residual)


def silu_and_mul(out: torch.Tensor, x: torch.Tensor) -> None:
    """``silu_and_mul(result, input)`` of ``src/bindings.cpp:22``: ``out = silu(x[..., :d]) * x[..., d:]``."""
    d = x.shape[-1] // 2
    x2 = x.reshape(-1, 2 * d)
    o2 = out.view(-1, d)
    assert x.shape[-1] == 2 * d and o2.shape[0] == x2.shape[0]
    assert x2.dtype == torch.bfloat16 and o2.dtype == torch.bfloat16 and x2.stride(1) == 1 and o2.stride(1) == 1
    _require_gpu(x2, o2)
    rc = _lib.load().infer_silu_and_mul_bf16(o2.data_ptr(), o2.stride(0), x2.data_ptr(), x2.stride(0),
                                             x2.shape[0], d, _stream_ptr(x))
    _lib.check(rc, "silu_and_mul")


def decode_metadata(seq_lens: torch.Tensor, block_table: torch.Tensor, block_size: int, position_offset: int,
                    positions: torch.Tensor, slot_mapping: torch.Tensor, context_lens: torch.Tensor) -> None:
    """Derives a decode step's ``positions`` / ``slot_mapping`` / ``context_lens`` on the device from
    the sequence lengths and the block table (``infer/engine/model_runner.py:110-126``); rows with
    length 0 are padding (slot -1, context length 0)."""
    b = seq_lens.numel()
    assert seq_lens.dtype == torch.int32 and seq_lens.is_contiguous()
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] == b
    assert block_table.stride(1) == 1
    assert positions.dtype == torch.int64 and slot_mapping.dtype == torch.int32 and context_lens.dtype == torch.int32
    for t in (positions, slot_mapping, context_lens):
        assert t.numel() == b and t.is_contiguous()
    _require_gpu(seq_lens, block_table, positions, slot_mapping, context_lens)
    rc = _lib.load().infer_decode_metadata(
        seq_lens.data_ptr(), block_table.data_ptr(), block_table.stride(0), b, int(block_size),
        block_table.shape[1], int(position_offset), positions.data_ptr(), slot_mapping.data_ptr(),
        context_lens.data_ptr(), _stream_ptr(seq_lens))
    _lib.check(rc, "decode_metadata")


_gemm_workspaces: dict = {}


def skinny_linear_supported(m: int, n: int, k: int) -> bool:
    """Shapes the split-K weight-streaming GEMM takes: decode-sized batches over aligned weights."""
    return 0 < m <= 128 and k % 128 == 0 and n % 8 == 0


def _gemm_workspace(device, need: int) -> torch.Tensor | None:
    key = str(device)
    ws = _gemm_workspaces.get(key)
    if need and (ws is None or ws.numel() < need):
        if ws is not None:
            _retired_workspaces.append(ws)
        ws = torch.empty(max(need, 64 << 20), dtype=torch.uint8, device=device)
        _gemm_workspaces[key] = ws
    return ws


class SplitKSum:
    """Result of a split-K GEMM that has not been reduced yet: ``partial`` ``[splits, M, N]`` float32
    lives in the shared GEMM workspace, so it must be consumed (``rms_norm`` does, ``materialize``
    does) before the next split-K GEMM on the device runs; ``generation`` guards that."""
    _generation: dict = {}

    def __init__(self, partial: torch.Tensor, dtype):
        self.partial = partial
        self.dtype = dtype
        key = str(partial.device)
        self.generation = SplitKSum._generation[key] = SplitKSum._generation.get(key, 0) + 1

    @property
    def shape(self):
        return self.partial.shape[1:]

    def check_alive(self):
        if SplitKSum._generation.get(str(self.partial.device)) != self.generation:
            raise RuntimeError("split-K partial sums were overwritten by a later GEMM before they were consumed")

    def materialize(self) -> torch.Tensor:
        self.check_alive()
        total = self.partial[0].clone()
        for s in range(1, self.partial.shape[0]):      # split order, as the kernels add them
            total += self.partial[s]
        return total.to(self.dtype)


def skinny_linear_deferred(x: torch.Tensor, weight: torch.Tensor):
    """``skinny_linear`` that leaves the split-K reduction to its consumer: returns a ``SplitKSum`` when
    the shape was split, the finished bf16 tensor otherwise."""
    m, k = x.shape
    n = weight.shape[0]
    assert weight.shape == (n, k) and weight.is_contiguous()
    assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.stride(1) == 1
    _require_gpu(x, weight)
    lib = _lib.load()
    need = lib.infer_skinny_gemm_workspace_bytes(m, n, k)
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    if not need:
        return skinny_linear(x, weight, out)
    ws = _gemm_workspace(x.device, need)
    splits = ctypes.c_int(0)
    rc = lib.infer_skinny_gemm_partial_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), out.data_ptr(),
                                            out.stride(0), m, n, k, ws.data_ptr(), ws.numel(),
                                            ctypes.byref(splits), _stream_ptr(x))
    _lib.check(rc, "skinny_linear_deferred")
    if splits.value <= 1:
        return out
    partial = ws[:splits.value * m * n * 4].view(torch.float32).view(splits.value, m, n)
    return SplitKSum(partial, x.dtype)


def skinny_linear(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """``F.linear(x, weight)`` for ``x`` ``[M, K]`` with ``M <= 128`` (``Linear.forward``,
    ``infer/ops/MLP.py:103-149``): the weight matrix ``[N, K]`` is streamed once by a hand-written
    split-K kernel.  The float32 workspace is cached per device and only ever grows (a captured graph
    keeps pointing at the one it was captured with, so outgrown buffers are kept alive)."""
    m, k = x.shape
    n = weight.shape[0]
    assert weight.shape == (n, k) and weight.is_contiguous()
    assert x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.stride(1) == 1
    if out is None:
        out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    assert out.shape == (m, n) and out.dtype == torch.bfloat16 and out.stride(1) == 1
    _require_gpu(x, weight, out)
    lib = _lib.load()
    need = lib.infer_skinny_gemm_workspace_bytes(m, n, k)
    ws = _gemm_workspace(x.device, need)
    if need:      # any unconsumed SplitKSum in this workspace is gone after this launch
        SplitKSum._generation[str(x.device)] = SplitKSum._generation.get(str(x.device), 0) + 1
    rc = lib.infer_skinny_gemm_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), out.data_ptr(), out.stride(0),
                                    m, n, k, ws.data_ptr() if need else None, ws.numel() if need else 0,
                                    _stream_ptr(x))
    _lib.check(rc, "skinny_linear")
    return out


_linear_choice: dict = {}
_linear_timings: dict = {}      # (device, batch bucket, N, K) -> (vendor ms, own ms), for inspection
_flush_buffers: dict = {}

# Weight matrices with at most this many rows go to the split-K kernel at decode batch sizes: the vendor
# GEMM has too few output tiles to fill the chip there (o_proj, down_proj: 4096 rows = 32 tiles of 128 on
# 256 compute units, 27 and 68 us against 22 and 38), and is ahead on every wider projection measured
# (qkv 6144, gate_up 24576, lm_head 151936 rows) and on short reductions (K below 2048).  On the three
# published Qwen3 shapes the rule picks what a cold-cache timing of both kernels picks, within 2.5 %
# of a decode step on the smallest.
SKINNY_MAX_ROWS = 5120


def _linear_mode() -> str:
    """``INFER_AMD_LINEAR``: ``static`` (default: the fixed rule above, the same kernel for a shape in every
    process), ``vendor`` (never the split-K kernel), ``measure`` (time both once per shape with cold caches and
    keep the faster: a tuning aid, not reproducible from run to run)."""
    import os
    mode = os.environ.get("INFER_AMD_LINEAR", "static")
    if mode not in ("static", "vendor", "measure"):
        raise RuntimeError(f"INFER_AMD_LINEAR must be static, vendor or measure, not {mode!r}")
    return mode


def _time_cold(fn, device, reps: int = 6) -> float:
    """Median GPU time of ``fn`` with the caches flushed before every launch (the weights of a decode
    step are read once per step, so a warm-cache timing would rank the kernels wrongly)."""
    flush = _flush_buffers.get(str(device))
    if flush is None:
        flush = _flush_buffers[str(device)] = torch.zeros(128 << 20, dtype=torch.int32, device=device)
    times = []
    for i in range(reps + 2):
        flush.sum()       # reading 512 MB leaves the caches full of clean lines, as the previous layers' weights do
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        if i >= 2:
            times.append(start.elapsed_time(end))
    times.sort()
    return times[len(times) // 2]


def linear(x: torch.Tensor, weight: torch.Tensor, defer: bool = False):
    """``F.linear(x, weight)`` that sends decode-sized batches over narrow weight matrices to the split-K
    weight-streaming kernel and everything else to the vendor GEMM.  The choice is a fixed rule on the
    shape (see ``_linear_mode`` for the alternatives), so a shape runs the same kernel, with the same
    rounding, in every process and inside and outside a captured graph."""
    if x.dim() != 2 or not x.is_cuda or x.dtype != torch.bfloat16:
        return torch.nn.functional.linear(x, weight)
    m, k = x.shape
    n = weight.shape[0]
    if not skinny_linear_supported(m, n, k) or not weight.is_contiguous() or x.stride(1) != 1:
        return torch.nn.functional.linear(x, weight)
    mode = _linear_mode()
    if mode == "vendor":
        return torch.nn.functional.linear(x, weight)
    if mode == "static":
        use = n <= SKINNY_MAX_ROWS and k >= 2048
    else:
        bucket = 16 if m <= 16 else 32 if m <= 32 else 64 if m <= 64 else 128
        key = (str(x.device), bucket, n, k)
        use = _linear_choice.get(key)
        if use is None:
            if torch.cuda.is_current_stream_capturing():
                return torch.nn.functional.linear(x, weight)
            probe = x if m == bucket else torch.zeros((bucket, k), dtype=x.dtype, device=x.device)
            t_lib = _time_cold(lambda: torch.nn.functional.linear(probe, weight), x.device)
            t_own = _time_cold(lambda: skinny_linear(probe, weight), x.device)
            _linear_timings[key] = (t_lib, t_own)
            use = _linear_choice[key] = bool(t_own < 0.95 * t_lib)
    if not use:
        return torch.nn.functional.linear(x, weight)
    # ``defer``: the caller hands the result straight to ``rms_norm``, which adds the partial sums itself
    return skinny_linear_deferred(x, weight) if defer else skinny_linear(x, weight)
