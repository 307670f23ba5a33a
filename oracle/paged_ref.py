"""CPU oracle for the paged KV-cache hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``oracle/`` is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The product path (``infer_amd``) never
falls back to this code.

What is restated here, and from where (all paths are into the reference tree):

* ``append_ref``         - ``infer/ops/attention.py:16-45`` (``store_kvcache_kernel`` /
  ``store_kvcache``): ``cache.flat[slot*D : slot*D+D] = row``.  The reference has no guard for
  negative slots (a ``-1`` would write before the buffer); the build requirement is that
  padding slots (``slot < 0``) are skipped, which is what this function does.
* ``paged_decode_ref``   - the call at ``infer/ops/attention.py:118-120``
  (``flash_attn_with_kvcache(q[B,1,Hq,D], k_cache, v_cache, cache_seqlens, block_table,
  softmax_scale, causal=True)``).  ``flash_attn`` (Dao-AILab flash-attention, version unpinned
  by the reference: no requirements file names it) is NOT vendored in the reference, so the
  arithmetic restated is its published semantics: token ``t`` of sequence ``b`` lives at
  ``cache[block_table[b, t // bs], t % bs, h // G, :]``; the output is
  ``softmax(scale * q . K^T) V`` over the first ``cache_seqlens[b]`` tokens, KV head
  ``h // (Hq/Hkv)``; with one query token ``causal=True`` hides nothing.  Rows with
  ``cache_seqlens == 0`` produce zeros.
* ``varlen_prefill_ref`` - the call at ``infer/ops/attention.py:110-116``
  (``flash_attn_varlen_func(..., causal=True, block_table=...)``): packed variable-length
  causal attention, the causal mask aligned to the bottom-right corner
  (key ``j`` visible to query ``i`` iff ``j <= i + (sk - sq)``); with ``block_table`` the keys
  of sequence ``b`` are tokens ``[0, sk_b)`` of its paged cache.
* ``sdpa_dense``         - ``infer/ops/attention.py:64-71`` (``forward_native`` =
  ``scaled_dot_product_attention(is_causal=False)``), the one torch attention the reference owns.

Parity status.  The reference holds no golden vector, known-answer test or fixture for any of
these functions (its ``test/op.py`` never calls them), so each one is pinned by what the
mathematics fixes instead (see ``tests/test_oracle.py``): the append against an independent
``numpy`` fancy-index copy and its invariants; the decode against a pure-Python brute force on
tiny shapes, closed forms (one token => ``O = V[0]``; equal keys => ``O = mean(V)``),
block-permutation invariance, and ``torch.nn.functional.scaled_dot_product_attention`` on the
gathered keys; the prefill against SDPA with ``is_causal=True`` when ``sq == sk`` (the
convention of ``test/op.py:278-283``) and an explicit mask otherwise.  At the ``flash_attn``
boundary itself parity is unpinned by the reference: there is nothing of flash-attn's to
compare with in this tree.

Arithmetic: bf16 storage is carried as ``uint16`` bit patterns, all math in float32 (float64
for the brute force), outputs returned in float32 so the caller chooses how to round.
"""
from __future__ import annotations

import math

import numpy as np


# --------------------------------------------------------------------------- bf16 <-> f32

def bf16_to_f32(u16: np.ndarray) -> np.ndarray:
    """Widen bf16 bit patterns (uint16) to float32 exactly."""
    u16 = np.ascontiguousarray(u16, dtype=np.uint16)
    return (u16.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round float32 to bf16 bit patterns, round-to-nearest-even; NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    lsb = (bits >> np.uint32(16)) & np.uint32(1)
    rounded = (bits + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    nan = np.isnan(x)
    out = rounded.astype(np.uint16)
    if nan.any():
        out = np.where(nan, ((bits >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), out)
    return out


# --------------------------------------------------------------------------- append

def append_ref(key: np.ndarray, value: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
               slot_mapping: np.ndarray) -> None:
    """Scatter rows of ``key``/``value`` ([N, Hkv, D] uint16) into the caches in place.

    ``k_cache``/``v_cache`` are [nblk, bs, Hkv, D] uint16 (C-contiguous), ``slot_mapping`` [N]
    integers; row ``i`` lands at flat row ``slot_mapping[i]``; rows with a negative slot are
    skipped.  Written as an explicit loop so that duplicate slots resolve in program order.
    """
    n, hkv, d = key.shape
    assert value.shape == key.shape and slot_mapping.shape == (n,)
    width = hkv * d
    kc = k_cache.reshape(-1, width)
    vc = v_cache.reshape(-1, width)
    assert kc.base is not None or kc is k_cache  # a view, not a copy
    for i in range(n):
        s = int(slot_mapping[i])
        if s < 0:
            continue
        kc[s, :] = key[i].reshape(width)
        vc[s, :] = value[i].reshape(width)


# --------------------------------------------------------------------------- decode

def gather_sequence(cache: np.ndarray, table_row: np.ndarray, length: int) -> np.ndarray:
    """Return the first ``length`` tokens of a sequence as [length, Hkv, D] (dtype of cache)."""
    bs = cache.shape[1]
    nb = (length + bs - 1) // bs
    blocks = [cache[int(table_row[j])] for j in range(nb)]
    if not blocks:
        return np.zeros((0,) + cache.shape[2:], dtype=cache.dtype)
    return np.concatenate(blocks, axis=0)[:length]


def _softmax_rows(s: np.ndarray) -> np.ndarray:
    m = s.max(axis=-1, keepdims=True)
    m = np.where(np.isfinite(m), m, 0.0)
    e = np.exp(s - m)
    z = e.sum(axis=-1, keepdims=True)
    return e / np.where(z == 0.0, 1.0, z)


def paged_decode_ref(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
                     block_table: np.ndarray, context_lens: np.ndarray, scale: float) -> np.ndarray:
    """Paged decode attention.  ``q`` [B, Hq, D] uint16 (bf16 bits); returns float32 [B, Hq, D]."""
    b, hq, d = q.shape
    hkv = k_cache.shape[2]
    g = hq // hkv
    assert hq == g * hkv
    out = np.zeros((b, hq, d), dtype=np.float32)
    qf = bf16_to_f32(q)
    for i in range(b):
        length = int(context_lens[i])
        if length <= 0:
            continue
        kf = bf16_to_f32(gather_sequence(k_cache, block_table[i], length))  # [L, Hkv, D]
        vf = bf16_to_f32(gather_sequence(v_cache, block_table[i], length))
        for h in range(hkv):
            qs = qf[i, h * g:(h + 1) * g]                      # [G, D]
            s = (qs @ kf[:, h, :].T) * np.float32(scale)       # [G, L]
            p = _softmax_rows(s.astype(np.float32))
            out[i, h * g:(h + 1) * g] = p @ vf[:, h, :]
    return out


def paged_decode_bruteforce(q, k_cache, v_cache, block_table, context_lens, scale):
    """Same contract as ``paged_decode_ref`` written as scalar Python loops in float64.

    Addresses every element as ``cache[block_table[b, t // bs], t % bs, h // G, x]`` directly, so
    a mistake in ``gather_sequence``, the head map or the softmax of the vectorised version shows
    up as a disagreement.  Only for tiny shapes.
    """
    b, hq, d = q.shape
    bs = k_cache.shape[1]
    hkv = k_cache.shape[2]
    g = hq // hkv
    qf = bf16_to_f32(q).astype(np.float64)
    kf = bf16_to_f32(k_cache).astype(np.float64)
    vf = bf16_to_f32(v_cache).astype(np.float64)
    out = np.zeros((b, hq, d), dtype=np.float64)
    for i in range(b):
        length = int(context_lens[i])
        for h in range(hq):
            kvh = h // g
            scores = []
            for t in range(length):
                blk = int(block_table[i, t // bs])
                dot = 0.0
                for x in range(d):
                    dot += qf[i, h, x] * kf[blk, t % bs, kvh, x]
                scores.append(dot * scale)
            if not scores:
                continue
            m = max(scores)
            w = [math.exp(s - m) for s in scores]
            z = sum(w)
            for t in range(length):
                blk = int(block_table[i, t // bs])
                for x in range(d):
                    out[i, h, x] += (w[t] / z) * vf[blk, t % bs, kvh, x]
    return out.astype(np.float32)


# --------------------------------------------------------------------------- prefill

def varlen_prefill_ref(q: np.ndarray, k: np.ndarray, v: np.ndarray, cu_seqlens_q: np.ndarray,
                       cu_seqlens_k: np.ndarray, scale: float,
                       block_table: np.ndarray | None = None, causal: bool = True) -> np.ndarray:
    """Packed variable-length attention.  ``q`` [Tq, Hq, D] uint16.

    Without ``block_table``: ``k``/``v`` are packed [Tk, Hkv, D] uint16 indexed by
    ``cu_seqlens_k``.  With ``block_table`` [nseq, MB]: ``k``/``v`` are the paged caches
    [nblk, bs, Hkv, D] and sequence ``b`` uses tokens ``[0, sk_b)`` of its table row.
    Returns float32 [Tq, Hq, D].
    """
    tq, hq, d = q.shape
    nseq = len(cu_seqlens_q) - 1
    hkv = k.shape[-2]
    g = hq // hkv
    qf = bf16_to_f32(q)
    out = np.zeros((tq, hq, d), dtype=np.float32)
    for b in range(nseq):
        q0, q1 = int(cu_seqlens_q[b]), int(cu_seqlens_q[b + 1])
        k0, k1 = int(cu_seqlens_k[b]), int(cu_seqlens_k[b + 1])
        sq, sk = q1 - q0, k1 - k0
        if sq == 0 or sk == 0:
            continue
        if block_table is not None:
            kf = bf16_to_f32(gather_sequence(k, block_table[b], sk))
            vf = bf16_to_f32(gather_sequence(v, block_table[b], sk))
        else:
            kf = bf16_to_f32(k[k0:k1])
            vf = bf16_to_f32(v[k0:k1])
        if causal:
            qi = np.arange(sq)[:, None]
            kj = np.arange(sk)[None, :]
            visible = kj <= qi + (sk - sq)
        else:
            visible = np.ones((sq, sk), dtype=bool)
        for h in range(hq):
            s = (qf[q0:q1, h, :] @ kf[:, h // g, :].T) * np.float32(scale)
            s = np.where(visible, s, -np.inf).astype(np.float32)
            p = _softmax_rows(s)
            p = np.where(visible.any(axis=-1, keepdims=True), p, 0.0).astype(np.float32)
            out[q0:q1, h, :] = p @ vf[:, h // g, :]
    return out


# --------------------------------------------------------------------------- metadata closed forms

def decode_metadata_ref(lengths, block_tables, block_size):
    """Slot / context length / padded table for one decode step.

    Follows ``infer/engine/model_runner.py:110-126`` (``prepare_decode``) and ``:66-70``
    (``prepare_block_tables``) with ``infer/engine/sequence.py:59-64``: the newest token of a
    sequence of ``n`` tokens sits at ``table[-1] * bs + (n - (ceil(n/bs) - 1) * bs) - 1``.
    """
    slots, ctx = [], []
    for n, table in zip(lengths, block_tables):
        nblocks = (n + block_size - 1) // block_size
        last = n - (nblocks - 1) * block_size
        slots.append(table[-1] * block_size + last - 1)
        ctx.append(n)
    width = max(len(t) for t in block_tables)
    padded = [list(t) + [-1] * (width - len(t)) for t in block_tables]
    return (np.asarray(slots, dtype=np.int32), np.asarray(ctx, dtype=np.int32),
            np.asarray(padded, dtype=np.int32))


def prefill_metadata_ref(lengths, cached, block_tables, block_size):
    """``cu_seqlens_q/k``, maxima and slot_mapping of a prefill step.

    Follows ``infer/engine/model_runner.py:72-108`` (``prepare_prefill``): queries are the
    tokens after the cached prefix, keys the whole sequence, slots cover every non-cached block
    with the last block truncated to its fill.
    """
    cu_q, cu_k, slots = [0], [0], []
    max_q = max_k = 0
    for n, c, table in zip(lengths, cached, block_tables):
        cu_q.append(cu_q[-1] + n - c)
        cu_k.append(cu_k[-1] + n)
        max_q, max_k = max(max_q, n - c), max(max_k, n)
        nblocks = (n + block_size - 1) // block_size
        for i in range(c // block_size, nblocks):
            start = table[i] * block_size
            fill = block_size if i != nblocks - 1 else n - (nblocks - 1) * block_size
            slots.extend(range(start, start + fill))
    return (np.asarray(cu_q, dtype=np.int32), np.asarray(cu_k, dtype=np.int32), max_q, max_k,
            np.asarray(slots, dtype=np.int32))
