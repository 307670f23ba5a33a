"""CPU oracle for the step in front of the KV append: per-head RMSNorm of Q and K, neox RoPE, then
the append.  TEST INFRASTRUCTURE ONLY (see oracle/paged_ref.py for who may import this).

Restates, in numpy on bf16 bit patterns:

* ``rms_norm_ref``  - ``RMSNorm.rms_forward`` (``infer/ops/norm.py:63-73``) as applied per head by
  ``QwenAttention.forward`` (``infer/models/Qwen3.py:113-118``): float32 mean of squares over the
  head dimension, ``x * rsqrt(var + eps)`` in float32, rounded to bf16, then multiplied by the bf16
  weight with the product rounded to bf16 again (eager semantics; under ``torch.compile`` the
  reference may skip the intermediate rounding, a difference of at most one bf16 ulp).
* ``rope_neox_ref`` - the neox branch of ``apply_token_rotary_embedding``
  (``src/operators/rope/rope.cu:43-66``) = ``_apply_rotary_emb_torch`` (``infer/ops/rope.py:48-66``):
  ``o1 = x1*cos - x2*sin``, ``o2 = x2*cos + x1*sin`` with every product and the sum rounded to bf16
  (bf16 operands, bf16 arithmetic), ``x1``/``x2`` the two halves of the head, cos/sin read from
  ``cos_sin_cache[position] = [cos(64) | sin(64)]``.
* ``qk_norm_rope_append_ref`` - the sequence ``Qwen3.py:113-131``: norm(q), norm(k), rope(q, k) in
  place, then ``store_kvcache(k, v)`` (``infer/ops/attention.py:108-109``), padding slots skipped.

Pinned in ``tests/test_rope_norm_oracle.py`` against the same formulas written with torch's own
bf16 tensor arithmetic on the CPU (bit-exact for RoPE, within one bf16 ulp for the norm whose
float32 reduction order is not fixed), against closed forms (position 0 is the identity, a rotation
preserves the pair norms, unit weight and constant rows), and the reference's test tolerance
(``test/op.py`` rope test: atol = rtol = 1e-2).
"""
from __future__ import annotations

import numpy as np

from .paged_ref import append_ref, bf16_to_f32, f32_to_bf16


def _round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 value, returned as float32."""
    return bf16_to_f32(f32_to_bf16(x.astype(np.float32)))


def rms_norm_ref(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """``x`` [..., D] uint16, ``weight`` [D] uint16 -> uint16."""
    xf = bf16_to_f32(x)
    var = np.mean(xf * xf, axis=-1, keepdims=True, dtype=np.float32)
    y = _round(xf * (np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)))
    return f32_to_bf16(y * bf16_to_f32(weight))


def rope_neox_ref(x: np.ndarray, cos_sin_cache: np.ndarray, positions: np.ndarray) -> np.ndarray:
    """``x`` [N, H, D] uint16, ``cos_sin_cache`` [max_pos, D] uint16, ``positions`` [N] -> uint16."""
    n, h, d = x.shape
    half = d // 2
    xf = bf16_to_f32(x)
    cs = bf16_to_f32(cos_sin_cache[np.asarray(positions, dtype=np.int64)])    # [N, D]
    cos, sin = cs[:, None, :half], cs[:, None, half:]
    x1, x2 = xf[..., :half], xf[..., half:]
    o1 = _round(_round(x1 * cos) - _round(x2 * sin))
    o2 = _round(_round(x2 * cos) + _round(x1 * sin))
    return f32_to_bf16(np.concatenate([o1, o2], axis=-1))


def qk_norm_rope_append_ref(q, k, v, positions, q_weight, k_weight, eps, cos_sin_cache, k_cache, v_cache,
                            slot_mapping):
    """Returns the new (q, k) bit patterns and updates the caches in place."""
    q2 = rope_neox_ref(rms_norm_ref(q, q_weight, eps), cos_sin_cache, positions)
    k2 = rope_neox_ref(rms_norm_ref(k, k_weight, eps), cos_sin_cache, positions)
    append_ref(k2, v, k_cache, v_cache, slot_mapping)
    return q2, k2


def cos_sin_cache_ref(max_pos: int, rot_dim: int, base: float) -> np.ndarray:
    """cos/sin table in float64 rounded to bf16 ([max_pos, rot_dim] uint16).  The reference builds its
    table in bf16 arithmetic (``infer/ops/rope.py:89-100``), which is a property of its model set-up,
    not of the kernel; any table works as kernel input."""
    inv = 1.0 / (base ** (np.arange(0, rot_dim, 2, dtype=np.float64) / rot_dim))
    f = np.arange(max_pos, dtype=np.float64)[:, None] * inv[None, :]
    return f32_to_bf16(np.concatenate([np.cos(f), np.sin(f)], axis=-1).astype(np.float32))
