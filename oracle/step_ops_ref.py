"""TEST INFRASTRUCTURE ONLY: numpy restatements, with the reference's bf16 rounding points, of the two
elementwise operators a decode step runs around the KV-cache path.  Nothing in the product imports
this file.

* ``add_rms_norm_ref`` follows ``RMSNorm.rms_forward`` / ``add_rms_forward`` (``infer/ops/norm.py:63-86``):
  float32 sum of input and residual; the residual output is that sum rounded to bf16; the variance
  and the scaling use the unrounded sum; the scaled value is rounded to bf16 and multiplied by the
  bf16 weight (rounded again).
* ``silu_and_mul_ref`` follows ``act_and_mul_kernel`` with ``silu_kernel_vllm``
  (``src/operators/silu/silu.cu:13-31``): ``bf16(x / (1 + exp(-x)))`` times the up value, rounded.

Pinned in ``tests/test_step_ops_gpu.py``'s CPU part against torch's own bf16 arithmetic
(``torch.nn.functional.rms_norm`` in float64 for the value, torch bf16 tensors for the rounding)."""
from __future__ import annotations

import numpy as np

from .paged_ref import bf16_to_f32, f32_to_bf16


def _round(x: np.ndarray) -> np.ndarray:
    return bf16_to_f32(f32_to_bf16(np.asarray(x, dtype=np.float32)))


def add_rms_norm_ref(x: np.ndarray, weight: np.ndarray, eps: float, residual: np.ndarray | None = None):
    """``x`` [N, H] uint16 (bf16 bits), ``weight`` [H] uint16 -> ``out`` uint16, or ``(out, new_residual)``."""
    s = bf16_to_f32(x)
    new_residual = None
    if residual is not None:
        s = s + bf16_to_f32(residual)
        new_residual = f32_to_bf16(s)
    var = np.mean(s * s, axis=-1, keepdims=True, dtype=np.float32)
    y = _round(s * (np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)))
    out = f32_to_bf16(y * bf16_to_f32(weight))
    return out if residual is None else (out, new_residual)


def silu_and_mul_ref(x: np.ndarray) -> np.ndarray:
    """``x`` [N, 2 d] uint16 -> [N, d] uint16."""
    d = x.shape[-1] // 2
    g, u = bf16_to_f32(x[..., :d]), bf16_to_f32(x[..., d:])
    act = _round(g / (np.float32(1.0) + np.exp(-g, dtype=np.float32)))
    return f32_to_bf16(act * u)
