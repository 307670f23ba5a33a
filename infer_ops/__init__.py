"""``infer_ops``: the op namespace the reference's Python engine imports (``infer_ops/__init__.py``
there loads ``_C*.so`` and re-exports ``torch.ops._C.*``), here carrying the ops of the paged
KV-cache path.

``torch.ops._C.store_kvcache / paged_attn_decode / flash_attn_decode / paged_attn_prefill`` are
registered by ``infer_amd/_C_infer_kv.so`` (out-parameter style, ``-> ()``, as in the reference's
``src/bindings.cpp``).  The flash-attn-compatible functional forms come from ``infer_amd.ops``.
The reference's other eleven names (``infer_ops/__init__.py:25-45`` there) stay importable with the
reference's out-parameter signatures (``src/bindings.cpp:4-23``): ``rms_norm_vllm`` and ``silu_and_mul``
run this build's HIP kernels, the rest are stated with torch operators on the tensors' device at the
reference kernels' rounding points - they are not on the KV-cache path and not tuned."""
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(os.path.dirname(_HERE), "infer_amd", "_C_infer_kv.so")
if not os.path.exists(_LIB):
    raise ImportError("Could not find the C++ extension library "
                      f"({_LIB}); run `make -C infer_amd/csrc`")
torch.ops.load_library(_LIB)

store_kvcache = torch.ops._C.store_kvcache
paged_attn_decode = torch.ops._C.paged_attn_decode
flash_attn_decode = torch.ops._C.flash_attn_decode
paged_attn_prefill = torch.ops._C.paged_attn_prefill

from infer_amd import ops as _ops  # noqa: E402
from infer_amd.ops import flash_attn_varlen_func, flash_attn_with_kvcache  # noqa: E402

__all__ = ["store_kvcache", "paged_attn_decode", "flash_attn_decode", "paged_attn_prefill",
           "flash_attn_with_kvcache", "flash_attn_varlen_func"]


def add(a, b, output):
    """``add(Tensor a, Tensor b, Tensor! output)``."""
    torch.add(a, b, out=output)


def rms_norm(input, weight, output, bias, eps):
    """``rms_norm(Tensor input, Tensor weight, Tensor! output, Tensor? bias, float eps)``: one rounding,
    ``bf16(x * rsqrt(mean(x^2) + eps) * w [+ bias])`` (``src/operators/add_rms/add_rms.cu:59-70``)."""
    x = input.float()
    y = x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps) * weight.float()
    if bias is not None:
        y = y + bias.float()
    output.copy_(y)


def rms_norm_vllm(result, input, weight, epsilon):
    """``rms_norm_vllm(Tensor! result, Tensor input, Tensor weight, float epsilon)`` (``add_rms.cu:340-367``)."""
    _ops.rms_norm(input, weight, epsilon, out=result)


def rms_norm_fused(input, residual, weight, epsilon):
    """``fused_add_rms_norm(Tensor! input, Tensor! residual, Tensor weight, float epsilon)``: the sum is
    rounded to bf16 before the variance (``add_rms.cu:427-458``)."""
    residual.copy_(input + residual)
    x = residual.float()
    y = (x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + epsilon)).to(input.dtype)
    input.copy_(y * weight)


def matmul(input, weight, output):
    """``matmul(Tensor input, Tensor weight, Tensor! output)`` with ``weight`` ``[K, N]``."""
    torch.matmul(input, weight, out=output)


def embedding(output, input, weight):
    """``embedding(Tensor! output, Tensor input, Tensor weight)``."""
    output.copy_(torch.nn.functional.embedding(input, weight).view(output.shape))


def flash_attn_prefill(Q, K, V, O):
    """``flash_attn_prefill(Tensor Q, Tensor K, Tensor V, Tensor! O)``: dense causal attention over
    ``[B, H, S, D]`` (the layout of ``test/op.py:269-287``)."""
    O.copy_(torch.nn.functional.scaled_dot_product_attention(Q, K, V, is_causal=True))


def rope(positions, query, key, head_size, cos_sin_cache, is_neox):
    """``rotary_embedding(Tensor positions, Tensor! query, Tensor!? key, int head_size, Tensor
    cos_sin_cache, bool is_neox)``: in place, every product and sum rounded to the tensors' dtype."""
    cos, sin = cos_sin_cache.index_select(0, positions.flatten()).chunk(2, dim=-1)
    cos, sin = cos.unsqueeze(-2).to(query.dtype), sin.unsqueeze(-2).to(query.dtype)
    for t in (query, key):
        if t is None:
            continue
        x = t.view(positions.numel(), -1, head_size)
        rot = x[..., :cos.shape[-1] * 2]
        x1, x2 = (rot[..., ::2], rot[..., 1::2]) if not is_neox else rot.chunk(2, dim=-1)
        o1, o2 = x1 * cos - x2 * sin, x2 * cos + x1 * sin
        rot.copy_(torch.cat((o1, o2), dim=-1) if is_neox else torch.stack((o1, o2), dim=-1).flatten(-2))


def silu(output, input):
    """``silu(Tensor! output, Tensor input)``."""
    output.copy_(torch.nn.functional.silu(input.float()))


def softmax(output, input, axis):
    """``softmax(Tensor! output, Tensor input, int axis)``."""
    output.copy_(torch.softmax(input.float(), dim=axis))


def silu_and_mul(result, input):
    """``silu_and_mul(Tensor! result, Tensor input)`` (``src/operators/silu/silu.cu:13-54``)."""
    _ops.silu_and_mul(result, input)


__all__ += ["add", "rms_norm", "matmul", "embedding", "flash_attn_prefill", "rope", "silu", "softmax",
            "rms_norm_vllm", "rms_norm_fused", "silu_and_mul"]
