"""``infer_ops``: the op namespace the reference's Python engine imports (``infer_ops/__init__.py``
there loads ``_C*.so`` and re-exports ``torch.ops._C.*``), here carrying the ops of the paged
KV-cache path.

``torch.ops._C.store_kvcache / paged_attn_decode / flash_attn_decode / paged_attn_prefill`` are
registered by ``infer_amd/_C_infer_kv.so`` (out-parameter style, ``-> ()``, as in the reference's
``src/bindings.cpp``).  The flash-attn-compatible functional forms come from ``infer_amd.ops``.
The reference's other ops (add, rms_norm, rope, silu, matmul, ...) are not part of this build;
asking for one raises ``AttributeError`` with that explanation."""
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

from infer_amd.ops import flash_attn_varlen_func, flash_attn_with_kvcache  # noqa: E402

__all__ = ["store_kvcache", "paged_attn_decode", "flash_attn_decode", "paged_attn_prefill",
           "flash_attn_with_kvcache", "flash_attn_varlen_func"]

_NOT_BUILT = {"add", "rms_norm", "rms_norm_vllm", "rms_norm_fused", "matmul", "embedding", "flash_attn_prefill",
              "rope", "silu", "softmax", "silu_and_mul"}


def __getattr__(name):
    if name in _NOT_BUILT:
        raise AttributeError(f"infer_ops.{name} is outside the paged KV-cache path and is not built here")
    raise AttributeError(name)
