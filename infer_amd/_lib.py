"""ctypes binding of ``libinfer_kv.so`` (see ``include/infer_kv.h`` for the contract).

The library is built in-tree by ``infer_amd/csrc/Makefile``.  There is no fallback: if the
library is missing, loading raises ``ImportError`` and every op that needs it fails loudly.
"""
from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
# INFER_KV_LIB lets a developer point at an experimental build of the same library.
LIB_PATH = os.environ.get("INFER_KV_LIB") or os.path.join(_HERE, "libinfer_kv.so")

_lock = threading.Lock()
_lib = None

_c = ctypes
_i64, _i32, _f32, _vp, _sz = _c.c_int64, _c.c_int32, _c.c_float, _c.c_void_p, _c.c_size_t

# name -> (restype, argtypes); mirrors include/infer_kv.h declaration by declaration
SIGNATURES = {
    "infer_kv_version": (_c.c_char_p, []),
    "infer_kv_strerror": (_c.c_char_p, [_c.c_int]),
    "infer_kv_append_bf16": (_c.c_int, [_vp, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "infer_kv_gather_bf16": (_c.c_int, [_vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "infer_kv_qk_norm_rope_append_bf16": (_c.c_int, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _f32, _vp, _i64,
                                                     _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _c.c_int, _vp]),
    "infer_kv_init": (_c.c_int, []),
    "infer_paged_decode_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "infer_paged_decode_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp,
                                           _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _vp, _sz, _vp]),
    "infer_paged_decode_split_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _i64, _vp,
                                                 _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64, _vp, _sz, _vp]),
    "infer_paged_decode_noalloc_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _vp,
                                                   _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp]),
    "infer_paged_decode_uniform_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64,
                                                   _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp, _sz, _vp]),
    "infer_paged_decode_merge_bf16": (_c.c_int, [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "infer_paged_prefill_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _i64,
                                            _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _c.c_int, _vp]),
    "infer_rms_norm_bf16": (_c.c_int, [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _f32, _vp]),
    "infer_silu_and_mul_bf16": (_c.c_int, [_vp, _i64, _vp, _i64, _i64, _i64, _vp]),
    "infer_decode_metadata": (_c.c_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "infer_skinny_gemm_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "infer_skinny_gemm_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "infer_skinny_gemm_partial_bf16": (_c.c_int, [_vp, _i64, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _sz, _vp, _vp]),
    "infer_rms_norm_splitk_bf16": (_c.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _f32,
                                              _vp]),
    "infer_pool_create": (_vp, [_i32, _i32]),
    "infer_pool_destroy": (None, [_vp]),
    "infer_pool_last_error": (_c.c_char_p, []),
    "infer_pool_num_free": (_i32, [_vp]),
    "infer_pool_num_used": (_i32, [_vp]),
    "infer_pool_can_allocate": (_c.c_int, [_vp, _i64]),
    "infer_pool_allocate": (_i64, [_vp, _vp, _i64, _vp, _i64]),
    "infer_pool_deallocate": (_c.c_int, [_vp, _vp, _i64]),
    "infer_pool_can_append": (_c.c_int, [_vp, _i64]),
    "infer_pool_may_append": (_i64, [_vp, _vp, _i64, _vp, _i64, _i64]),
    "infer_pool_may_append_block": (_i64, [_vp, _vp, _i64, _vp, _i64, _i64]),
    "infer_pool_hash": (_c.c_uint64, [_vp, _i64, _c.c_int, _c.c_uint64]),
    "infer_xxh64": (_c.c_uint64, [_vp, _sz, _c.c_uint64]),
    "infer_pool_ref_count": (_i32, [_vp, _i32]),
    "infer_pool_block_hash": (_c.c_int, [_vp, _i32, _vp]),
    "infer_pool_free_ids": (_i64, [_vp, _vp, _i64]),
}


def load():
    """Load the shared library once and attach argument types.  Raises ImportError if absent."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise ImportError(
                    f"{LIB_PATH} is not built; run `make -C infer_amd/csrc` (or __graft_entry__.build())")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            _lib = lib
    return _lib


def check(code: int, what: str) -> None:
    """Turn a non-zero return code into RuntimeError (the reference's ops raise RuntimeError through
    TORCH_CHECK / std::runtime_error, e.g. src/operators/flashattn/flashattn.cu:272)."""
    if code != 0:
        msg = load().infer_kv_strerror(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")
