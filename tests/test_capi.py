"""The C-ABI library loads without a GPU and exports every symbol include/infer_kv.h declares."""
import ctypes
import os
import re

import pytest

from infer_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header="infer_kv.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(infer_[a-z0-9_]+)\s*\(", text)))


def test_one_c_header_one_library():
    assert sorted(fn for fn in os.listdir(os.path.join(ROOT, "include")) if fn.endswith(".h")) == ["infer_kv.h"]


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("infer_kv_append_bf16", "infer_paged_decode_bf16", "infer_paged_decode_workspace_bytes"):
        assert must in names


def test_library_exports_every_declared_symbol_and_binding_covers_it():
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    for name in _lib.SIGNATURES:
        assert name in declared_functions(), f"{name} bound but not declared in include/"


def test_host_only_entry_points():
    lib = _lib.load()
    assert lib.infer_kv_version() == b"0.3"
    assert b"workspace" in lib.infer_kv_strerror(-3)
    assert lib.infer_paged_decode_workspace_bytes(64, 32, 8, 128) > 0
    assert lib.infer_paged_decode_workspace_bytes(64, 32, 8, 64) == 0        # head_dim not built
    assert lib.infer_paged_decode_workspace_bytes(64, 30, 8, 128) == 0       # Hq % Hkv != 0
    small = lib.infer_paged_decode_workspace_bytes(1, 32, 8, 128)
    assert lib.infer_paged_decode_workspace_bytes(512, 32, 8, 128) > small


def test_argument_errors_are_reported_before_anything_is_launched():
    lib = _lib.load()
    # null pointers / bad sizes are rejected by the host-side checks (no device is touched)
    assert lib.infer_kv_append_bf16(None, 1024, None, 1024, None, None, None, 4, 1024, 256, None) == -1
    assert lib.infer_kv_append_bf16(None, 1024, None, 1024, None, None, None, 0, 1024, 256, None) == 0
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    assert lib.infer_kv_append_bf16(p16, 1024, p16, 1024, p16, p16, p16, 4, 1020, 256, None) == -2   # dkv % 8
    assert lib.infer_kv_append_bf16(p16 + 2, 1024, p16, 1024, p16, p16, p16, 4, 1024, 256, None) == -2
    assert lib.infer_kv_gather_bf16(None, None, 5, 1024, 256, 4, None, None) == -1
    assert lib.infer_kv_gather_bf16(None, None, 0, 1024, 256, 4, None, None) == 0
    assert lib.infer_kv_gather_bf16(p16, p16, 5, 1020, 256, 4, p16, None) == -2
    assert lib.infer_paged_decode_bf16(None, 0, None, None, 0, 0, None, 0, None, 0, 1, None,
                                       1, 32, 8, 128, 256, 4, 1.0, 0, None, 0, None) == -1
    # the combined decode call rejects what its second launch would reject before the first is enqueued
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16 + 2, 4096, p16, 1, 1, p16,
                                       1, 32, 8, 128, 256, 4, 1.0, 0, p16, 1 << 30, None) == -2  # out not 8-byte aligned
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4095, p16, 1, 1, p16,
                                       1, 32, 8, 128, 256, 4, 1.0, 0, p16, 1 << 30, None) == -1  # out rows overlap
    # a block table without columns, a row stride shorter than the row, a negative split count, and a
    # batch whose step count would not fit 32 bits
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 1, 0, p16,
                                       1, 32, 8, 128, 256, 4, 1.0, 0, p16, 1 << 30, None) == -1
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 3, 4, p16,
                                       2, 32, 8, 128, 256, 4, 1.0, 0, p16, 1 << 30, None) == -1
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 4, 4, p16,
                                       2, 32, 8, 128, 256, 4, 1.0, -1, p16, 1 << 30, None) == -1
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 1 << 23, 1 << 23, p16,
                                       1 << 10, 32, 8, 128, 256, 4, 1.0, 0, p16, 1 << 40, None) == -1
    # the lengths array is required where it is an argument; the uniform form takes a non-negative length,
    # an output it can store to and a workspace for the shapes that need one
    assert lib.infer_paged_decode_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 4, 4, None,
                                       2, 32, 8, 128, 256, 4, 1.0, 0, p16, 1 << 30, None) == -1
    assert lib.infer_paged_decode_uniform_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 4, 4, -1,
                                               2, 32, 8, 128, 256, 4, 1.0, p16, 1 << 30, None) == -1
    assert lib.infer_paged_decode_uniform_bf16(p16, 4096, p16, p16, 262144, 1024, p16 + 2, 4096, p16, 4, 4, 100,
                                               2, 32, 8, 128, 256, 4, 1.0, p16, 1 << 30, None) == -2
    assert lib.infer_paged_decode_uniform_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 4, 4, 100,
                                               2, 32, 8, 128, 256, 4, 1.0, p16, 64, None) == -3
    assert lib.infer_paged_decode_uniform_bf16(p16, 4096, p16, p16, 262144, 1024, p16, 4096, p16, 4, 4, 100,
                                               2, 32, 8, 64, 256, 4, 1.0, p16, 1 << 30, None) == -4   # head_dim
    # prefill: the scale must be positive (the row maximum is taken before scaling)
    for bad_scale in (0.0, -0.1, float("nan")):
        assert lib.infer_paged_prefill_bf16(p16, 4096, p16, p16, 262144, 1024, 1024, p16, 4096, p16, p16, p16, 4, 4,
                                            1, 16, 32, 8, 128, 256, 4, bad_scale, 1, None) == -1
    assert lib.infer_paged_decode_merge_bf16(p16 + 4, 4096, p16, 1, 32, 8, 128, p16, 1 << 30, None) == -2
    with pytest.raises(RuntimeError, match="workspace too small"):
        _lib.check(-3, "x")
