"""infer::KVCachePool<T> handing its views to the HIP kernels (tests/cpp/test_kvcache_pool_gpu.cpp, built
by infer_amd/csrc/Makefile): the C++ program builds a pool over device storage, appends through
infer_kv_append_bf16 at slots derived from the views' block tables and attends through
infer_paged_decode_bf16 with the views' pointers and strides.  Here its dumped inputs and results are
checked against the CPU oracle: caches bit-exact, attention within 2e-2."""
import os
import subprocess

import numpy as np
import pytest

from oracle import paged_ref
from tests.helpers import ATTN_ATOL

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_views_feed_append_and_decode(gpu, tmp_path):
    exe = os.path.join(ROOT, "tests", "cpp", "test_kvcache_pool_gpu")
    assert os.path.exists(exe), "build it with `make -C infer_amd/csrc tests`"
    run = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout + run.stderr

    def load(name, dtype):
        return np.fromfile(os.path.join(tmp_path, name), dtype=dtype)
    b, hq, hkv, d, bs, nblk, cols, total = (int(x) for x in load("meta.i64", np.int64))
    q = load("q.u16", np.uint16).reshape(b, hq, d)
    out = load("out.u16", np.uint16).reshape(b, hq, d)
    k_rows = load("k_rows.u16", np.uint16).reshape(total, hkv, d)
    v_rows = load("v_rows.u16", np.uint16).reshape(total, hkv, d)
    k_layer = load("k_layer.u16", np.uint16).reshape(nblk, bs, hkv, d)
    v_layer = load("v_layer.u16", np.uint16).reshape(nblk, bs, hkv, d)
    table = load("table.i32", np.int32).reshape(b, cols)
    lens = load("lens.i32", np.int32)
    slots1, slots2 = load("slots1.i32", np.int32), load("slots2.i32", np.int32)
    # every token got exactly one slot over the two appends, all slots distinct
    assert ((slots1 >= 0) ^ (slots2 >= 0)).all()
    slots = np.where(slots1 >= 0, slots1, slots2)
    assert len(set(slots.tolist())) == total
    # caches: what the oracle's append leaves, on storage that started as 0xffff
    ek = np.full_like(k_layer, 0xffff)
    ev = np.full_like(v_layer, 0xffff)
    paged_ref.append_ref(k_rows, v_rows, ek, ev, slots1)
    paged_ref.append_ref(k_rows, v_rows, ek, ev, slots2)
    assert np.array_equal(k_layer, ek) and np.array_equal(v_layer, ev)
    # attention through the pool's block tables
    want = paged_ref.paged_decode_ref(q, ek, ev, table, lens, d ** -0.5)
    got = paged_ref.bf16_to_f32(out)
    assert np.isfinite(got).all()
    assert float(np.abs(got - want).max()) <= ATTN_ATOL
