"""KV append on the GPU against the oracle: bit-exact (pure copy)."""
import numpy as np
import pytest
import torch

from infer_amd import ops, workloads
from oracle import paged_ref
from tests.helpers import assert_seeded_inputs, bits

pytestmark = pytest.mark.gpu


def run_both(key, value, k_cache, v_cache, slots):
    """Runs the HIP append on copies of the caches and the oracle on host copies; returns both."""
    kc, vc = k_cache.clone(), v_cache.clone()
    ops.store_kvcache(key, value, kc, vc, slots)
    torch.cuda.synchronize()
    ek, ev = bits(k_cache).copy(), bits(v_cache).copy()
    slots_host = slots.cpu().numpy()
    if int(slots_host.max(initial=-1)) < ek.shape[0] * ek.shape[1]:      # the oracle has no notion of a slot past the end
        paged_ref.append_ref(bits(key), bits(value), ek, ev, slots_host)
    return bits(kc), bits(vc), ek, ev


def test_cfg1_decode_rows(gpu):
    wl = workloads.cfg1().to(gpu)
    gk, gv, ek, ev = run_both(wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.slot_mapping)
    assert np.array_equal(gk, ek) and np.array_equal(gv, ev)
    # and the new rows really are where the block table says the newest token lives
    for i, n in enumerate(wl.lengths):
        blk = int(wl.block_table[i, (n - 1) // 256])
        assert np.array_equal(gk[blk, (n - 1) % 256], bits(wl.k_new)[i])


def test_cfg3_prefill_rows_with_padding(gpu):
    wl = workloads.cfg3()
    assert_seeded_inputs(wl, "cfg3")
    wl = wl.to(gpu)
    assert int((wl.slot_mapping < 0).sum()) > 0
    gk, gv, ek, ev = run_both(wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.slot_mapping)
    assert np.array_equal(gk, ek) and np.array_equal(gv, ev)


def test_strided_rows_from_fused_qkv(gpu):
    """K and V are views of one qkv projection (row stride (Hq + 2 Hkv) D), as in
    infer/models/Qwen3.py:110-111."""
    g = torch.Generator(device="cpu").manual_seed(3)
    hq, hkv, d, n = 32, 8, 128, 77
    qkv = torch.randn((n, (hq + 2 * hkv) * d), generator=g).to(torch.bfloat16).to(gpu)
    _, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
    k, v = k.view(n, hkv, d), v.view(n, hkv, d)
    assert not k.is_contiguous()
    cache = torch.randn((2, 6, 256, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    slots = torch.randperm(6 * 256, generator=g)[:n].to(torch.int32).to(gpu)
    gk, gv, ek, ev = run_both(k, v, cache[0], cache[1], slots)
    assert np.array_equal(gk, ek) and np.array_equal(gv, ev)


@pytest.mark.parametrize("hkv,d", [(1, 64), (2, 128), (4, 128), (8, 64), (8, 128), (16, 128), (3, 40)])
def test_row_widths(gpu, hkv, d):
    g = torch.Generator(device="cpu").manual_seed(hkv * 131 + d)
    n, nblk, bs = 53, 3, 64
    key = torch.randn((n, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    val = torch.randn((n, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    kc = torch.randn((nblk, bs, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    vc = torch.randn((nblk, bs, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    slots = torch.randperm(nblk * bs, generator=g)[:n].to(torch.int32)
    slots[::7] = -1
    gk, gv, ek, ev = run_both(key, val, kc, vc, slots.to(gpu))
    assert np.array_equal(gk, ek) and np.array_equal(gv, ev)


@pytest.mark.parametrize("hkv,d,n", [(8, 128, 3073), (8, 128, 20011), (4, 128, 40000), (16, 128, 9001), (8, 64, 5000),
                                     (3, 40, 5000)])
def test_many_rows_take_the_ring_shape(gpu, hkv, d, n):
    """Above 3072 rows the append runs as a fixed grid of wavefronts that each keep a ring of rows in
    registers.  Covers: the first row count of that shape, counts that make every wavefront go round
    its ring more than once (20,011 rows of 2 KiB; 40,000 of 1 KiB; 9,001 of 4 KiB), a width the ring
    is not built for (falls back to one wavefront per row), strided rows out of a fused qkv
    projection, padding and out-of-range slots in between."""
    g = torch.Generator(device="cpu").manual_seed(hkv * 977 + d + n)
    width = hkv * d
    nblk = (n + 255) // 256 + 3
    qkv = torch.randn((n, 3 * width + 16), generator=g).to(torch.bfloat16).to(gpu)
    key, val = qkv[:, 8:8 + width].view(n, hkv, d), qkv[:, 8 + width:8 + 2 * width].view(n, hkv, d)
    assert not key.is_contiguous()
    kc = torch.randn((nblk, 256, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    vc = torch.randn((nblk, 256, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    slots = torch.randperm(nblk * 256, generator=g)[:n].to(torch.int32)
    slots[::13] = -1
    skipped = slots.clone()
    slots[5::101] = nblk * 256 + 7          # past the end of the cache: skipped like a padding row
    skipped[5::101] = -1                    # (the oracle knows only the padding value)
    gk, gv, _, _ = run_both(key, val, kc, vc, slots.to(gpu))
    ek, ev = bits(kc).copy(), bits(vc).copy()
    paged_ref.append_ref(bits(key), bits(val), ek, ev, skipped.numpy())
    assert np.array_equal(gk, ek) and np.array_equal(gv, ev)


def test_all_padding_and_empty(gpu):
    hkv, d = 8, 128
    kc = torch.zeros((2, 256, hkv, d), dtype=torch.bfloat16, device=gpu)
    vc = torch.zeros_like(kc)
    key = torch.ones((5, hkv, d), dtype=torch.bfloat16, device=gpu)
    ops.store_kvcache(key, key, kc, vc, torch.full((5,), -1, dtype=torch.int32, device=gpu))
    ops.store_kvcache(key[:0], key[:0], kc, vc, torch.zeros((0,), dtype=torch.int32, device=gpu))
    torch.cuda.synchronize()
    assert not kc.any() and not vc.any()


def test_out_of_range_slot_is_skipped(gpu):
    hkv, d = 8, 128
    kc = torch.zeros((1, 256, hkv, d), dtype=torch.bfloat16, device=gpu)
    vc = torch.zeros_like(kc)
    key = torch.ones((3, hkv, d), dtype=torch.bfloat16, device=gpu)
    slots = torch.tensor([255, 256, 1 << 30], dtype=torch.int32, device=gpu)
    ops.store_kvcache(key, key, kc, vc, slots)
    torch.cuda.synchronize()
    assert bool(kc[0, 255].eq(1).all()) and int(kc.ne(0).sum()) == hkv * d


def test_scatter_then_gather_roundtrip_full_size(gpu):
    """Size-independent property at cfg3 scale: after the append, reading the caches back through
    slot_mapping returns exactly the appended rows, and every other cache row is untouched."""
    wl = workloads.cfg3().to(gpu)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    torch.cuda.synchronize()
    valid = wl.slot_mapping >= 0
    rows = wl.slot_mapping[valid].long()
    width = wl.num_kv_heads * wl.head_dim
    assert torch.equal(kc.view(-1, width)[rows], wl.k_new[valid].reshape(-1, width))
    assert torch.equal(vc.view(-1, width)[rows], wl.v_new[valid].reshape(-1, width))
    untouched = torch.ones(kc.shape[0] * kc.shape[1], dtype=torch.bool, device=gpu)
    untouched[rows] = False
    assert torch.equal(kc.view(-1, width)[untouched], wl.k_cache.view(-1, width)[untouched])
    assert torch.equal(vc.view(-1, width)[untouched], wl.v_cache.view(-1, width)[untouched])


def test_gather_is_the_inverse_of_the_append(gpu):
    """ops.gather_kvcache hands out a sequence as the dense [len, Hkv, D] tensor the reference's pool getters
    promise: bit-exact against the oracle's gather on every sequence of the prefill configuration after its
    append, and equal to the rows that were appended."""
    wl = workloads.cfg3().to(gpu)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    torch.cuda.synchronize()
    hk, table = bits(kc), wl.block_table.cpu().numpy()
    new_rows = wl.k_new[wl.row_of_query]                      # the appended rows in sequence order
    at = 0
    for i, (n, c) in enumerate(zip(wl.lengths, wl.cached)):
        dense = ops.gather_kvcache(kc, wl.block_table[i].contiguous(), n)
        torch.cuda.synchronize()
        assert dense.shape == (n, wl.num_kv_heads, wl.head_dim)
        assert np.array_equal(bits(dense), paged_ref.gather_sequence(hk, table[i], n))
        assert torch.equal(dense[c:], new_rows[at:at + n - c])
        at += n - c
    assert ops.gather_kvcache(vc, wl.block_table[0].contiguous(), 0).shape[0] == 0
    # a corrupt table entry is clamped into the pool instead of read out of bounds
    bad = torch.tensor([10 ** 6, -5], dtype=torch.int32, device=gpu)
    got = ops.gather_kvcache(kc, bad, 300)
    torch.cuda.synchronize()
    assert torch.equal(got[:256], kc[kc.shape[0] - 1]) and torch.equal(got[256:], kc[0, :44])
