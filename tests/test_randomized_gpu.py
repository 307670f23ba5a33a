"""Randomized parity sweeps of the append and the decode op against the CPU oracle, from fixed seeds.

Each case draws head counts, block size, batch, lengths, split count (decode) or row width, row count,
source stride and slot pattern (append) from its seed, so the sweep covers combinations no hand-written
case names.  Bars as everywhere: append bit-exact, attention max abs error <= 2e-2 against fp32."""
import numpy as np
import pytest
import torch

from infer_amd import _lib, ops, workloads
from oracle import paged_ref
from tests.helpers import ATTN_ATOL, bits, f32, oracle_decode

pytestmark = pytest.mark.gpu

HEADS = [(32, 8), (16, 8), (40, 8), (8, 8), (4, 4), (12, 2), (64, 8), (16, 1), (128, 8), (32, 16)]


@pytest.mark.parametrize("seed", range(28))
def test_decode_random_case(gpu, seed):
    rng = np.random.default_rng(1000 + seed)
    hq, hkv = HEADS[rng.integers(len(HEADS))]
    bs = int(rng.choice([32, 64, 128, 256]))
    mode = rng.integers(4)
    if mode == 0:       # a few long sequences
        lens = rng.integers(1, 9000, size=int(rng.integers(1, 6)))
    elif mode == 1:     # many very short ones: spans that cover dozens of sequences
        lens = rng.integers(1, 90, size=int(rng.integers(50, 400)))
    elif mode == 2:
        lens = rng.integers(1, 1500, size=int(rng.integers(8, 80)))
    else:               # a few long among many tiny
        b = int(rng.integers(2, 40))
        lens = np.where(rng.random(b) < 0.3, rng.integers(2000, 5000, size=b), rng.integers(1, 40, size=b))
    lens = [int(x) for x in lens]
    while sum(lens) * hq > 2_500_000:        # keeps the CPU oracle to a fraction of a second
        lens = lens[:-1] if len(lens) > 1 else [lens[0] // 2]
    splits = int(rng.choice([0, 0, 1, 3, 7, 64, 200, 300, 1000]))
    wl = workloads.make_decode_workload(f"rnd{seed}", lens, hq, hkv, bs=bs, seed=seed).to(gpu)
    out = torch.empty_like(wl.q)
    ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, out,
                          split_workgroups=splits)
    torch.cuda.synchronize()
    got = f32(out)
    err = float(np.abs(got - oracle_decode(wl)).max())
    assert np.isfinite(got).all() and err <= ATTN_ATOL, (seed, hq, hkv, bs, len(lens), splits, err)
    if splits == 0:     # the entry point without a workspace runs the same kernels: same bits, or a clean refusal
        lib = _lib.load()
        nblk, _, _, d = wl.k_cache.shape
        again = torch.full_like(wl.q, float("nan"))
        rc = lib.infer_paged_decode_noalloc_bf16(
            wl.q.data_ptr(), wl.q.stride(0), wl.k_cache.data_ptr(), wl.v_cache.data_ptr(), wl.k_cache.stride(0),
            wl.k_cache.stride(1), again.data_ptr(), again.stride(0), wl.block_table.data_ptr(), wl.block_table.stride(0),
            wl.block_table.shape[1], wl.context_lens.data_ptr(), len(lens), hq, hkv, d, bs, nblk, float(wl.scale),
            torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert rc in (0, -3)
        if rc == 0:
            assert np.array_equal(bits(again), bits(out))


@pytest.mark.parametrize("seed", range(24))
def test_append_random_case(gpu, seed):
    rng = np.random.default_rng(seed)
    hkv = int(rng.choice([1, 2, 4, 8, 16, 5, 3]))
    d = int(rng.choice([128, 64, 8, 256, 40]))
    dkv = hkv * d
    bs = int(rng.choice([32, 256]))
    n = int(rng.integers(1, 700)) if seed % 3 else int(rng.integers(3073, 21000))     # every third case takes the ring shape
    nblk = int(rng.integers(1, 12)) if seed % 3 else n // bs + int(rng.integers(1, 9))
    slots_total = nblk * bs
    wide = int(rng.choice([0, 8, 128]))       # rows as views of a wider (fused) buffer
    g = torch.Generator().manual_seed(seed)
    kbuf = torch.randn(n, dkv + wide, generator=g).to(torch.bfloat16)
    vbuf = torch.randn(n, dkv + wide, generator=g).to(torch.bfloat16)
    k_cache = torch.randn(nblk, bs, hkv, d, generator=g).to(torch.bfloat16)
    v_cache = torch.randn(nblk, bs, hkv, d, generator=g).to(torch.bfloat16)
    take = min(n, slots_total)
    slots = np.full(n, -1, dtype=np.int64)
    slots[:take] = rng.permutation(slots_total)[:take]
    rng.shuffle(slots)
    bad = rng.random(n) < 0.1
    slots[bad] = rng.choice([-1, -7, slots_total, slots_total + 5], size=int(bad.sum()))
    # expectation from the oracle, which knows only the padding value: out-of-range slots count as padding
    ek, ev = bits(k_cache).copy(), bits(v_cache).copy()
    key_host = kbuf[:, wide:].reshape(n, hkv, d) if wide else kbuf.view(n, hkv, d)
    val_host = vbuf[:, :dkv].reshape(n, hkv, d)
    paged_ref.append_ref(bits(key_host.contiguous()), bits(val_host.contiguous()), ek, ev,
                         np.where((slots >= 0) & (slots < slots_total), slots, -1))
    kd, vd = kbuf.to(gpu), vbuf.to(gpu)
    key = kd[:, wide:].view(n, hkv, d) if wide else kd.view(n, hkv, d)
    val = vd[:, :dkv].view(n, hkv, d)
    kg, vg = k_cache.to(gpu), v_cache.to(gpu)
    if dkv % 8 or (dkv + wide) % 8 or wide % 8:
        with pytest.raises(RuntimeError):      # rows that are not 16-byte aligned are refused, not copied wrongly
            ops.store_kvcache(key, val, kg, vg, torch.from_numpy(slots.astype(np.int32)).to(gpu))
        return
    ops.store_kvcache(key, val, kg, vg, torch.from_numpy(slots.astype(np.int32)).to(gpu))
    torch.cuda.synchronize()
    assert np.array_equal(bits(kg), ek) and np.array_equal(bits(vg), ev), (seed, hkv, d, n, wide)


@pytest.mark.parametrize("seed", range(24))
def test_decode_uniform_length_random_case(gpu, seed):
    """The length as one host integer: shapes drawn on both sides of the rule that picks the single-kernel
    form (batch x KV heads x pieces / 8 workgroups against the compute units), odd lengths, every block size."""
    rng = np.random.default_rng(3000 + seed)
    hq, hkv = HEADS[rng.integers(len(HEADS))]
    bs = int(rng.choice([32, 64, 128, 256]))
    batch = int(rng.choice([1, 5, 31, 32, 60, 64, 100, 128, 250, 256, 300]))
    length = int(rng.integers(1, 3000))
    while batch * length * hq > 2_500_000:     # keeps the CPU oracle to a fraction of a second
        length = max(1, length // 2)
    wl = workloads.make_decode_workload(f"uni{seed}", [length] * batch, hq, hkv, bs=bs, seed=seed).to(gpu)
    out = torch.full_like(wl.q, 3.0)
    ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, length, wl.scale, out)
    torch.cuda.synchronize()
    got = f32(out)
    err = float(np.abs(got - oracle_decode(wl)).max())
    assert np.isfinite(got).all() and err <= ATTN_ATOL, (seed, hq, hkv, bs, batch, length, err)
