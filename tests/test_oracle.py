"""Pins the CPU oracle (oracle/paged_ref.py, oracle/torch_path.py) without a GPU.

The reference ships no golden vector for this path, so every function is checked against things
the mathematics fixes: an independent formulation, closed forms, invariants and a scalar brute
force on tiny inputs - each chosen so that a plausible slip (wrong head map, wrong block index,
missing scale, transposed operand, off-by-one in the length or the causal mask) fails one."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from infer_amd import workloads
from oracle import paged_ref, torch_path
from tests.helpers import bits, oracle_decode


# ----------------------------------------------------------------------------- bf16 helpers

def test_bf16_widening_matches_torch_for_every_bit_pattern():
    u = np.arange(65536, dtype=np.uint16)
    mine = paged_ref.bf16_to_f32(u)
    theirs = torch.from_numpy(u.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(mine.view(np.uint32), theirs.view(np.uint32))


def test_bf16_rounding_matches_torch_including_ties():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-20, 20, 200000)
    ties = (rng.integers(0, 1 << 16, 5000).astype(np.uint32) << 16) | np.uint32(0x8000)   # exactly halfway
    x = np.concatenate([x, ties.view(np.float32), np.array([0.0, -0.0, np.inf, -np.inf], np.float32)])
    x = x[np.isfinite(x) | np.isinf(x)]
    mine = paged_ref.f32_to_bf16(x)
    theirs = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(mine, theirs)


# ----------------------------------------------------------------------------- append

def _append_case(seed, n=40, hkv=8, d=128, nblk=3, bs=64, pad_every=5, strided=False):
    rng = np.random.default_rng(seed)
    width = hkv * d
    if strided:   # rows are slices of a wider buffer, as K/V are slices of a fused qkv projection
        big = rng.integers(0, 1 << 16, (n, 3 * width), dtype=np.uint16)
        key = big[:, width:2 * width].reshape(n, hkv, d)
        val = big[:, 2 * width:].reshape(n, hkv, d)
    else:
        key = rng.integers(0, 1 << 16, (n, hkv, d), dtype=np.uint16)
        val = rng.integers(0, 1 << 16, (n, hkv, d), dtype=np.uint16)
    kc = rng.integers(0, 1 << 16, (nblk, bs, hkv, d), dtype=np.uint16)
    vc = rng.integers(0, 1 << 16, (nblk, bs, hkv, d), dtype=np.uint16)
    slots = rng.permutation(nblk * bs)[:n].astype(np.int32)
    if pad_every:
        slots[::pad_every] = -1
    return key, val, kc, vc, slots


@pytest.mark.parametrize("strided", [False, True])
def test_append_equals_fancy_index_copy_and_leaves_other_rows_alone(strided):
    key, val, kc, vc, slots = _append_case(1, strided=strided)
    k0, v0 = kc.copy(), vc.copy()
    paged_ref.append_ref(key, val, kc, vc, slots)
    width = key.shape[1] * key.shape[2]
    valid = slots >= 0
    ek, ev = k0.reshape(-1, width).copy(), v0.reshape(-1, width).copy()
    ek[slots[valid]] = key.reshape(len(slots), width)[valid]        # independent formulation
    ev[slots[valid]] = val.reshape(len(slots), width)[valid]
    assert np.array_equal(kc.reshape(-1, width), ek) and np.array_equal(vc.reshape(-1, width), ev)
    untouched = np.ones(ek.shape[0], bool)
    untouched[slots[valid]] = False
    assert np.array_equal(kc.reshape(-1, width)[untouched], k0.reshape(-1, width)[untouched])
    assert not np.array_equal(kc, k0)
    # K rows never land in the V cache and vice versa
    assert np.array_equal(vc.reshape(-1, width)[slots[valid]], val.reshape(len(slots), width)[valid])


def test_append_matches_torch_index_copy():
    key, val, kc, vc, slots = _append_case(2)
    tk = torch.from_numpy(kc.view(np.int16).copy())
    tv = torch.from_numpy(vc.view(np.int16).copy())
    torch_path.append_torch(torch.from_numpy(key.view(np.int16)), torch.from_numpy(val.view(np.int16)), tk, tv,
                            torch.from_numpy(slots))
    paged_ref.append_ref(key, val, kc, vc, slots)
    assert np.array_equal(tk.numpy().view(np.uint16), kc) and np.array_equal(tv.numpy().view(np.uint16), vc)


def test_append_all_padding_is_a_no_op():
    key, val, kc, vc, slots = _append_case(3)
    k0 = kc.copy()
    paged_ref.append_ref(key, val, kc, vc, np.full_like(slots, -1))
    assert np.array_equal(kc, k0)


# ----------------------------------------------------------------------------- decode

def tiny(seed=0, lengths=(1, 5, 64, 70), hq=4, hkv=2, d=16, bs=32, nblk=12):
    return workloads.make_decode_workload("tiny", list(lengths), hq, hkv, d=d, bs=bs, nblk=nblk, seed=seed)


def test_decode_matches_scalar_bruteforce():
    wl = tiny()
    want = paged_ref.paged_decode_bruteforce(bits(wl.q), bits(wl.k_cache), bits(wl.v_cache),
                                             wl.block_table.numpy(), wl.context_lens.numpy(), wl.scale)
    got = oracle_decode(wl)
    assert np.abs(got - want).max() < 2e-6


def test_decode_bruteforce_catches_a_wrong_head_map():
    """The brute force addresses head h // G directly; a vectorised version that used h % Hkv would
    differ - make sure the two head maps really give different numbers on this input, so the
    agreement above means something."""
    wl = tiny(hq=4, hkv=2)
    good = oracle_decode(wl)
    swapped = paged_ref.paged_decode_ref(bits(wl.q)[:, [0, 2, 1, 3]], bits(wl.k_cache), bits(wl.v_cache),
                                         wl.block_table.numpy(), wl.context_lens.numpy(), wl.scale)[:, [0, 2, 1, 3]]
    assert np.abs(good - swapped).max() > 1e-3


def test_decode_single_token_returns_v():
    wl = tiny(lengths=(1, 1))
    got = oracle_decode(wl)
    for i in range(2):
        v0 = paged_ref.bf16_to_f32(bits(wl.v_cache)[int(wl.block_table[i, 0]), 0])     # [Hkv, D]
        assert np.array_equal(got[i], np.repeat(v0, 2, axis=0))


def test_decode_equal_keys_give_mean_of_values():
    wl = tiny(lengths=(37, 64))
    wl.k_cache[:] = wl.k_cache[0, 0]
    got = oracle_decode(wl)
    for i, n in enumerate(wl.lengths):
        rows = torch.cat([wl.v_cache[int(b)] for b in wl.block_table[i, : (n + 31) // 32]])[:n].float()
        assert np.abs(got[i] - np.repeat(rows.mean(0).numpy(), 2, axis=0)).max() < 1e-5


def test_decode_is_invariant_under_physical_block_permutation():
    wl = tiny(lengths=(70, 33, 5))
    a = oracle_decode(wl)
    nblk = wl.k_cache.shape[0]
    perm = torch.randperm(nblk, generator=torch.Generator().manual_seed(4))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nblk)
    wl2 = tiny(lengths=(70, 33, 5))
    wl2.k_cache, wl2.v_cache = wl.k_cache[perm], wl.v_cache[perm]
    wl2.block_table = torch.where(wl.block_table >= 0, inv[wl.block_table.clamp(min=0).long()].int(), wl.block_table)
    assert np.array_equal(a, oracle_decode(wl2))


def test_decode_ignores_everything_past_the_length_and_unused_table_entries():
    wl = tiny(lengths=(5, 33))
    a = oracle_decode(wl)
    for i, n in enumerate(wl.lengths):
        blk = int(wl.block_table[i, (n - 1) // 32])
        wl.k_cache[blk, n % 32 or 32:] = float("nan")
        wl.v_cache[blk, n % 32 or 32:] = float("nan")
    wl.block_table[wl.block_table < 0] = 10 ** 6
    assert np.array_equal(a, oracle_decode(wl))


def test_decode_zero_length_row_is_zero():
    wl = tiny(lengths=(5, 9))
    wl.context_lens[0] = 0
    got = oracle_decode(wl)
    assert not got[0].any() and got[1].any()


@pytest.mark.parametrize("hq,hkv", [(16, 8), (32, 8), (8, 8), (8, 1)])
def test_decode_matches_the_reference_torch_attention_on_gathered_keys(hq, hkv):
    """Second, independently written formulation: gather + F.scaled_dot_product_attention
    (the attention of infer/ops/attention.py:64-71), tolerance far below the 2e-2 bar."""
    wl = workloads.make_decode_workload("sdpa", [37, 256, 300], hq, hkv, d=128, bs=256, nblk=8, seed=hq + hkv)
    a = oracle_decode(wl)
    b = torch_path.paged_decode_torch(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale).numpy()
    assert np.abs(a - b).max() < 1e-5


def test_decode_scale_is_applied():
    wl = tiny(lengths=(40,))
    a = oracle_decode(wl)
    wl.scale = wl.scale * 2
    assert np.abs(a - oracle_decode(wl)).max() > 1e-3


# ----------------------------------------------------------------------------- prefill

def _sdpa_masked(q, k, v, scale, mask):
    # q [sq, Hq, D], k/v [sk, Hkv, D] float -> [sq, Hq, D]
    g = q.shape[1] // k.shape[1]
    k = k.permute(1, 0, 2).repeat_interleave(g, 0)
    v = v.permute(1, 0, 2).repeat_interleave(g, 0)
    return F.scaled_dot_product_attention(q.permute(1, 0, 2), k, v, attn_mask=mask, scale=scale).permute(1, 0, 2)


def test_prefill_without_prefix_equals_causal_sdpa():
    """sq == sk reduces to is_causal=True, the convention of test/op.py:278-283."""
    g = torch.Generator().manual_seed(0)
    lens = [7, 33, 1]
    hq, hkv, d = 4, 2, 16
    q = torch.randn((sum(lens), hq, d), generator=g).to(torch.bfloat16)
    k = torch.randn((sum(lens), hkv, d), generator=g).to(torch.bfloat16)
    v = torch.randn((sum(lens), hkv, d), generator=g).to(torch.bfloat16)
    cu = np.cumsum([0] + lens).astype(np.int32)
    got = paged_ref.varlen_prefill_ref(bits(q), bits(k), bits(v), cu, cu, d ** -0.5)
    at = 0
    for n in lens:
        qq, kk, vv = q[at:at + n].float(), k[at:at + n].float(), v[at:at + n].float()
        rep = hq // hkv
        want = F.scaled_dot_product_attention(qq.permute(1, 0, 2), kk.permute(1, 0, 2).repeat_interleave(rep, 0),
                                              vv.permute(1, 0, 2).repeat_interleave(rep, 0), is_causal=True,
                                              scale=d ** -0.5).permute(1, 0, 2).numpy()
        assert np.abs(got[at:at + n] - want).max() < 1e-5
        at += n


def test_prefill_with_cached_prefix_uses_bottom_right_mask_and_the_block_table():
    wl = workloads.make_prefill_workload("p", [70, 40, 96], [32, 0, 64], 4, 2, d=16, bs=32, seed=1, pad_fraction=0.1)
    # put the new rows into the cache first (the reference appends before it attends)
    kc, vc = bits(wl.k_cache).copy(), bits(wl.v_cache).copy()
    paged_ref.append_ref(bits(wl.k_new), bits(wl.v_new), kc, vc, wl.slot_mapping.numpy())
    got = paged_ref.varlen_prefill_ref(bits(wl.q), kc, vc, wl.cu_seqlens_q.numpy(), wl.cu_seqlens_k.numpy(),
                                       wl.scale, block_table=wl.block_table.numpy())
    kcf = torch.from_numpy(paged_ref.bf16_to_f32(kc))
    vcf = torch.from_numpy(paged_ref.bf16_to_f32(vc))
    at = 0
    for i, (n, c) in enumerate(zip(wl.lengths, wl.cached)):
        sq = n - c
        blocks = wl.block_table[i, : (n + 31) // 32].long()
        kk = kcf[blocks].reshape(-1, 2, 16)[:n]
        vv = vcf[blocks].reshape(-1, 2, 16)[:n]
        mask = torch.arange(n)[None, :] <= (torch.arange(sq)[:, None] + c)
        want = _sdpa_masked(wl.q[at:at + sq].float(), kk, vv, wl.scale, mask).numpy()
        assert np.abs(got[at:at + sq] - want).max() < 1e-5
        at += sq
    # the appended rows are really what the last queries see: query i's own key is visible
    assert got.any()


def test_prefill_of_one_query_token_is_decode():
    wl = tiny(lengths=(40, 7))
    dec = oracle_decode(wl)
    cu_q = np.array([0, 1, 2], np.int32)
    cu_k = np.array([0, 40, 47], np.int32)
    pre = paged_ref.varlen_prefill_ref(bits(wl.q), bits(wl.k_cache), bits(wl.v_cache), cu_q, cu_k, wl.scale,
                                       block_table=wl.block_table.numpy())
    assert np.abs(pre - dec).max() < 1e-6


# ----------------------------------------------------------------------------- metadata

def test_slots_and_tables_agree_scatter_then_gather_restores_token_order():
    """Writing token t of every sequence at its slot and reading the sequence back through its
    block table returns the tokens in order (ties slot_mapping to block_table)."""
    bs = 16
    lengths, cached = [40, 16, 33], [16, 0, 32]
    tables = [[5, 2, 7], [0], [9, 1, 4]]
    cu_q, cu_k, max_q, max_k, slots = paged_ref.prefill_metadata_ref(lengths, cached, tables, bs)
    assert cu_q.tolist() == [0, 24, 40, 41] and cu_k.tolist() == [0, 40, 56, 89] and (max_q, max_k) == (24, 40)
    cache = np.full((10 * bs,), -1, np.int64)
    ids = np.concatenate([np.arange(c, n) + 1000 * i for i, (n, c) in enumerate(zip(lengths, cached))])
    cache[slots] = ids
    for i, (n, c, t) in enumerate(zip(lengths, cached, tables)):
        seq = np.concatenate([cache[b * bs:(b + 1) * bs] for b in t])[:n]
        assert np.array_equal(seq[c:], np.arange(c, n) + 1000 * i)
    # decode: the newest token's slot is the last position of the sequence
    dslots, ctx, padded = paged_ref.decode_metadata_ref(lengths, tables, bs)
    assert dslots.tolist() == [7 * bs + 7, 0 * bs + 15, 4 * bs + 0] and ctx.tolist() == lengths
    assert padded.tolist() == [[5, 2, 7], [0, -1, -1], [9, 1, 4]]


def test_workload_generator_is_consistent_with_the_metadata_closed_form():
    wl = workloads.cfg1()
    tables = [[int(x) for x in row if x >= 0] for row in wl.block_table.tolist()]
    slots, ctx, padded = paged_ref.decode_metadata_ref(wl.lengths, tables, 256)
    assert np.array_equal(slots, wl.slot_mapping.numpy()) and np.array_equal(ctx, wl.context_lens.numpy())
    assert np.array_equal(padded, wl.block_table.numpy())
    flat = [b for t in tables for b in t]
    assert len(set(flat)) == len(flat) == 9      # rows use disjoint blocks: 1 + 1 + 3 + 4


def test_cfg1_golden_fixture_is_reproduced_by_generator_and_oracle():
    """The committed fixture of the reference's CPU-runnable configuration: seeded inputs, caches
    after the append (bit-exact) and the oracle's attention output must not drift."""
    import json
    import os
    from tests.golden import make_cfg1_golden as G
    with open(os.path.join(os.path.dirname(G.__file__), "cfg1_golden.json")) as f:
        want = json.load(f)
    got = json.loads(json.dumps(G.build()))
    assert got["config"] == want["config"]
    assert got["inputs_sha256"] == want["inputs_sha256"]
    assert got["after_append_sha256"] == want["after_append_sha256"]
    for key in ("first8", "last8", "row_sums"):
        assert np.allclose(np.array(got["attention_out"][key]), np.array(want["attention_out"][key]), atol=2e-5)
