"""Paged varlen causal prefill attention on the GPU against the fp32 CPU oracle
(oracle/paged_ref.varlen_prefill_ref).  Bar: bf16 output, max abs error <= 2e-2."""
import numpy as np
import pytest
import torch

from infer_amd import ops, workloads
from infer_amd.attention import Attention
from infer_amd.context import reset_context, set_context
from oracle import paged_ref
from tests.helpers import ATTN_ATOL, bits, f32

pytestmark = pytest.mark.gpu


def run_paged(wl):
    """Reference step order (infer/ops/attention.py:108-116): append, then attend over the cache."""
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    out = ops.flash_attn_varlen_func(wl.q, kc, vc, max_seqlen_q=wl.max_seqlen_q, cu_seqlens_q=wl.cu_seqlens_q,
                                     max_seqlen_k=wl.max_seqlen_k, cu_seqlens_k=wl.cu_seqlens_k,
                                     softmax_scale=wl.scale, causal=True, block_table=wl.block_table)
    torch.cuda.synchronize()
    return out, kc, vc


def oracle_paged(wl, kc, vc):
    return paged_ref.varlen_prefill_ref(bits(wl.q), bits(kc), bits(vc), wl.cu_seqlens_q.cpu().numpy(),
                                        wl.cu_seqlens_k.cpu().numpy(), wl.scale,
                                        block_table=wl.block_table.cpu().numpy())


def test_cfg3_prefix_cached_prefill(gpu):
    wl = workloads.cfg3().to(gpu)
    out, kc, vc = run_paged(wl)
    want = oracle_paged(wl, kc, vc)
    err = float(np.abs(f32(out) - want).max())
    print("cfg3 prefill max abs err", err)
    assert np.isfinite(f32(out)).all() and err <= ATTN_ATOL


@pytest.mark.parametrize("hq,hkv", [(8, 8), (16, 8), (32, 8), (64, 8), (8, 2), (16, 1), (24, 8), (5, 1), (12, 2), (7, 1), (12, 1), (10, 1)])
def test_small_shapes_with_and_without_prefix(gpu, hq, hkv):
    wl = workloads.make_prefill_workload("p", [1, 15, 16, 17, 33, 300, 257, 600], [0, 0, 0, 0, 0, 256, 256, 512],
                                         hq, hkv, seed=hq + hkv, pad_fraction=0.1).to(gpu)
    out, kc, vc = run_paged(wl)
    assert np.abs(f32(out) - oracle_paged(wl, kc, vc)).max() <= ATTN_ATOL


def test_row_maximum_covers_every_key_of_a_step(gpu):
    """One key per prompt whose score lies some 350 log2 units above all others, at each of the 32
    positions of a step in turn: every query behind it gives it weight 1.  A running maximum taken over
    part of a step only leaves the exponential of that key to overflow."""
    n = 32
    wl = workloads.make_prefill_workload("spike", [96] * n, [0] * n, 16, 8, seed=12, pad_fraction=0.0).to(gpu)
    g = wl.num_q_heads // wl.num_kv_heads
    for j in range(n):
        rows = slice(96 * j, 96 * (j + 1))
        wl.q[rows] = wl.q[96 * j]                                        # one query vector per head for the whole prompt
        q0 = wl.q[96 * j, ::g].float()
        c = 250.0 / (wl.scale * (q0 * q0).sum(dim=-1, keepdim=True))
        wl.k_new[96 * j + 32 + j] = (c * q0).to(torch.bfloat16)           # key 32 + j of prompt j
    out, kc, vc = run_paged(wl)
    got, want = f32(out), oracle_paged(wl, kc, vc)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= ATTN_ATOL
    for j in range(n):                                                   # queries at and behind the key return its value row
        p = 96 * j + 32 + j
        assert np.array_equal(got[p:96 * (j + 1), ::g], np.broadcast_to(f32(wl.v_new[p]), (96 * (j + 1) - p, 8, 128)))


@pytest.mark.parametrize("direction", [1, -1])
def test_scores_that_rise_or_fall_along_the_sequence(gpu, direction):
    """Keys that are multiples of one query vector shared by a prompt, the factor rising (or falling) by a
    fixed amount per token: the running maximum of every query row grows at every step, or is set by key 0
    and never again, with the later keys hundreds of log2 units below it."""
    lens = [300, 97, 640]
    wl = workloads.make_prefill_workload("ramp", lens, [0, 0, 256], 16, 8, seed=14, pad_fraction=0.0).to(gpu)
    g = wl.num_q_heads // wl.num_kv_heads
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    aq = 0
    for i, (n, c) in enumerate(zip(lens, wl.cached)):
        wl.q[aq:aq + n - c] = wl.q[aq]
        q0 = wl.q[aq, ::g].float()
        unit = q0 / (wl.scale * (q0 * q0).sum(dim=-1, keepdim=True))
        for pos in range(n):
            f = 0.5 * (pos if direction > 0 else -pos)
            blk = int(wl.block_table[i, pos // wl.block_size])
            kc[blk, pos % wl.block_size] = (f * unit).to(torch.bfloat16)
        aq += n - c
    out = ops.flash_attn_varlen_func(wl.q, kc, vc, max_seqlen_q=wl.max_seqlen_q, cu_seqlens_q=wl.cu_seqlens_q,
                                     max_seqlen_k=wl.max_seqlen_k, cu_seqlens_k=wl.cu_seqlens_k,
                                     softmax_scale=wl.scale, causal=True, block_table=wl.block_table)
    torch.cuda.synchronize()
    got, want = f32(out), oracle_paged(wl, kc, vc)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= ATTN_ATOL


@pytest.mark.parametrize("bs", [32, 64, 512])
def test_block_sizes(gpu, bs):
    wl = workloads.make_prefill_workload("p", [70, 200, 5], [bs if bs <= 64 else 0, 0, 0], 16, 8, bs=bs, seed=bs,
                                         pad_fraction=0.0).to(gpu)
    out, kc, vc = run_paged(wl)
    assert np.abs(f32(out) - oracle_paged(wl, kc, vc)).max() <= ATTN_ATOL


@pytest.mark.parametrize("cached", [3008, 16512])
def test_long_block_table_rows(gpu, cached):
    """Sequences of 95 and 518 blocks (block size 32): the kernel keeps the first 512 block ids of a
    sequence in LDS and looks the rest up in memory; tiles far into the ring's steady state."""
    wl = workloads.make_prefill_workload("p", [cached + 40, 100], [cached, 0], 4, 2, bs=32, seed=cached,
                                         pad_fraction=0.0).to(gpu)
    out, kc, vc = run_paged(wl)
    assert np.abs(f32(out) - oracle_paged(wl, kc, vc)).max() <= ATTN_ATOL


@pytest.mark.parametrize("seed", range(8))
def test_random_ragged_batches(gpu, seed):
    """Random head shapes, block sizes, lengths and cached prefixes (prefix lengths are whole blocks, as
    the block manager hands them out): every path of the tile ring (first, steady, last partial tile,
    several query blocks per workgroup) against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    hkv = int(rng.choice([1, 2, 4, 8]))
    hq = hkv * int(rng.choice([1, 2, 3, 4, 6, 8]))
    bs = int(rng.choice([32, 64, 256]))
    nseq = int(rng.integers(1, 7))
    lens, cached = [], []
    for _ in range(nseq):
        c = int(rng.integers(0, 4)) * bs if rng.random() < 0.5 else 0
        n = c + int(rng.integers(1, 400))
        lens.append(n); cached.append(c)
    wl = workloads.make_prefill_workload("r", lens, cached, hq, hkv, bs=bs, seed=seed, pad_fraction=0.05).to(gpu)
    out, kc, vc = run_paged(wl)
    err = np.abs(f32(out) - oracle_paged(wl, kc, vc)).max()
    assert err <= ATTN_ATOL, (hq, hkv, bs, lens, cached, float(err))


def test_packed_keys_without_block_table_equals_causal_sdpa(gpu):
    """No prefix cached: K and V are the packed new rows and sq == sk, which reduces to
    scaled_dot_product_attention(is_causal=True), the convention of the reference's own attention
    test (test/op.py:278-283, atol 2e-2)."""
    g = torch.Generator().manual_seed(5)
    lens = [64, 1, 100, 513]
    hq, hkv, d = 32, 8, 128
    t = sum(lens)
    q = torch.randn((t, hq, d), generator=g).to(torch.bfloat16).to(gpu)
    k = torch.randn((t, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    v = torch.randn((t, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    cu = torch.tensor(np.cumsum([0] + lens), dtype=torch.int32, device=gpu)
    out = ops.flash_attn_varlen_func(q, k, v, max_seqlen_q=max(lens), cu_seqlens_q=cu, max_seqlen_k=max(lens),
                                     cu_seqlens_k=cu, softmax_scale=d ** -0.5, causal=True)
    at = 0
    for n in lens:
        qq = q[at:at + n].float().cpu().permute(1, 0, 2)
        kk = k[at:at + n].float().cpu().permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        vv = v[at:at + n].float().cpu().permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        want = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, is_causal=True).permute(1, 0, 2)
        assert (out[at:at + n].float().cpu() - want).abs().max() <= ATTN_ATOL
        at += n
    # strided K/V views of a fused qkv projection (infer/models/Qwen3.py:110-111) give the same result
    qkv = torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], dim=1)
    _, k2, v2 = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)
    out2 = ops.flash_attn_varlen_func(q, k2.view(t, hkv, d), v2.view(t, hkv, d), max_seqlen_q=max(lens),
                                      cu_seqlens_q=cu, max_seqlen_k=max(lens), cu_seqlens_k=cu, causal=True)
    assert torch.equal(out, out2)


def test_one_query_per_sequence_equals_decode(gpu):
    wl = workloads.make_decode_workload("d", [37, 256, 700, 1023], 16, 8, nblk=16, seed=2).to(gpu)
    dec = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), wl.k_cache, wl.v_cache, cache_seqlens=wl.context_lens,
                                      block_table=wl.block_table, softmax_scale=wl.scale)[:, 0]
    cu_q = torch.arange(5, dtype=torch.int32, device=gpu)
    cu_k = torch.tensor(np.cumsum([0] + wl.lengths), dtype=torch.int32, device=gpu)
    pre = ops.flash_attn_varlen_func(wl.q, wl.k_cache, wl.v_cache, max_seqlen_q=1, cu_seqlens_q=cu_q,
                                     max_seqlen_k=1023, cu_seqlens_k=cu_k, softmax_scale=wl.scale, causal=True,
                                     block_table=wl.block_table)
    assert (pre.float() - dec.float()).abs().max() <= 4e-3     # two bf16 roundings of the same fp32 value


def test_stale_nan_beyond_length_is_ignored(gpu):
    wl = workloads.make_prefill_workload("p", [37, 300], [0, 256], 16, 8, seed=3, pad_fraction=0.0).to(gpu)
    for i, n in enumerate(wl.lengths):
        blk = int(wl.block_table[i, (n - 1) // 256])
        wl.k_cache[blk, n % 256:] = float("nan")
        wl.v_cache[blk, n % 256:] = float("nan")
    out, kc, vc = run_paged(wl)
    assert np.isfinite(f32(out)).all()
    assert np.abs(f32(out) - oracle_paged(wl, kc, vc)).max() <= ATTN_ATOL


def test_attention_module_prefill_then_decode(gpu):
    """The reference's module-level flow (infer/ops/attention.py:96-122) on one layer: a prefill step
    with a cached prefix, then a decode step for the same sequences."""
    wl = workloads.make_prefill_workload("m", [300, 70], [256, 0], 16, 8, seed=9, pad_fraction=0.0).to(gpu)
    att = Attention(16, 128, wl.scale, 8)
    att.k_cache, att.v_cache = wl.k_cache.clone(), wl.v_cache.clone()
    set_context(True, wl.cu_seqlens_q, wl.cu_seqlens_k, wl.max_seqlen_q, wl.max_seqlen_k, wl.slot_mapping, None,
                wl.block_table)
    o = att(wl.q.reshape(-1, 16 * 128), wl.k_new.reshape(-1, 8 * 128), wl.v_new.reshape(-1, 8 * 128))
    want = oracle_paged(wl, att.k_cache, att.v_cache)
    assert np.abs(f32(o).reshape(want.shape) - want).max() <= ATTN_ATOL
    # decode one more token per sequence
    g = torch.Generator().manual_seed(1)
    q1 = torch.randn((2, 16 * 128), generator=g).to(torch.bfloat16).to(gpu)
    k1 = torch.randn((2, 8 * 128), generator=g).to(torch.bfloat16).to(gpu)
    v1 = torch.randn((2, 8 * 128), generator=g).to(torch.bfloat16).to(gpu)
    lens = [n + 1 for n in wl.lengths]
    slots = torch.tensor([int(wl.block_table[i, (n - 1) // 256]) * 256 + (n - 1) % 256 for i, n in enumerate(lens)],
                         dtype=torch.int32, device=gpu)
    ctx = torch.tensor(lens, dtype=torch.int32, device=gpu)
    set_context(False, slot_mapping=slots, context_lens=ctx, block_tables=wl.block_table)
    o1 = att(q1, k1, v1)
    want1 = paged_ref.paged_decode_ref(bits(q1.view(2, 16, 128)), bits(att.k_cache), bits(att.v_cache),
                                       wl.block_table.cpu().numpy(), ctx.cpu().numpy(), wl.scale)
    assert np.abs(f32(o1).reshape(want1.shape) - want1).max() <= ATTN_ATOL
    reset_context()


def _packed_case(gpu, lens_q, lens_k, hq, hkv, seed):
    g = torch.Generator().manual_seed(seed)
    d = 128
    q = torch.randn((sum(lens_q), hq, d), generator=g).to(torch.bfloat16).to(gpu)
    k = torch.randn((sum(lens_k), hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    v = torch.randn((sum(lens_k), hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    cu_q = torch.tensor(np.cumsum([0] + lens_q), dtype=torch.int32, device=gpu)
    cu_k = torch.tensor(np.cumsum([0] + lens_k), dtype=torch.int32, device=gpu)
    return q, k, v, cu_q, cu_k


@pytest.mark.parametrize("hq,hkv", [(32, 8), (16, 8), (8, 8)])
def test_non_causal_sees_every_key(gpu, hq, hkv):
    """causal=False: every query sees all sk keys of its sequence, also with more keys than queries.
    Pinned twice: the oracle, and scaled_dot_product_attention without a mask on each sequence."""
    lens_q, lens_k = [40, 1, 130, 64], [100, 33, 130, 700]
    q, k, v, cu_q, cu_k = _packed_case(gpu, lens_q, lens_k, hq, hkv, seed=11)
    scale = 0.11
    out = ops.flash_attn_varlen_func(q, k, v, max_seqlen_q=max(lens_q), cu_seqlens_q=cu_q, max_seqlen_k=max(lens_k),
                                     cu_seqlens_k=cu_k, softmax_scale=scale, causal=False)
    want = paged_ref.varlen_prefill_ref(bits(q), bits(k), bits(v), cu_q.cpu().numpy(), cu_k.cpu().numpy(), scale,
                                        causal=False)
    assert np.abs(f32(out) - want).max() <= ATTN_ATOL
    aq = ak = 0
    for nq, nk in zip(lens_q, lens_k):
        qq = q[aq:aq + nq].float().cpu().permute(1, 0, 2)
        kk = k[ak:ak + nk].float().cpu().permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        vv = v[ak:ak + nk].float().cpu().permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        ref = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, scale=scale).permute(1, 0, 2)
        assert (out[aq:aq + nq].float().cpu() - ref).abs().max() <= ATTN_ATOL
        aq += nq
        ak += nk


def test_more_keys_than_queries_is_bottom_right_aligned(gpu):
    """sq < sk with packed keys: query i sees keys 0 .. i + (sk - sq), the alignment the prefix-cache
    branch relies on (infer/ops/attention.py:110-116)."""
    lens_q, lens_k = [5, 64, 1], [37, 64, 300]
    q, k, v, cu_q, cu_k = _packed_case(gpu, lens_q, lens_k, 16, 8, seed=12)
    out = ops.flash_attn_varlen_func(q, k, v, max_seqlen_q=max(lens_q), cu_seqlens_q=cu_q, max_seqlen_k=max(lens_k),
                                     cu_seqlens_k=cu_k, causal=True)
    want = paged_ref.varlen_prefill_ref(bits(q), bits(k), bits(v), cu_q.cpu().numpy(), cu_k.cpu().numpy(), 128 ** -0.5)
    assert np.abs(f32(out) - want).max() <= ATTN_ATOL
    # the single query of the last sequence sees all 300 keys: one softmax row
    s = (q[-1].float().cpu().view(8, 2, 128) @ k[-300:].float().cpu().permute(1, 2, 0)) * 128 ** -0.5
    ref = torch.softmax(s, -1) @ v[-300:].float().cpu().permute(1, 0, 2)
    assert (out[-1].float().cpu().view(8, 2, 128) - ref).abs().max() <= ATTN_ATOL


def test_more_queries_than_keys_gives_zero_rows_without_a_visible_key(gpu):
    """sq > sk (outside what the engine produces, since every query's own key is in the cache): with the
    bottom-right alignment the first sq - sk queries see no key at all.  Their rows are zeros (what
    flash-attn documents for a fully masked row); the others see keys 0 .. i - (sq - sk)."""
    lens_q, lens_k = [48, 70, 40], [16, 64, 40]
    q, k, v, cu_q, cu_k = _packed_case(gpu, lens_q, lens_k, 16, 8, seed=13)
    out = ops.flash_attn_varlen_func(q, k, v, max_seqlen_q=max(lens_q), cu_seqlens_q=cu_q, max_seqlen_k=max(lens_k),
                                     cu_seqlens_k=cu_k, causal=True)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    aq = ak = 0
    for nq, nk in zip(lens_q, lens_k):
        dead = max(nq - nk, 0)
        assert (got[aq:aq + dead] == 0).all()
        live = nq - dead                                    # the last `live` queries against the first nk keys, sq == sk form
        qq = q[aq + dead:aq + nq].float().cpu().permute(1, 0, 2)
        kk = k[ak:ak + nk].float().cpu().permute(1, 0, 2).repeat_interleave(2, 0)
        vv = v[ak:ak + nk].float().cpu().permute(1, 0, 2).repeat_interleave(2, 0)
        mask = torch.ones(live, nk, dtype=torch.bool).tril(diagonal=nk - live)
        ref = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, attn_mask=mask).permute(1, 0, 2)
        assert (got[aq + dead:aq + nq] - ref).abs().max() <= ATTN_ATOL
        aq += nq
        ak += nk


@pytest.mark.parametrize("scale", [0.02, 0.25])
def test_softmax_scale_is_honoured(gpu, scale):
    wl = workloads.make_prefill_workload("p", [90, 300, 700], [0, 256, 512], 32, 8, seed=21, pad_fraction=0.0).to(gpu)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    out = ops.flash_attn_varlen_func(wl.q, kc, vc, max_seqlen_q=wl.max_seqlen_q, cu_seqlens_q=wl.cu_seqlens_q,
                                     max_seqlen_k=wl.max_seqlen_k, cu_seqlens_k=wl.cu_seqlens_k,
                                     softmax_scale=scale, causal=True, block_table=wl.block_table)
    want = paged_ref.varlen_prefill_ref(bits(wl.q), bits(kc), bits(vc), wl.cu_seqlens_q.cpu().numpy(),
                                        wl.cu_seqlens_k.cpu().numpy(), scale, block_table=wl.block_table.cpu().numpy())
    assert np.abs(f32(out) - want).max() <= ATTN_ATOL


def test_query_rows_as_views_of_the_qkv_projection(gpu):
    """Q is a column slice of the fused qkv matrix in the reference (infer/models/Qwen3.py:110-111): its
    rows are (Hq + 2 Hkv) * D apart.  Same bits as with a contiguous copy."""
    wl = workloads.make_prefill_workload("p", [70, 513, 33], [0, 256, 0], 32, 8, seed=22, pad_fraction=0.0).to(gpu)
    out, kc, vc = run_paged(wl)
    t, hq, d = wl.q.shape
    qkv = torch.randn((t, (hq + 16) * d), device=gpu).to(torch.bfloat16)
    qkv[:, :hq * d] = wl.q.reshape(t, -1)
    q_view = qkv.split([hq * d, 8 * d, 8 * d], dim=-1)[0].view(t, hq, d)
    assert not q_view.is_contiguous()
    out2 = ops.flash_attn_varlen_func(q_view, kc, vc, max_seqlen_q=wl.max_seqlen_q, cu_seqlens_q=wl.cu_seqlens_q,
                                      max_seqlen_k=wl.max_seqlen_k, cu_seqlens_k=wl.cu_seqlens_k,
                                      softmax_scale=wl.scale, causal=True, block_table=wl.block_table)
    assert torch.equal(out, out2)
