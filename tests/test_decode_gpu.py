"""Paged decode attention on the GPU against the fp32 CPU oracle.

Bar: max abs error of the bf16 output <= 2e-2 against the fp32 oracle (tests/helpers.ATTN_ATOL)."""
import numpy as np
import pytest
import torch

from infer_amd import ops, workloads
from tests.helpers import ATTN_ATOL, assert_seeded_inputs, bits, f32, oracle_decode

pytestmark = pytest.mark.gpu


def gpu_decode(wl, splits=None):
    if splits is None:
        out = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), wl.k_cache, wl.v_cache,
                                          cache_seqlens=wl.context_lens, block_table=wl.block_table,
                                          softmax_scale=wl.scale, causal=True)[:, 0]
    else:   # the split count is an argument of the call; the library keeps no setting
        out = torch.empty_like(wl.q)
        ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, out,
                              split_workgroups=splits)
    torch.cuda.synchronize()
    return out


def check(wl, splits=None, atol=ATTN_ATOL):
    got = f32(gpu_decode(wl, splits))
    want = oracle_decode(wl)
    err = float(np.abs(got - want).max())
    assert np.isfinite(got).all()
    assert err <= atol, f"{wl.name}: max abs err {err}"
    return err


def test_cfg1_append_then_decode(gpu):
    """The reference's step order (infer/ops/attention.py:108-120): append the new row, then attend."""
    wl = workloads.cfg1().to(gpu)
    ops.store_kvcache(wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.slot_mapping)
    err = check(wl)
    print("cfg1 max abs err", err)


def test_cfg1_against_the_committed_golden_fixture(gpu):
    """HIP path against ``tests/golden/cfg1_golden.json``: caches after the append hash to the
    committed values (bit-exact), the attention output is within the bar of the committed float32
    output."""
    import hashlib
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "cfg1_golden.json")) as f:
        gold = json.load(f)
    wl = workloads.cfg1().to(gpu)
    ops.store_kvcache(wl.k_new, wl.v_new, wl.k_cache, wl.v_cache, wl.slot_mapping)
    torch.cuda.synchronize()
    sha = lambda t: hashlib.sha256(np.ascontiguousarray(bits(t)).tobytes()).hexdigest()
    assert sha(wl.k_cache) == gold["after_append_sha256"]["k_cache"]
    assert sha(wl.v_cache) == gold["after_append_sha256"]["v_cache"]
    got = f32(gpu_decode(wl))
    assert list(got.shape) == gold["attention_out"]["shape"]
    assert np.abs(got[:, :, :8] - np.array(gold["attention_out"]["first8"])).max() <= ATTN_ATOL
    assert np.abs(got[:, :, -8:] - np.array(gold["attention_out"]["last8"])).max() <= ATTN_ATOL
    assert np.abs(got.sum(-1) - np.array(gold["attention_out"]["row_sums"])).max() <= 128 * 2 ** -9 * 4


@pytest.mark.parametrize("splits", [1, 3, 64, 1024])
def test_split_count_invariance(gpu, splits):
    wl = workloads.cfg1().to(gpu)
    check(wl, splits=splits)


@pytest.mark.parametrize("hq,hkv", [(8, 8), (16, 8), (32, 8), (64, 8), (4, 1), (8, 2), (32, 4), (32, 16), (16, 1)])
def test_group_sizes_and_head_counts(gpu, hq, hkv):
    wl = workloads.make_decode_workload(f"g{hq}-{hkv}", [1, 31, 32, 33, 255, 256, 257, 600], hq, hkv,
                                        seed=hq * 7 + hkv).to(gpu)
    check(wl)


@pytest.mark.parametrize("bs", [32, 64, 128, 256, 512])
def test_block_sizes(gpu, bs):
    wl = workloads.make_decode_workload(f"bs{bs}", [5, 97, 511, 512, 513, 1300], 32, 8, bs=bs, seed=bs).to(gpu)
    check(wl)


def test_single_token_returns_v(gpu):
    """L = 1: softmax over one key is 1, so O = V[0] exactly (bf16 round trip)."""
    wl = workloads.make_decode_workload("one", [1, 1, 1], 32, 8, seed=5).to(gpu)
    got = gpu_decode(wl)
    for i in range(3):
        v0 = wl.v_cache[int(wl.block_table[i, 0]), 0]                    # [Hkv, D]
        assert torch.equal(got[i], v0.repeat_interleave(4, dim=0))


def test_equal_keys_give_mean_of_values(gpu):
    wl = workloads.make_decode_workload("mean", [300, 64], 16, 8, seed=6).to(gpu)
    wl.k_cache[:] = wl.k_cache[0, 0]          # every key identical -> uniform softmax
    got = f32(gpu_decode(wl))
    for i, n in enumerate(wl.lengths):
        rows = torch.cat([wl.v_cache[int(b)] for b in wl.block_table[i, : (n + 255) // 256]])[:n]
        mean = rows.float().mean(dim=0).cpu().numpy()                    # [Hkv, D]
        assert np.abs(got[i] - np.repeat(mean, 2, axis=0)).max() <= 1e-2


def test_row_maximum_covers_every_key_of_a_step(gpu):
    """One key whose score lies some 350 log2 units above all others, once at each of the 32 positions of
    a step: the softmax gives it weight 1 wherever it sits.  A running maximum taken over part of a step
    only (say, the keys one row of lanes holds) leaves the exponential of that key to overflow."""
    lens = [96] * 32
    wl = workloads.make_decode_workload("spike", lens, 16, 8, seed=11).to(gpu)
    g = wl.num_q_heads // wl.num_kv_heads
    for i in range(32):
        pos = 32 + i                                                     # the second of three steps
        blk = int(wl.block_table[i, pos // wl.block_size])
        q0 = wl.q[i, ::g].float()                                        # first query head of every KV head
        c = 250.0 / (wl.scale * (q0 * q0).sum(dim=-1, keepdim=True))     # score * scale = 250 for that head
        wl.k_cache[blk, pos % wl.block_size] = (c * q0).to(torch.bfloat16)
    got = f32(gpu_decode(wl))
    want = oracle_decode(wl)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= ATTN_ATOL
    for i in range(32):                                                  # weight 1: the key's value row, bit for bit
        pos = 32 + i
        blk = int(wl.block_table[i, pos // wl.block_size])
        assert np.array_equal(got[i, ::g], f32(wl.v_cache[blk, pos % wl.block_size]))


@pytest.mark.parametrize("direction", [1, -1])
def test_scores_that_rise_or_fall_along_the_sequence(gpu, direction):
    """Keys that are multiples of the query, the factor rising (or falling) by a fixed amount per token: the
    running maximum grows at every step (the accumulators are rescaled every time), or is set by the very
    first key and never again, with all later keys hundreds of log2 units below it."""
    lens = [700, 257, 33, 1024]
    wl = workloads.make_decode_workload("ramp", lens, 16, 8, seed=13).to(gpu)
    g = wl.num_q_heads // wl.num_kv_heads
    for i, n in enumerate(lens):
        q0 = wl.q[i, ::g].float()                                         # [Hkv, D]
        unit = q0 / (wl.scale * (q0 * q0).sum(dim=-1, keepdim=True))      # score * scale = 1 per unit factor
        for pos in range(n):
            f = 0.5 * (pos if direction > 0 else -pos)                   # 16 log2-ish units per 32-token step
            blk = int(wl.block_table[i, pos // wl.block_size])
            wl.k_cache[blk, pos % wl.block_size] = (f * unit).to(torch.bfloat16)
    got = f32(gpu_decode(wl))
    want = oracle_decode(wl)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= ATTN_ATOL


def test_block_permutation_invariance(gpu):
    """Same logical tokens under a different physical placement give bit-identical output."""
    wl = workloads.make_decode_workload("perm", [700, 1023, 40], 32, 8, nblk=32, seed=7).to(gpu)
    a = gpu_decode(wl)
    perm = torch.randperm(32, generator=torch.Generator().manual_seed(1)).to(gpu)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(32, device=gpu)
    kc2, vc2 = wl.k_cache[perm], wl.v_cache[perm]      # new block j holds old block perm[j]
    bt2 = torch.where(wl.block_table >= 0, inv[wl.block_table.clamp(min=0).long()].int(), wl.block_table)
    out = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), kc2, vc2, cache_seqlens=wl.context_lens,
                                      block_table=bt2, softmax_scale=wl.scale)[:, 0]
    assert torch.equal(a, out)


def test_zero_length_rows_and_graph_padding(gpu):
    """Rows with context_len 0 (the reference zero-fills its graph buffers:
    infer/engine/model_runner.py:144-146) give zeros and do not disturb their neighbours; unused
    table entries may hold -1 or garbage."""
    wl = workloads.make_decode_workload("pad", [300, 1, 513, 77], 32, 8, seed=8).to(gpu)
    ctx = wl.context_lens.clone()
    ctx[1] = 0
    bt = wl.block_table.clone()
    bt[bt < 0] = 10_000_000           # must never be dereferenced
    bt[1] = -1
    out = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), wl.k_cache, wl.v_cache, cache_seqlens=ctx,
                                      block_table=bt, softmax_scale=wl.scale)[:, 0]
    torch.cuda.synchronize()
    want = oracle_decode(wl)
    got = f32(out)
    assert not got[1].any()
    for i in (0, 2, 3):
        assert np.abs(got[i] - want[i]).max() <= ATTN_ATOL
    ctx[:] = 0
    out = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), wl.k_cache, wl.v_cache, cache_seqlens=ctx,
                                      block_table=bt, softmax_scale=wl.scale)
    assert not out.any()


def test_stale_nan_beyond_length_is_ignored(gpu):
    """Cache rows past a sequence's length may hold anything (a freed sequence's data, NaN bit
    patterns of never-written memory): they must not reach the output."""
    wl = workloads.make_decode_workload("nan", [37, 289, 1000], 32, 8, seed=9).to(gpu)
    want = oracle_decode(wl)
    for i, n in enumerate(wl.lengths):
        blk = int(wl.block_table[i, (n - 1) // 256])
        wl.k_cache[blk, n % 256 or 256:] = float("nan")
        wl.v_cache[blk, n % 256 or 256:] = float("nan")
    got = f32(gpu_decode(wl))
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= ATTN_ATOL


def test_large_batch(gpu):
    g = torch.Generator().manual_seed(11)
    lens = torch.randint(1, 700, (300,), generator=g).tolist()
    wl = workloads.make_decode_workload("b300", lens, 16, 8, seed=11).to(gpu)
    check(wl)


@pytest.mark.parametrize("splits", [4, 40, None])
def test_many_tiny_sequences_in_one_span(gpu, splits):
    """Hundreds of sequences shorter than a span: one wavefront walks many segments, more than fit its
    LDS plan table (32) or its parked-partials area (4 at group size 4), so the batching and the
    early-drain paths run."""
    g = torch.Generator().manual_seed(21)
    lens = torch.randint(1, 70, (900,), generator=g).tolist()
    wl = workloads.make_decode_workload("tiny900", lens, 32, 8, bs=32, seed=21).to(gpu)
    check(wl, splits=splits)


@pytest.mark.parametrize("hq", [8, 64, 128])
def test_many_short_sequences_other_group_sizes(gpu, hq):
    g = torch.Generator().manual_seed(22)
    lens = torch.randint(1, 100, (200,), generator=g).tolist()
    wl = workloads.make_decode_workload("short200", lens, hq, 8, bs=32, seed=22).to(gpu)
    check(wl, splits=8)


def test_one_span_longer_than_64_blocks(gpu):
    """A single wavefront streaming 150 blocks of one sequence: block ids past the 64 held in the
    lane-indexed register come from the table directly."""
    wl = workloads.make_decode_workload("long1", [4800, 33], 16, 8, bs=32, nblk=160, seed=23).to(gpu)
    check(wl, splits=1)
    check(wl, splits=2)


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_and_split_counts(gpu, seed):
    """Head counts, block sizes, batch shapes (a few long, hundreds of tiny, mixed) and split-workgroup
    counts drawn at random; sizes kept small enough for the CPU oracle."""
    heads = [(32, 8), (16, 8), (40, 8), (8, 8), (4, 4), (12, 2), (64, 8), (16, 1), (128, 8), (32, 16)]
    rng = np.random.default_rng(1000 + seed)
    hq, hkv = heads[rng.integers(len(heads))]
    bs = int(rng.choice([32, 64, 128, 256]))
    mode = rng.integers(4)
    if mode == 0:
        lens = rng.integers(1, 9000, size=int(rng.integers(1, 6)))
    elif mode == 1:
        lens = rng.integers(1, 90, size=int(rng.integers(50, 400)))
    elif mode == 2:
        lens = rng.integers(1, 1500, size=int(rng.integers(8, 80)))
    else:
        b = int(rng.integers(2, 40))
        lens = np.where(rng.random(b) < 0.3, rng.integers(2000, 5000, size=b), rng.integers(1, 40, size=b))
    lens = [int(x) for x in lens]
    while sum(lens) * hq > 2_500_000:
        lens = lens[:-1] if len(lens) > 1 else [lens[0] // 2]
    splits = int(rng.choice([0, 0, 1, 3, 7, 64, 200, 300, 1000]))
    wl = workloads.make_decode_workload(f"rnd{seed}", lens, hq, hkv, bs=bs, seed=seed).to(gpu)
    check(wl, splits=splits)


@pytest.mark.parametrize("w", [256, 100, 7])
def test_span_count_reported_in_the_workspace_header(gpu, w):
    """The streaming kernel leaves (spans used, total steps, spans per workgroup and KV head) in the first
    words of the workspace.  A launch has W = span positions x spans per workgroup wavefront spans.  With
    more steps than that it must use the fewest spans that keep the longest one at ceil(total / W) steps,
    so no wavefront does more than the grid forces; otherwise all of them."""
    for lens in ([4000, 77, 1300, 2048, 31, 900] * 4, [40, 33, 1], workloads.cfg2_lengths(64)):
        wl = workloads.make_decode_workload("hdr", lens, 32, 8, seed=5).to(gpu)
        ws = ops.decode_workspace(gpu, len(lens), 32, 8, 128)
        ops.paged_attn_decode_split(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, ws,
                                    split_workgroups=w)
        torch.cuda.synchronize()
        spans, total, parts = (int(v) for v in ws[:12].view(torch.int32)[:3].tolist())
        assert total == sum((n + 31) // 32 for n in lens)
        assert parts in (1, 2, 4, 8)
        W = w * parts
        if total <= W:
            assert spans == W
        else:
            longest = -(-total // W)
            assert -(-total // spans) == longest                    # the longest span is as short as W allows
            assert spans == W or -(-total // (spans - 1)) > longest  # and no fewer spans would do
            assert spans <= W


def test_cfg2_full_size(gpu):
    wl = workloads.cfg2()                 # drawn on the CPU from the seed, the bits the checksums name
    assert_seeded_inputs(wl, "cfg2")
    wl = wl.to(gpu)
    err = check(wl)
    print("cfg2 max abs err", err)


def test_cfg4_long_context(gpu):
    wl = workloads.cfg4()
    assert_seeded_inputs(wl, "cfg4")
    wl = wl.to(gpu)
    err = check(wl)
    print("cfg4 max abs err", err)


def test_layer_view_of_fused_cache(gpu):
    """Caches as per-layer views of one [2, layers, nblk, bs, Hkv, D] tensor
    (infer/engine/model_runner.py:58-64)."""
    wl = workloads.make_decode_workload("layers", [400, 90], 32, 8, nblk=6, seed=12).to(gpu)
    big = torch.zeros((2, 3, 6, 256, 8, 128), dtype=torch.bfloat16, device=gpu)
    big[0, 1], big[1, 1] = wl.k_cache, wl.v_cache
    out = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), big[0, 1], big[1, 1], cache_seqlens=wl.context_lens,
                                      block_table=wl.block_table, softmax_scale=wl.scale)[:, 0]
    assert np.abs(f32(out) - oracle_decode(wl)).max() <= ATTN_ATOL


def test_errors_are_loud(gpu):
    wl = workloads.make_decode_workload("err", [10], 32, 8, seed=1).to(gpu)
    with pytest.raises(RuntimeError):
        ops.flash_attn_with_kvcache(wl.q.cpu().unsqueeze(1), wl.k_cache, wl.v_cache,
                                    cache_seqlens=wl.context_lens, block_table=wl.block_table)
    q64 = torch.zeros((1, 1, 32, 64), dtype=torch.bfloat16, device=gpu)
    kc = torch.zeros((2, 256, 8, 64), dtype=torch.bfloat16, device=gpu)
    with pytest.raises(RuntimeError):
        ops.flash_attn_with_kvcache(q64, kc, kc, cache_seqlens=wl.context_lens, block_table=wl.block_table)


def test_two_streams_with_different_split_counts(gpu):
    """The split count is per call and the library holds no launch state: two decode calls with
    different counts, each with its own workspace, run concurrently on two streams and both match
    the oracle; the same two calls run one after the other give the same bits."""
    wa = workloads.make_decode_workload("s0", [1500, 700, 2300, 90] * 4, 32, 8, seed=11).to(gpu)
    wb = workloads.make_decode_workload("s1", [3100, 33, 512] * 3, 32, 8, seed=12).to(gpu)
    lib_bytes = ops._lib.load().infer_paged_decode_workspace_bytes
    ws_a = torch.empty(lib_bytes(16, 32, 8, 128), dtype=torch.uint8, device=gpu)
    ws_b = torch.empty(lib_bytes(9, 32, 8, 128), dtype=torch.uint8, device=gpu)
    serial = []
    for wl, ws, w in ((wa, ws_a, 37), (wb, ws_b, 256)):
        out = torch.empty_like(wl.q)
        ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, out, ws,
                              split_workgroups=w)
        serial.append(out)
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    outs = [torch.empty_like(wa.q), torch.empty_like(wb.q)]
    for _ in range(3):
        with torch.cuda.stream(sa):
            ops.paged_attn_decode(wa.q, wa.k_cache, wa.v_cache, wa.block_table, wa.context_lens, wa.scale, outs[0],
                                  ws_a, split_workgroups=37)
        with torch.cuda.stream(sb):
            ops.paged_attn_decode(wb.q, wb.k_cache, wb.v_cache, wb.block_table, wb.context_lens, wb.scale, outs[1],
                                  ws_b, split_workgroups=256)
    torch.cuda.synchronize()
    for wl, got, ref in ((wa, outs[0], serial[0]), (wb, outs[1], serial[1])):
        assert np.array_equal(bits(got), bits(ref))
        assert float(np.abs(f32(got) - oracle_decode(wl)).max()) <= ATTN_ATOL


def test_shared_workspace_refuses_a_second_stream_while_the_first_is_busy(gpu):
    """Calls without a workspace of their own share one per shape, which holds partial results until the
    merge kernel has run: a call on another stream while the last stream still has work pending is refused
    instead of overwriting them; once that stream is idle the other one may use it."""
    wl = workloads.make_decode_workload("ws", [900, 300, 2000, 64], 32, 8, seed=21).to(gpu)
    out = torch.empty_like(wl.q)
    call = lambda: ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, out)
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(sa):
        torch.cuda._sleep(200_000_000)          # keeps stream sa busy for a moment
        call()
    with torch.cuda.stream(sb):
        with pytest.raises(RuntimeError, match="still in use on another stream"):
            call()
    sa.synchronize()
    with torch.cuda.stream(sb):
        call()
    torch.cuda.synchronize()
    assert float(np.abs(f32(out) - oracle_decode(wl)).max()) <= ATTN_ATOL


def test_split_then_merge_need_not_agree_on_a_setting(gpu):
    """The merge phase locates the partial results from the workspace alone: a split launched with any
    split count is merged correctly by the same merge call."""
    wl = workloads.make_decode_workload("sm", [2000, 300, 4096, 1], 32, 8, seed=13).to(gpu)
    ws = ops.decode_workspace(gpu, 4, 32, 8, 128)
    want = oracle_decode(wl)
    for w in (1, 5, 64, 1024):
        out = torch.full_like(wl.q, float("nan"))
        ops.paged_attn_decode_split(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, ws,
                                    split_workgroups=w)
        ops.paged_attn_decode_merge(out, wl.context_lens, 8, ws)
        torch.cuda.synchronize()
        assert float(np.abs(f32(out) - want).max()) <= ATTN_ATOL


def test_length_beyond_the_table_is_cut_to_the_table(gpu):
    """A context length larger than table_cols * block_size (a corrupt length) must not make the kernel
    read block ids past its table row: the row is attended as if it were table_cols blocks long."""
    wl = workloads.make_decode_workload("clamp", [512, 700, 256], 16, 8, seed=14).to(gpu)
    cols = wl.block_table.shape[1]                      # 3 blocks
    full = [cols * 256] * 3
    bad = torch.tensor([10 ** 6, 2 ** 31 - 1, cols * 256 + 1], dtype=torch.int32, device=gpu)
    bt = wl.block_table.clamp(min=0).contiguous()       # every entry of the row is a real block
    out_bad = torch.empty_like(wl.q)
    out_full = torch.empty_like(wl.q)
    ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, bt, bad, wl.scale, out_bad)
    ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, bt, torch.tensor(full, dtype=torch.int32, device=gpu),
                          wl.scale, out_full)
    torch.cuda.synchronize()
    assert np.array_equal(bits(out_bad), bits(out_full))


@pytest.mark.parametrize("scale", [0.02, 0.3])
def test_softmax_scale_is_honoured(gpu, scale):
    """A scale other than head_dim ** -0.5 (the reference passes its own, infer/models/Qwen3.py:76)."""
    wl = workloads.make_decode_workload("scale", [37, 300, 1025, 700], 32, 8, nblk=16, seed=31).to(gpu)
    wl.scale = scale
    check(wl)


def test_query_and_output_rows_as_strided_views(gpu):
    """Q as a column slice of the fused qkv matrix (infer/models/Qwen3.py:110-111) and the output as a
    slice of a wider buffer: same bits as with contiguous tensors."""
    wl = workloads.make_decode_workload("views", [37, 300, 1025, 700], 32, 8, nblk=16, seed=32).to(gpu)
    want = gpu_decode(wl, splits=0)
    b, hq, d = wl.q.shape
    qkv = torch.randn((b, (hq + 16) * d), device=gpu).to(torch.bfloat16)
    qkv[:, :hq * d] = wl.q.reshape(b, -1)
    q_view = qkv.split([hq * d, 8 * d, 8 * d], dim=-1)[0].view(b, hq, d)
    wide = torch.full((b, hq * d + 256), 7.0, dtype=torch.bfloat16, device=gpu)
    out_view = wide[:, :hq * d].view(b, hq, d)
    assert not q_view.is_contiguous() and not out_view.is_contiguous()
    ops.paged_attn_decode(q_view, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens, wl.scale, out_view)
    torch.cuda.synchronize()
    assert torch.equal(out_view, want)
    assert (wide[:, hq * d:] == 7.0).all()      # nothing written beside the output rows


def uniform_decode(wl, length):
    out = torch.full_like(wl.q, 7.0)
    ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, length, wl.scale, out)
    torch.cuda.synchronize()
    return out


# batch, context length, Hq, Hkv: shapes on both sides of the rule that picks the one-kernel form
# (batch x Hkv x pieces / 8 workgroups within 80-100 % of the compute units, even pieces)
UNIFORM_SHAPES = [
    (64, 512, 32, 8),     # 4 pieces per KV head
    (64, 517, 64, 8),     # ... a ragged last step, group size 8
    (128, 300, 32, 8),    # 2 pieces
    (32, 1000, 16, 8),    # 8 pieces: one KV head per workgroup
    (256, 100, 8, 8),     # 1 piece: a sequence per workgroup, nothing to fold
    (240, 65, 16, 8),     # 240 of 256 workgroups
    (128, 130, 128, 16),  # 16 KV heads, group size 8
    (256, 128, 8, 2),     # 2 KV heads: 4 pieces
    (64, 33, 32, 8),      # fewer steps than pieces: span kernels without a lengths array
    (4, 700, 16, 8),      # too few sequences to fill the chip: span kernels
    (100, 260, 32, 8),    # 100 or 200 workgroups: span kernels
    (3, 1, 16, 8),
]


@pytest.mark.parametrize("batch,length,hq,hkv", UNIFORM_SHAPES)
def test_one_length_for_the_batch_as_a_host_integer(gpu, batch, length, hq, hkv):
    """cache_seqlens given as one int (flash_attn_with_kvcache accepts both): same result as the tensor
    form, against the oracle, whichever kernels the library picks for the shape."""
    wl = workloads.make_decode_workload("uniform", [length] * batch, hq, hkv, seed=batch + length).to(gpu)
    got = uniform_decode(wl, length)
    want = oracle_decode(wl)
    assert np.isfinite(f32(got)).all()
    assert np.abs(f32(got) - want).max() <= ATTN_ATOL
    # the tensor form folds the same partial sums in another order: two bf16 roundings of close fp32 values
    assert (got.float() - gpu_decode(wl, splits=0).float()).abs().max() <= 8e-3
    via_flash = ops.flash_attn_with_kvcache(wl.q.unsqueeze(1), wl.k_cache, wl.v_cache, cache_seqlens=length,
                                            block_table=wl.block_table, softmax_scale=wl.scale)[:, 0]
    assert torch.equal(via_flash, got)


def test_uniform_length_edge_cases(gpu):
    wl = workloads.make_decode_workload("uniform-edges", [300] * 64, 32, 8, seed=77).to(gpu)
    assert (uniform_decode(wl, 0) == 0).all()                       # no context: zeros, as the tensor form
    # one token: softmax over one key is 1, the output is that token's V row for every head of the group
    one = uniform_decode(wl, 1)
    v_first = wl.v_cache[wl.block_table[:, 0].long(), 0]            # [B, Hkv, D]
    assert torch.equal(one, v_first.repeat_interleave(4, dim=1))
    # a length the table row cannot address is cut to the row: 2 columns x 256 tokens
    cut = uniform_decode(wl, 10_000)
    wl2 = workloads.make_decode_workload("uniform-edges", [300] * 64, 32, 8, seed=77).to(gpu)
    wl2.context_lens[:] = wl2.block_table.shape[1] * 256
    # the table rows address 512 tokens: the same as asking for 512, in either form
    assert torch.equal(cut, uniform_decode(wl, wl.block_table.shape[1] * 256))
    assert (cut.float() - gpu_decode(wl2, splits=0).float()).abs().max() <= 8e-3
    # stale NaN behind the length is never read into the result
    for i in range(64):
        blk = int(wl.block_table[i, 1])
        wl.k_cache[blk, 300 % 256:] = float("nan")
        wl.v_cache[blk, 300 % 256:] = float("nan")
    got = uniform_decode(wl, 300)
    assert np.isfinite(f32(got)).all()
    keep = wl.context_lens.clone()
    assert np.abs(f32(got) - oracle_decode(wl)).max() <= ATTN_ATOL and torch.equal(keep, wl.context_lens)


def test_uniform_form_on_strided_views_and_other_block_sizes(gpu):
    for bs in (32, 64, 512):
        wl = workloads.make_decode_workload("uniform-bs", [2 * bs + 5] * 64, 32, 8, bs=bs, seed=bs).to(gpu)
        assert np.abs(f32(uniform_decode(wl, 2 * bs + 5)) - oracle_decode(wl)).max() <= ATTN_ATOL
    wl = workloads.make_decode_workload("uniform-views", [400] * 64, 32, 8, seed=5).to(gpu)
    want = uniform_decode(wl, 400)
    b, hq, d = wl.q.shape
    qkv = torch.randn((b, (hq + 16) * d), device=gpu).to(torch.bfloat16)
    qkv[:, :hq * d] = wl.q.reshape(b, -1)
    q_view = qkv.split([hq * d, 8 * d, 8 * d], dim=-1)[0].view(b, hq, d)
    wide = torch.full((b, hq * d + 256), 7.0, dtype=torch.bfloat16, device=gpu)
    out_view = wide[:, :hq * d].view(b, hq, d)
    ops.paged_attn_decode(q_view, wl.k_cache, wl.v_cache, wl.block_table, 400, wl.scale, out_view)
    torch.cuda.synchronize()
    assert torch.equal(out_view, want) and (wide[:, hq * d:] == 7.0).all()


def test_uniform_form_with_pieces_longer_than_64_blocks(gpu):
    """Block size 32 and 16,896 tokens: each of the 8 pieces of a sequence spans 66 blocks, two more than
    the block-id register holds, so the last ones are looked up in the table.  Checked against the tensor
    form (whose own long-span case is checked against the oracle above)."""
    length = 8 * 66 * 32
    wl = workloads.make_decode_workload("uniform-long", [length] * 256, 4, 1, bs=32, seed=9, pool_factor=1.0,
                                        device=gpu, device_fill=True)
    got = uniform_decode(wl, length)
    want = gpu_decode(wl, splits=0)
    assert np.isfinite(f32(got)).all()
    assert (got.float() - want.float()).abs().max() <= 8e-3
    # and one sequence of it against the oracle
    one = workloads.DecodeWorkload(**{**wl.__dict__, "q": wl.q[:1], "block_table": wl.block_table[:1],
                                      "context_lens": wl.context_lens[:1], "lengths": wl.lengths[:1],
                                      "k_new": wl.k_new[:1], "v_new": wl.v_new[:1],
                                      "slot_mapping": wl.slot_mapping[:1]})
    assert np.abs(f32(got[:1]) - oracle_decode(one)).max() <= ATTN_ATOL
