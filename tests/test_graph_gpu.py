"""A decode step (append + paged decode attention) recorded into a HIP graph and replayed from
static buffers, the way the reference runs decode (infer/engine/model_runner.py:139-153, :163-198):
metadata buffers are overwritten before every replay, rows past the live batch are padding
(context length 0).  Every replay is checked against the eager result of the same inputs."""
import numpy as np
import pytest
import torch

from infer_amd import ops, workloads
from tests.helpers import ATTN_ATOL, f32, oracle_decode

pytestmark = pytest.mark.gpu


def test_decode_step_graph_replays_match_eager(gpu):
    hq, hkv, d, bs, max_bs, max_blocks, nblk = 32, 8, 128, 256, 8, 6, 64
    g = torch.Generator().manual_seed(0)
    k_cache = torch.randn((nblk, bs, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    v_cache = torch.randn((nblk, bs, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    # static buffers, as graph_vars in the reference
    q = torch.zeros((max_bs, hq, d), dtype=torch.bfloat16, device=gpu)
    k_new = torch.zeros((max_bs, hkv, d), dtype=torch.bfloat16, device=gpu)
    v_new = torch.zeros_like(k_new)
    slots = torch.full((max_bs,), -1, dtype=torch.int32, device=gpu)
    ctx = torch.zeros((max_bs,), dtype=torch.int32, device=gpu)
    tables = torch.zeros((max_bs, max_blocks), dtype=torch.int32, device=gpu)
    out = torch.zeros_like(q)
    ws = ops.decode_workspace(gpu, max_bs, hq, hkv, d)

    def step():
        ops.store_kvcache(k_new, v_new, k_cache, v_cache, slots)
        ops.paged_attn_decode(q, k_cache, v_cache, tables, ctx, d ** -0.5, out, ws)

    def fill(seed, lengths):
        """Writes one decode step for `lengths` live sequences into the static buffers."""
        gg = torch.Generator().manual_seed(seed)
        n = len(lengths)
        perm = torch.randperm(nblk, generator=gg).tolist()
        rows, at = [], 0
        for L in lengths:
            c = (L + bs - 1) // bs
            rows.append(perm[at:at + c])
            at += c
        q.zero_(); k_new.zero_(); v_new.zero_(); ctx.zero_(); tables.zero_()
        slots.fill_(-1)                                   # padding rows are skipped by the append
        q[:n] = torch.randn((n, hq, d), generator=gg).to(torch.bfloat16).to(gpu)
        k_new[:n] = torch.randn((n, hkv, d), generator=gg).to(torch.bfloat16).to(gpu)
        v_new[:n] = torch.randn((n, hkv, d), generator=gg).to(torch.bfloat16).to(gpu)
        ctx[:n] = torch.tensor(lengths, dtype=torch.int32)
        for i, r in enumerate(rows):
            tables[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
            slots[i] = r[-1] * bs + (lengths[i] - 1) % bs
        return n

    fill(1, [300, 17, 1024])
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):                            # warm-up outside the capture
        step()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()

    for seed, lengths in ((2, [513, 40, 700, 256, 9]), (3, [1]), (4, [1536] * 8), (5, [255, 257]), (6, [90, 600, 33])):
        n = fill(seed, lengths)
        cache_before = (k_cache.clone(), v_cache.clone())
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        kc_g, vc_g = k_cache.clone(), v_cache.clone()
        # eager run of the same step from the same starting cache
        k_cache.copy_(cache_before[0]); v_cache.copy_(cache_before[1])
        step()
        torch.cuda.synchronize()
        assert torch.equal(k_cache, kc_g) and torch.equal(v_cache, vc_g), f"append differs on replay {seed}"
        assert torch.equal(out, got), f"attention differs on replay {seed}"
        assert not got[n:].any()                          # padding rows give zeros
        # and both agree with the oracle
        wl = workloads.DecodeWorkload("g", hq, hkv, d, bs, d ** -0.5, q[:n], k_new[:n], v_new[:n], k_cache, v_cache,
                                      slots[:n], tables[:n], ctx[:n], list(lengths))
        assert np.abs(f32(got[:n]) - oracle_decode(wl)).max() <= ATTN_ATOL


def test_uniform_length_decode_graph_replays_match_eager(gpu):
    """The single-kernel form (one host integer as the length of every sequence) recorded into a graph:
    the length is frozen at capture, the tensors it reads are not.  Each replay runs between eager work and
    synchronisations and is compared with the eager result of the same inputs and with the oracle."""
    length = 700
    wl = workloads.make_decode_workload("uniform-graph", [length] * 64, 32, 8, seed=41).to(gpu)
    out = torch.zeros_like(wl.q)
    ws = ops.decode_workspace(gpu, 64, 32, 8, 128)

    def step():
        ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, length, wl.scale, out, ws)

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()                                            # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    g = torch.Generator().manual_seed(42)
    for replay in range(4):
        wl.q.copy_(torch.randn(wl.q.shape, generator=g).to(torch.bfloat16))
        if replay == 2:                                   # another permutation of the same blocks
            perm = torch.randperm(64, generator=g).to(gpu)
            wl.block_table.copy_(wl.block_table[perm])
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        out.zero_()
        step()
        torch.cuda.synchronize()
        assert torch.equal(got, out), f"replay {replay} differs from eager"
        assert np.abs(f32(got) - oracle_decode(wl)).max() <= ATTN_ATOL
