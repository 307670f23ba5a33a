"""The decode entry point that allocates nothing (infer_paged_decode_noalloc_bf16) against the
workspace-taking entry point it shares its kernels with: same bits, on two calls in a row, the
second with a smaller input, through the C ABI."""
import numpy as np
import pytest
import torch

from infer_amd import _lib, workloads
from tests.helpers import ATTN_ATOL, bits, f32, oracle_decode

pytestmark = pytest.mark.gpu


def _call(entry, wl, out, workspace=None):
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    nblk, bs, hkv, d = wl.k_cache.shape
    b, hq, _ = wl.q.shape
    head = (wl.q.data_ptr(), wl.q.stride(0), wl.k_cache.data_ptr(), wl.v_cache.data_ptr(), wl.k_cache.stride(0),
            wl.k_cache.stride(1), out.data_ptr(), out.stride(0), wl.block_table.data_ptr(), wl.block_table.stride(0),
            wl.block_table.shape[1], wl.context_lens.data_ptr(), b, hq, hkv, d, bs, nblk, float(wl.scale))
    if entry == "noalloc":
        return lib.infer_paged_decode_noalloc_bf16(*head, stream)
    return lib.infer_paged_decode_bf16(*head, 0, workspace.data_ptr(), workspace.numel(), stream)


def test_two_calls_in_a_row_match_the_workspace_entry_point(gpu):
    lib = _lib.load()
    big = workloads.make_decode_workload("na-big", [1500, 37, 2300, 256, 700, 4096, 1023, 90] * 4, 32, 8, seed=21).to(gpu)
    small = workloads.make_decode_workload("na-small", [300, 1, 64], 32, 8, seed=22).to(gpu)
    ws = torch.empty(lib.infer_paged_decode_workspace_bytes(32, 32, 8, 128), dtype=torch.uint8, device=gpu)
    for wl in (big, small):                       # second call: smaller input, scratch still holds the first call's records
        want = torch.empty_like(wl.q)
        got = torch.full_like(wl.q, float("nan"))
        assert _call("workspace", wl, want, ws) == 0
        assert _call("noalloc", wl, got) == 0
        torch.cuda.synchronize()
        assert np.array_equal(bits(got), bits(want)), wl.name
        assert float(np.abs(f32(got) - oracle_decode(wl)).max()) <= ATTN_ATOL


def test_allocates_nothing_and_rejects_what_does_not_fit(gpu):
    wl = workloads.make_decode_workload("na-mem", [700, 33], 64, 8, seed=23).to(gpu)
    out = torch.empty_like(wl.q)
    assert _call("noalloc", wl, out) == 0          # first call on the device resolves the scratch address
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(gpu)[0]
    for _ in range(5):
        assert _call("noalloc", wl, out) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(gpu)[0] == free_before
    assert float(np.abs(f32(out) - oracle_decode(wl)).max()) <= ATTN_ATOL
    # partial results of batch 4096 at 32/8 heads need 8 * (256 + 4096) records of 2080 bytes = 72 MB > 16 MiB
    many = workloads.make_decode_workload("na-many", [5] * 4096, 32, 8, nblk=4100, bs=32, seed=24).to(gpu)
    assert _call("noalloc", many, torch.empty_like(many.q)) == -3


def test_replays_inside_a_hip_graph(gpu):
    """What the entry point is for: a captured decode step that may not allocate.  The graph is replayed
    with new lengths, tables and queries in its static buffers, with eager work in between; every replay
    must give the bits of the eager workspace call on the same inputs."""
    lib = _lib.load()
    shapes = ([900, 33, 2047, 256], [64, 1300, 5, 700], [1, 1, 4096, 12])
    wls = [workloads.make_decode_workload(f"na-g{i}", lens, 32, 8, nblk=40, seed=30 + i).to(gpu)
           for i, lens in enumerate(shapes)]
    st = wls[0]
    static = workloads.DecodeWorkload(**{k: (v.clone() if isinstance(v, torch.Tensor) else v)
                                         for k, v in st.__dict__.items()})
    cols = max(w.block_table.shape[1] for w in wls)
    static.block_table = torch.zeros((4, cols), dtype=torch.int32, device=gpu)
    out = torch.empty_like(static.q)
    assert _call("noalloc", wls[0], torch.empty_like(st.q)) == 0      # resolves the scratch address outside capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert _call("noalloc", static, out) == 0
    torch.cuda.synchronize()
    ws = torch.empty(lib.infer_paged_decode_workspace_bytes(4, 32, 8, 128), dtype=torch.uint8, device=gpu)
    for wl in wls + wls[::-1]:
        static.q.copy_(wl.q)
        static.k_cache.copy_(wl.k_cache)
        static.v_cache.copy_(wl.v_cache)
        static.context_lens.copy_(wl.context_lens)
        static.block_table.zero_()
        static.block_table[:, :wl.block_table.shape[1]] = wl.block_table.clamp(min=0)
        graph.replay()
        want = torch.empty_like(wl.q)
        assert _call("workspace", wl, want, ws) == 0                     # eager work between the replays
        torch.cuda.synchronize()
        assert np.array_equal(bits(out), bits(want)), wl.name


def test_another_stream_is_refused_while_the_last_one_is_busy(gpu):
    """All calls on a GPU share the library's scratch array: a call on another stream than the previous one
    is refused while that stream still has work pending, and accepted once it has drained."""
    wl = workloads.make_decode_workload("na-busy", [900, 70, 300], 32, 8, seed=25).to(gpu)
    out_a, out_b = torch.empty_like(wl.q), torch.empty_like(wl.q)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(sa):
        assert _call("noalloc", wl, out_a) == 0
        torch.cuda._sleep(400_000_000)            # keeps stream A busy for a fraction of a second
    with torch.cuda.stream(sb):
        assert _call("noalloc", wl, out_b) == -7  # INFER_KV_EBUSY: nothing was enqueued
    sa.synchronize()
    with torch.cuda.stream(sb):
        assert _call("noalloc", wl, out_b) == 0
    torch.cuda.synchronize()
    assert np.array_equal(bits(out_a), bits(out_b))
    assert _call("noalloc", wl, out_b) == 0       # back on the default stream, everything drained
    torch.cuda.synchronize()
