"""torch.ops._C.* registration and the operator-registry classes (infer_amd/csrc/torch_ops.cpp)."""
import numpy as np
import pytest
import torch

from infer_amd import workloads
from tests.helpers import ATTN_ATOL, bits, f32, oracle_decode


def test_library_loads_and_schemas_follow_the_reference_convention():
    import infer_ops
    for name in ("store_kvcache", "paged_attn_decode", "flash_attn_decode", "paged_attn_prefill"):
        op = getattr(torch.ops._C, name)
        schema = str(op.default._schema)
        assert schema.endswith("-> ()"), schema                 # out-parameter style, returns nothing
        assert "(a!)" in schema or "!" in schema, schema       # mutated tensors are annotated
    assert infer_ops.store_kvcache is torch.ops._C.store_kvcache
    for name in ("add", "rms_norm", "rms_norm_vllm", "rms_norm_fused", "matmul", "embedding", "flash_attn_prefill",
                 "rope", "silu", "softmax", "silu_and_mul"):       # the reference's eleven names stay importable
        assert callable(getattr(infer_ops, name))


def test_cpu_tensors_are_rejected():
    import infer_ops
    k = torch.zeros(2, 8, 128, dtype=torch.bfloat16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        infer_ops.store_kvcache(k, k, k, k, torch.zeros(2, dtype=torch.int32))


@pytest.mark.gpu
def test_torch_ops_match_the_oracle(gpu):
    import infer_ops
    wl = workloads.cfg1().to(gpu)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    infer_ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    from oracle import paged_ref
    ek, ev = bits(wl.k_cache).copy(), bits(wl.v_cache).copy()
    paged_ref.append_ref(bits(wl.k_new), bits(wl.v_new), ek, ev, wl.slot_mapping.cpu().numpy())
    assert np.array_equal(bits(kc), ek) and np.array_equal(bits(vc), ev)
    out = torch.empty_like(wl.q)
    infer_ops.paged_attn_decode(wl.q, kc, vc, wl.block_table, wl.context_lens, wl.scale, out)
    wl.k_cache, wl.v_cache = kc, vc
    want = oracle_decode(wl)
    assert np.abs(f32(out) - want).max() <= ATTN_ATOL
    out2 = torch.empty_like(wl.q)
    infer_ops.flash_attn_decode(wl.q, kc, vc, True, wl.block_table, wl.context_lens, out2)
    assert torch.equal(out, out2)


@pytest.mark.gpu
def test_torch_op_workspace_refuses_a_second_stream_while_the_first_is_busy(gpu):
    """torch.ops._C.paged_attn_decode keeps one workspace per shape: a call on another stream while the last
    stream still has work pending raises instead of overwriting partial results in use."""
    import infer_ops
    wl = workloads.make_decode_workload("tws", [700, 90, 1500, 33, 260], 16, 8, seed=22).to(gpu)
    out = torch.empty_like(wl.q)
    call = lambda: infer_ops.paged_attn_decode(wl.q, wl.k_cache, wl.v_cache, wl.block_table, wl.context_lens,
                                               wl.scale, out)
    torch.cuda.synchronize()
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(sa):
        torch.cuda._sleep(200_000_000)
        call()
    with torch.cuda.stream(sb):
        with pytest.raises(RuntimeError, match="still in use on another stream"):
            call()
    sa.synchronize()
    with torch.cuda.stream(sb):
        call()
    torch.cuda.synchronize()
    assert np.abs(f32(out) - oracle_decode(wl)).max() <= ATTN_ATOL


@pytest.mark.gpu
def test_registry_operators_run_the_kernels(gpu):
    """KVAppendOperator / PagedAttentionOperator are fetched from the OperatorRegistry through the
    UnifiedOp facade and really override forward()."""
    import infer_ops  # noqa: F401
    wl = workloads.cfg1().to(gpu)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    kc2, vc2 = wl.k_cache.clone(), wl.v_cache.clone()
    torch.ops._C.registry_store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    torch.ops._C.store_kvcache(wl.k_new, wl.v_new, kc2, vc2, wl.slot_mapping)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2) and not torch.equal(kc, wl.k_cache)
    a, b = torch.empty_like(wl.q), torch.empty_like(wl.q)
    torch.ops._C.registry_paged_attn_decode(wl.q, kc, vc, wl.block_table, wl.context_lens, wl.scale, a)
    torch.ops._C.paged_attn_decode(wl.q, kc, vc, wl.block_table, wl.context_lens, wl.scale, b)
    assert torch.equal(a, b)


@pytest.mark.gpu
def test_prefill_op(gpu):
    import infer_ops
    from infer_amd import ops
    wl = workloads.make_prefill_workload("p", [300, 70], [256, 0], 16, 8, seed=4, pad_fraction=0.0).to(gpu)
    kc, vc = wl.k_cache.clone(), wl.v_cache.clone()
    infer_ops.store_kvcache(wl.k_new, wl.v_new, kc, vc, wl.slot_mapping)
    out = torch.empty_like(wl.q)
    infer_ops.paged_attn_prefill(wl.q, kc, vc, wl.cu_seqlens_q, wl.cu_seqlens_k, wl.max_seqlen_q, wl.block_table,
                                 wl.scale, True, out)
    want = ops.flash_attn_varlen_func(wl.q, kc, vc, max_seqlen_q=wl.max_seqlen_q, cu_seqlens_q=wl.cu_seqlens_q,
                                      max_seqlen_k=wl.max_seqlen_k, cu_seqlens_k=wl.cu_seqlens_k,
                                      softmax_scale=wl.scale, causal=True, block_table=wl.block_table)
    assert torch.equal(out, want)


@pytest.mark.gpu
def test_the_reference_op_names_compute_what_their_schemas_say(gpu):
    """Shapes and tolerances of the reference's own op tests (``test/op.py``)."""
    import infer_ops
    g = torch.Generator().manual_seed(0)
    bf = dict(dtype=torch.bfloat16, device=gpu)
    a, b = torch.randn(64, 256, generator=g).to(**bf), torch.randn(64, 256, generator=g).to(**bf)
    out = torch.empty_like(a)
    infer_ops.add(a, b, out)
    assert torch.equal(out, a + b)
    w = (1 + 0.1 * torch.randn(256, generator=g)).to(**bf)
    want = torch.nn.functional.rms_norm(a.float(), (256,), w.float(), 1e-6)
    for call in (lambda: infer_ops.rms_norm(a, w, out, None, 1e-6), lambda: infer_ops.rms_norm_vllm(out, a, w, 1e-6)):
        call()
        assert torch.allclose(out.float(), want, atol=2e-2, rtol=1e-2)
    x, res = a.clone(), b.clone()
    infer_ops.rms_norm_fused(x, res, w, 1e-6)
    assert torch.equal(res, a + b)
    assert torch.allclose(x.float(), torch.nn.functional.rms_norm((a + b).float(), (256,), w.float(), 1e-6),
                          atol=2e-2, rtol=1e-2)
    wt = torch.randn(256, 128, generator=g).to(**bf)
    mm = torch.empty(64, 128, **bf)
    infer_ops.matmul(a, wt, mm)
    assert torch.allclose(mm.float(), a.float() @ wt.float(), atol=0.5, rtol=2e-2)
    ids = torch.randint(0, 64, (10,), generator=g).to(gpu)
    emb = torch.empty(10, 256, **bf)
    infer_ops.embedding(emb, ids, a)
    assert torch.equal(emb, a[ids])
    q, k, v = (torch.randn(1, 4, 64, 128, generator=g).to(**bf) for _ in range(3))
    o = torch.empty_like(q)
    infer_ops.flash_attn_prefill(q, k, v, o)
    s = (q.float() @ k.float().transpose(-1, -2)) / 128 ** 0.5
    s = s.masked_fill(~torch.ones(64, 64, dtype=torch.bool, device=gpu).tril(), float("-inf"))
    assert torch.allclose(o.float(), torch.softmax(s, -1) @ v.float(), atol=2e-2, rtol=1e-3)
    act = torch.empty(64, 128, **bf)
    infer_ops.silu_and_mul(act, a)
    assert torch.allclose(act.float(), torch.nn.functional.silu(a[:, :128].float()) * a[:, 128:].float(),
                          atol=2e-2, rtol=2e-2)
    infer_ops.silu(out, a)
    assert torch.allclose(out.float(), torch.nn.functional.silu(a.float()), atol=1e-2, rtol=1e-2)
    infer_ops.softmax(out, a, 1)
    assert torch.allclose(out.float().sum(-1), torch.ones(64, device=gpu), atol=2e-2)
    # rope: rotating by position p then comparing with the closed form on one pair
    from infer_amd.layers import cos_sin_table
    table = cos_sin_table(128, 64, 1e4, gpu)
    pos = torch.arange(32, device=gpu)
    qq = torch.randn(32, 2, 128, generator=g).to(**bf)
    q0 = qq.clone()
    infer_ops.rope(pos, qq, None, 128, table, True)
    c, sn = table[pos, :64].float(), table[pos, 64:].float()
    want1 = q0[:, 0, :64].float() * c - q0[:, 0, 64:].float() * sn
    assert torch.allclose(qq[:, 0, :64].float(), want1, atol=3e-2, rtol=2e-2)
    assert torch.equal(qq[0], q0[0])                    # position 0 is the identity
