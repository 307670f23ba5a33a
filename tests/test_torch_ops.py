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
    with pytest.raises(AttributeError, match="outside the paged KV-cache path"):
        infer_ops.rms_norm


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
