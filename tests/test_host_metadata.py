"""Host logic of a step (infer_amd/kv_runner.py, sequence.py, context.py) against the oracle's closed
forms (oracle/paged_ref.py: decode_metadata_ref / prefill_metadata_ref).  Runs on the CPU."""
import numpy as np
import pytest
import torch

from infer_amd import kv_runner
from infer_amd.block_manager import BlockManager
from infer_amd.context import get_context, reset_context
from infer_amd.sequence import Sequence
from oracle import paged_ref


@pytest.fixture(autouse=True)
def block16():
    old = Sequence.block_size
    Sequence.block_size = 16
    yield
    Sequence.block_size = old
    reset_context()


def make_seqs(lengths, pool):
    seqs = []
    for i, n in enumerate(lengths):
        s = Sequence([(7 * i + t) % 50 for t in range(n)])
        pool.allocate(s)
        seqs.append(s)
    return seqs


def test_prepare_decode_matches_closed_form():
    pool = BlockManager(32, 16)
    seqs = make_seqs([40, 16, 33, 1], pool)
    ids, pos = kv_runner.prepare_decode(seqs, device="cpu")
    ctx = get_context()
    slots, lens, padded = paged_ref.decode_metadata_ref([len(s) for s in seqs], [s.block_table for s in seqs], 16)
    assert not ctx.is_prefill
    assert ctx.slot_mapping.dtype == torch.int32 and ctx.context_lens.dtype == torch.int32
    assert ctx.block_tables.dtype == torch.int32
    assert np.array_equal(ctx.slot_mapping.numpy(), slots)
    assert np.array_equal(ctx.context_lens.numpy(), lens)
    assert np.array_equal(ctx.block_tables.numpy(), padded)
    assert ids.tolist() == [s.last_token for s in seqs]
    assert pos.tolist() == [len(s) for s in seqs]          # the reference's decode position (model_runner.py:117)


def test_prepare_prefill_with_and_without_prefix():
    pool = BlockManager(32, 16)
    first = make_seqs([40], pool)                           # nothing cached yet
    kv_runner.prepare_prefill(first, device="cpu")
    ctx = get_context()
    assert ctx.is_prefill and ctx.block_tables is None      # no prefix hit -> no block tables (:100-101)
    assert ctx.cu_seqlens_q.tolist() == [0, 40] == ctx.cu_seqlens_k.tolist()
    # a second sequence sharing the first 32 tokens hits two cached blocks
    s2 = Sequence(first[0].token_ids[:32] + [3, 4, 5])
    pool.allocate(s2)
    assert s2.num_cached_tokens == 32
    s3 = Sequence(list(range(100, 120)))
    pool.allocate(s3)
    ids, pos = kv_runner.prepare_prefill([s2, s3], device="cpu")
    ctx = get_context()
    cu_q, cu_k, max_q, max_k, slots = paged_ref.prefill_metadata_ref(
        [len(s2), len(s3)], [32, 0], [s2.block_table, s3.block_table], 16)
    assert np.array_equal(ctx.cu_seqlens_q.numpy(), cu_q) and np.array_equal(ctx.cu_seqlens_k.numpy(), cu_k)
    assert (ctx.max_seqlen_q, ctx.max_seqlen_k) == (max_q, max_k)
    assert np.array_equal(ctx.slot_mapping.numpy(), slots)
    assert ctx.block_tables is not None and ctx.block_tables.shape == (2, 3)
    assert ids.tolist() == s2.token_ids[32:] + s3.token_ids
    assert pos.tolist() == list(range(32, 35)) + list(range(20))


def test_cache_sizing_formula():
    # Qwen3-8B: 36 layers, block 256, 8 KV heads, head_dim 128, bf16 -> 37.7 MB per block
    bb = kv_runner.kv_block_bytes(36, 256, 8, 128)
    assert bb == 2 * 36 * 256 * 8 * 128 * 2 == 37748736
    total = 288 * 2 ** 30
    assert kv_runner.num_kvcache_blocks(total, 20 * 2 ** 30, 18 * 2 ** 30, 16 * 2 ** 30, 0.9, bb) == \
        int(total * 0.9 - 20 * 2 ** 30 - 18 * 2 ** 30 + 16 * 2 ** 30) // bb


def test_bind_kv_cache_hands_out_layer_views():
    from infer_amd.attention import Attention
    model = torch.nn.Sequential(Attention(4, 8, 1.0, 2), torch.nn.Linear(2, 2), Attention(4, 8, 1.0, 2))
    kv = kv_runner.allocate_kv_cache(3, 2, 16, 2, 8, device="cpu")
    assert kv_runner.bind_kv_cache(model, kv) == 2
    assert model[2].k_cache.data_ptr() == kv[0, 1].data_ptr() and model[0].v_cache.data_ptr() == kv[1, 0].data_ptr()
    assert model[0].k_cache.stride(1) == 2 * 8      # what store_kvcache asserts (attention.py:43)


def test_attention_module_refuses_cpu_tensors():
    from infer_amd.attention import Attention
    from infer_amd.context import set_context
    att = Attention(4, 128, 1.0, 2)
    att.k_cache = torch.zeros(2, 16, 2, 128, dtype=torch.bfloat16)
    att.v_cache = torch.zeros(2, 16, 2, 128, dtype=torch.bfloat16)
    set_context(False, slot_mapping=torch.zeros(1, dtype=torch.int32), context_lens=torch.ones(1, dtype=torch.int32),
                block_tables=torch.zeros(1, 1, dtype=torch.int32))
    q = torch.zeros(1, 4 * 128, dtype=torch.bfloat16)
    kv = torch.zeros(1, 2 * 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        att(q, kv, kv)       # no CPU fallback: the HIP kernels are the only implementation
