"""Pins ``oracle/qwen3_ref.py`` (the float32 whole-model restatement used to check the engine) against
the independent Qwen3 implementation of the ``transformers`` package, and checks the host-side
pieces of the engine that need no GPU: scheduler invariants and the sequence wire form."""
import math
import pickle

import pytest
import torch

from infer_amd.config import Config, ModelConfig
from infer_amd.sampling_params import SamplingParams
from infer_amd.scheduler import Scheduler
from infer_amd.sequence import Sequence, SequenceStatus
from oracle import qwen3_ref

TINY = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
            num_key_value_heads=2, head_dim=128, max_position_embeddings=2048, rope_theta=1e6, rms_norm_eps=1e-6,
            tie_word_embeddings=False)


def _hf_model():
    transformers = pytest.importorskip("transformers")
    from transformers.models.qwen3.modeling_qwen3 import Qwen3ForCausalLM
    torch.manual_seed(1)
    model = Qwen3ForCausalLM(transformers.Qwen3Config(**TINY)).eval().float()
    with torch.no_grad():                      # norm weights away from one so that they matter
        for name, p in model.named_parameters():
            if "norm" in name:
                p.copy_(1.0 + 0.1 * torch.randn_like(p))
    return model


def _packed(state: dict) -> dict:
    out = {}
    for name, t in state.items():
        if any(k in name for k in ("q_proj", "k_proj", "v_proj", "gate_proj", "up_proj")):
            continue
        out[name] = t
    for l in range(TINY["num_hidden_layers"]):
        p = f"model.layers.{l}."
        out[p + "self_attn.qkv_proj.weight"] = torch.cat(
            [state[p + f"self_attn.{n}_proj.weight"] for n in "qkv"], dim=0)
        out[p + "mlp.gate_up_proj.weight"] = torch.cat(
            [state[p + "mlp.gate_proj.weight"], state[p + "mlp.up_proj.weight"]], dim=0)
    return out


def test_oracle_matches_transformers_qwen3():
    model = _hf_model()
    cfg = ModelConfig(**TINY)
    weights = _packed(model.state_dict())
    torch.manual_seed(2)
    for T in (1, 7, 40):
        tokens = torch.randint(0, TINY["vocab_size"], (T,))
        with torch.no_grad():
            want = model(tokens[None]).logits[0]
        got = qwen3_ref.forward_full(weights, cfg, tokens, list(range(T)))
        assert torch.allclose(got, want, atol=1e-4, rtol=1e-4), (T, (got - want).abs().max())


def test_oracle_positions_matter_and_shift_is_relative():
    """Rotary attention depends on position differences only: shifting all positions leaves the
    logits unchanged, shifting some of them does not (so a wrong position would be seen)."""
    model = _hf_model()
    cfg = ModelConfig(**TINY)
    weights = _packed(model.state_dict())
    tokens = torch.randint(0, TINY["vocab_size"], (12,), generator=torch.Generator().manual_seed(3))
    base = qwen3_ref.forward_full(weights, cfg, tokens, list(range(12)))
    shifted = qwen3_ref.forward_full(weights, cfg, tokens, [p + 5 for p in range(12)])
    assert torch.allclose(base, shifted, atol=2e-4)
    bent = qwen3_ref.forward_full(weights, cfg, tokens, qwen3_ref.engine_positions(8, 12, 1))
    assert (bent[-1] - base[-1]).abs().max() > 1e-4
    assert torch.allclose(bent[:8], base[:8], atol=1e-5)       # causal: the prompt part is untouched


def test_oracle_attention_core_vs_scalar_loop():
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(9, 16, generator=g) for _ in range(3))
    want = qwen3_ref.attention_scalar(q, k, v, 1 / math.sqrt(16))
    s = (q @ k.T) / math.sqrt(16)
    s = s.masked_fill(~torch.ones(9, 9, dtype=torch.bool).tril(), float("-inf"))
    assert torch.allclose((torch.softmax(s, -1) @ v).double(), want, atol=1e-5)


def test_engine_positions():
    assert qwen3_ref.engine_positions(3, 6, 1) == [0, 1, 2, 4, 5, 6]
    assert qwen3_ref.engine_positions(3, 6, 0) == [0, 1, 2, 3, 4, 5]


# ---------------------------------------------------------------------------- scheduler (host only)

def _config(num_blocks, **kw):
    return Config(hf_config=ModelConfig(**TINY), num_kvcache_blocks=num_blocks, max_model_len=2048,
                  max_num_batched_tokens=kw.pop("max_num_batched_tokens", 4096), **kw)


def _drive(sched: Scheduler, steps=10_000):
    """Runs the scheduler with a fake model (next token = step counter) and checks pool invariants."""
    order = []
    n = 0
    while not sched.is_finished():
        seqs, is_prefill = sched.schedule()
        assert seqs
        bm = sched.block_manager
        for s in seqs:
            assert s.status == SequenceStatus.RUNNING
            assert len(s.block_table) == s.num_blocks
        tables = [b for s in sched.running for b in s.block_table]
        assert set(tables) <= bm.used_block_ids
        assert bm.num_free_blocks + len(bm.used_block_ids) == bm.num_blocks
        order.append((is_prefill, [s.seq_id for s in seqs]))
        sched.postprocess(seqs, [1000 + n] * len(seqs))
        n += 1
        assert n < steps
    return order


def test_scheduler_prefill_first_then_decode_until_done():
    sched = Scheduler(_config(64, max_num_seqs=8))
    seqs = [Sequence(list(range(10 * i, 10 * i + 300 + i)), SamplingParams(0.0, 5, True)) for i in range(3)]
    for s in seqs:
        sched.add(s)
    order = _drive(sched)
    assert order[0][0] is True and len(order[0][1]) == 3
    assert all(not p for p, _ in order[1:])
    assert len(order) == 1 + 4                      # the prefill yields token 1, four decodes the rest
    assert all(s.is_finished and s.num_completion_tokens == 5 for s in seqs)
    assert sched.block_manager.num_free_blocks == 64


def test_scheduler_token_budget_splits_prefill():
    sched = Scheduler(_config(64, max_num_seqs=8, max_num_batched_tokens=2048))
    for i in range(3):
        sched.add(Sequence([i] * 1000, SamplingParams(0.0, 2, True)))
    order = _drive(sched)
    assert order[0] == (True, order[0][1]) and len(order[0][1]) == 2     # 2 x 1000 fit, the third waits
    assert order[1][0] is True and len(order[1][1]) == 1


def test_scheduler_preempts_youngest_when_pool_runs_dry():
    # two sequences of 256 tokens fill one block each; the pool has exactly two blocks, so the first
    # decode step (token 257 opens a block) must evict the younger sequence and later re-run it
    sched = Scheduler(_config(3, max_num_seqs=4))
    a = Sequence(list(range(256)), SamplingParams(0.0, 3, True))
    b = Sequence(list(range(500, 756)), SamplingParams(0.0, 3, True))
    c = Sequence(list(range(900, 1156)), SamplingParams(0.0, 3, True))
    for s in (a, b, c):
        sched.add(s)
    order = _drive(sched)
    assert all(s.is_finished and s.num_completion_tokens == 3 for s in (a, b, c))
    prefills = [ids for p, ids in order if p]
    assert sum(len(ids) for ids in prefills) > 3        # somebody was prefetched twice: a preemption happened
    assert sched.block_manager.num_free_blocks == 3


def test_scheduler_eos_stops_a_sequence():
    cfg = _config(16, max_num_seqs=4)
    cfg.eos = 1001
    sched = Scheduler(cfg)
    s = Sequence([1, 2, 3], SamplingParams(0.0, 50, False))
    sched.add(s)
    _drive(sched)
    assert s.completion_token_ids == [1000, 1001]


def test_sequence_wire_form_roundtrip():
    s = Sequence([5, 6, 7], SamplingParams(0.5, 9, True))
    s.block_table = [4]
    t = pickle.loads(pickle.dumps(s))
    assert t.token_ids == [5, 6, 7] and t.num_tokens == 3 and t.block_table == [4]
    s.append_token(8)
    t = pickle.loads(pickle.dumps(s))
    assert t.last_token == 8 and t.num_tokens == 4 and not hasattr(t, "token_ids")


def test_weight_loader_maps_a_checkpoint_onto_the_packed_parameters(tmp_path):
    """A checkpoint in the published tensor naming (separate q/k/v and gate/up projections), written
    by the ``transformers`` model, must land in the engine's packed parameters so that the oracle on
    the loaded weights reproduces the ``transformers`` logits."""
    from safetensors.torch import save_file
    from infer_amd.qwen3 import QwenForCausalLM
    from infer_amd.weight_loader import has_checkpoint, load_model
    model = _hf_model()
    assert not has_checkpoint(str(tmp_path))
    state = {k: v.to(torch.bfloat16).contiguous() for k, v in model.state_dict().items()}
    names = sorted(state)
    save_file({k: state[k] for k in names[::2]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({k: state[k] for k in names[1::2]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    (tmp_path / "config.json").write_text(__import__("json").dumps({**TINY, "torch_dtype": "bfloat16"}))
    assert has_checkpoint(str(tmp_path))
    cfg = Config(model=str(tmp_path), max_model_len=2048)
    assert cfg.hf_config.num_key_value_heads == 2 and cfg.hf_config.torch_dtype == torch.bfloat16
    engine_model = QwenForCausalLM(cfg.hf_config)
    assert load_model(engine_model, str(tmp_path)) == len(state)
    want = _packed(state)
    got = dict(engine_model.named_parameters())
    assert set(got) == set(want)
    for name in want:
        assert torch.equal(got[name].data, want[name]), name
    tokens = torch.randint(0, TINY["vocab_size"], (9,), generator=torch.Generator().manual_seed(8))
    model_bf = _hf_model()                                      # same rounded weights on both sides
    model_bf.load_state_dict({k: v.float() for k, v in state.items()})
    with torch.no_grad():
        ref = model_bf(tokens[None]).logits[0]
    mine = qwen3_ref.forward_full(got, cfg.hf_config, tokens, list(range(9)))
    assert torch.allclose(mine, ref, atol=1e-4, rtol=1e-4)
