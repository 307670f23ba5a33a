"""The engine end to end on the GPU (scheduler -> model runner -> fused front end -> paged attention ->
sampler) on a tiny random Qwen3, against ``oracle/qwen3_ref.py`` (float32, dense attention over the
whole sequence, pinned against the ``transformers`` implementation on the CPU).

Bar: logits of every step within ``LOGIT_TOL`` (relative to the largest logit of the row; the model
computes in bf16, the oracle in float32); the token the engine picks is within that tolerance of the
oracle's best token; a HIP-graph replay is bit-identical to the eager step on the same inputs."""
import numpy as np
import pytest
import torch

from infer_amd.config import Config, ModelConfig
from infer_amd.context import reset_context
from infer_amd.sampling_params import SamplingParams
from oracle import qwen3_ref

pytestmark = pytest.mark.gpu

TINY = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
            num_key_value_heads=2, head_dim=128, max_position_embeddings=2048, rope_theta=1e6, rms_norm_eps=1e-6,
            tie_word_embeddings=False)
LOGIT_TOL = 4e-2


def make_config(**kw):
    base = dict(hf_config=ModelConfig(**TINY), num_kvcache_blocks=24, max_model_len=2048,
                max_num_batched_tokens=4096, max_num_seqs=16, enforce_eager=True, seed=11)
    base.update(kw)
    return Config(**base)


def prompts(lengths, seed=0):
    g = np.random.default_rng(seed)
    return [[int(t) for t in g.integers(0, TINY["vocab_size"], size=n)] for n in lengths]


def oracle_logits(runner, seq, offset):
    """Oracle logits for the newest token of ``seq``, from the engine's weights, its rotary table and the
    positions it feeds."""
    from infer_amd.layers import cos_sin_table
    cfg = runner.config.hf_config
    table = cos_sin_table(cfg.head_dim, cfg.max_position_embeddings, cfg.rope_theta, runner.device)
    pos = qwen3_ref.engine_positions(seq.num_prompt_tokens, len(seq), offset)
    return qwen3_ref.forward_full(dict(runner.model.named_parameters()), cfg, seq.token_ids, pos, table)[-1]


def check_step(runner, seqs, logits, offset):
    picked = logits.float().argmax(dim=-1).tolist()
    for seq, row, tok in zip(seqs, logits.float().cpu(), picked):
        want = oracle_logits(runner, seq, offset)
        scale = want.abs().max().item()
        assert torch.isfinite(row).all()
        assert (row - want).abs().max().item() <= LOGIT_TOL * scale, (len(seq), (row - want).abs().max().item(), scale)
        assert want.max().item() - want[tok].item() <= 2 * LOGIT_TOL * scale
    return picked


@pytest.mark.parametrize("offset", [1, 0])
def test_prefill_then_decode_steps_match_oracle(gpu, offset):
    from infer_amd.model_runner import ModelRunner
    from infer_amd.scheduler import Scheduler
    from infer_amd.sequence import Sequence
    config = make_config(decode_position_offset=offset)
    runner = ModelRunner(config)
    sched = Scheduler(config)
    for p in prompts([5, 300, 517]):
        sched.add(Sequence(p, SamplingParams(0.0, 6, True)))
    steps = 0
    while not sched.is_finished():
        seqs, is_prefill = sched.schedule()
        assert is_prefill == (steps == 0)
        logits = runner.run_model(seqs, is_prefill)
        reset_context()
        tokens = check_step(runner, seqs, logits, offset)
        sched.postprocess(seqs, tokens)
        steps += 1
    assert steps == 6


def test_graph_replay_is_bit_identical_to_eager_and_padding_rows_touch_nothing(gpu):
    from infer_amd.model_runner import ModelRunner
    from infer_amd.scheduler import Scheduler
    from infer_amd.sequence import Sequence
    config = make_config(enforce_eager=False, max_num_seqs=16)
    runner = ModelRunner(config)
    assert runner.graph_bs == [1, 2, 4, 8, 16] and set(runner.graphs) == set(runner.graph_bs)
    sched = Scheduler(config)
    seqs = [Sequence(p, SamplingParams(0.0, 8, True)) for p in prompts([40, 255, 256], seed=3)]
    for s in seqs:
        sched.add(s)
    batch, is_prefill = sched.schedule()
    sched.postprocess(batch, runner.run(batch, is_prefill))
    owned = {b for s in seqs for b in s.block_table}
    runner.kv_cache[:, :, [b for b in range(config.num_kvcache_blocks) if b not in owned]] = 77.0
    for step in range(5):
        batch, is_prefill = sched.schedule()
        assert not is_prefill and len(batch) == 3
        owned |= {b for s in seqs for b in s.block_table}
        run_bs = runner.prepare_decode(batch)
        assert run_bs == 4                                   # three sequences ride the graph of four
        with torch.inference_mode():
            eager = runner._decode_forward(run_bs).clone()
            reset_context()
            torch.cuda.synchronize()
            runner.graphs[run_bs].replay()
            torch.cuda.synchronize()
            replay = runner.d_outputs[:run_bs].clone()
            assert torch.equal(eager[:3], replay[:3]), f"replay {step} differs from eager"
            logits = runner.model.compute_logits(replay[:3])
        tokens = check_step(runner, batch, logits, config.decode_position_offset)
        sched.postprocess(batch, tokens)
    free = [b for b in range(config.num_kvcache_blocks) if b not in owned]
    assert (runner.kv_cache[:, :, free] == 77.0).all()       # the padding row wrote to no block


def test_graph_replays_at_qwen3_8b_layer_shapes_match_eager(gpu):
    """Two layers of the real Qwen3-8B geometry (hidden 4096, 32/8 heads, intermediate 12288), batch
    128: the vendor GEMMs that a replay runs are the ones of the full model.  Five replays, with eager
    work and synchronisation between them, must each reproduce the eager step bit for bit (a graph
    node that misbehaves on later replays, such as a memset recorded by a library, would show here)."""
    from infer_amd.model_runner import ModelRunner
    from infer_amd.scheduler import Scheduler
    from infer_amd.sequence import Sequence
    hf = ModelConfig(vocab_size=2048, hidden_size=4096, intermediate_size=12288, num_hidden_layers=2,
                     num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=4096)
    config = Config(hf_config=hf, num_kvcache_blocks=300, max_model_len=4096, max_num_batched_tokens=16384,
                    max_num_seqs=128, enforce_eager=False, seed=3)
    runner = ModelRunner(config)
    sched = Scheduler(config)
    g = np.random.default_rng(1)
    seqs = [Sequence([int(t) for t in g.integers(0, 2048, size=int(n))], SamplingParams(0.0, 8, True))
            for n in g.integers(64, 300, size=128)]
    for s in seqs:
        sched.add(s)
    while sched.waiting:                                  # the token budget splits the prefill in two
        batch, is_prefill = sched.schedule()
        assert is_prefill
        sched.postprocess(batch, runner.run(batch, True))
    for step in range(5):
        batch, is_prefill = sched.schedule()
        assert not is_prefill and len(batch) == 128
        run_bs = runner.prepare_decode(batch)
        assert run_bs == 128
        with torch.inference_mode():
            eager = runner._decode_forward(run_bs).clone()
            reset_context()
            torch.cuda.synchronize()
            runner.graphs[run_bs].replay()
            torch.cuda.synchronize()
            replay = runner.d_outputs[:run_bs]
            assert torch.isfinite(replay.float()).all()
            assert torch.equal(eager, replay), f"replay {step} differs from the eager step"
            tokens = runner.model.compute_logits(replay).float().argmax(dim=-1).tolist()
        sched.postprocess(batch, tokens)


def test_qwen3_8b_geometry_prefill_and_decode_steps_match_oracle(gpu):
    """Two layers of the Qwen3-8B geometry of the end-to-end configuration (hidden 4096, 32 query and 8 KV
    heads of 128, intermediate 12288), batch 16 with mixed prompt lengths on both sides of a block
    boundary: one prefill and three decode steps, the decode steps as HIP-graph replays.  The logits of
    every step are compared with the float32 whole-sequence oracle (one oracle pass per sequence over its
    final tokens gives the rows of all four steps: dense causal attention does not look ahead)."""
    from infer_amd.layers import cos_sin_table
    from infer_amd.model_runner import ModelRunner
    from infer_amd.scheduler import Scheduler
    from infer_amd.sequence import Sequence
    hf = ModelConfig(vocab_size=2048, hidden_size=4096, intermediate_size=12288, num_hidden_layers=2,
                     num_attention_heads=32, num_key_value_heads=8, head_dim=128, max_position_embeddings=4096)
    config = Config(hf_config=hf, num_kvcache_blocks=64, max_model_len=4096, max_num_batched_tokens=16384,
                    max_num_seqs=16, enforce_eager=False, seed=5)
    runner = ModelRunner(config)
    sched = Scheduler(config)
    g = np.random.default_rng(2)
    lengths = [3, 17, 64, 100, 129, 200, 254, 255, 256, 257, 300, 31, 150, 90, 222, 400]
    seqs = [Sequence([int(t) for t in g.integers(0, hf.vocab_size, size=n)], SamplingParams(0.0, 4, True))
            for n in lengths]
    for s in seqs:
        sched.add(s)
    rows = {id(s): [] for s in seqs}            # logits of each step, per sequence
    for step in range(4):
        batch, is_prefill = sched.schedule()
        assert is_prefill == (step == 0) and len(batch) == 16
        if not is_prefill:
            assert runner.prepare_decode(batch) in runner.graphs     # the step below is a graph replay
        logits = runner.run_model(batch, is_prefill)
        reset_context()
        assert torch.isfinite(logits.float()).all()
        for s, row in zip(batch, logits.float().cpu()):
            rows[id(s)].append(row)
        sched.postprocess(batch, logits.float().argmax(dim=-1).tolist())
    weights = {k: v.detach().float().cpu() for k, v in runner.model.named_parameters()}
    table = cos_sin_table(hf.head_dim, hf.max_position_embeddings, hf.rope_theta, runner.device).float().cpu()
    worst = 0.0
    for s in seqs:
        n = s.num_prompt_tokens
        fed = s.token_ids[:n + 3]               # the prompt and the three tokens fed by the decode steps
        pos = qwen3_ref.engine_positions(n, len(fed), config.decode_position_offset)
        want = qwen3_ref.forward_full(weights, hf, fed, pos, table)
        for k, got in enumerate(rows[id(s)]):
            ref = want[n - 1 + k]
            scale = ref.abs().max().item()
            err = (got - ref).abs().max().item()
            worst = max(worst, err / scale)
            assert err <= LOGIT_TOL * scale, (n, k, err, scale)
            assert ref.max().item() - ref[int(got.argmax())].item() <= 2 * LOGIT_TOL * scale
    print("8B-geometry logits: worst error relative to the largest logit", worst)


def test_generate_graph_and_eager_agree_and_prefix_cache_hits(gpu):
    from infer_amd.llm_engine import LLMEngine
    ps = prompts([30, 130, 260, 511], seed=5)
    sp = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    kw = dict(hf_config=ModelConfig(**TINY), num_kvcache_blocks=24, max_model_len=2048,
              max_num_batched_tokens=4096, max_num_seqs=16, seed=11)
    eager = LLMEngine(enforce_eager=True, **kw)
    graph = LLMEngine(enforce_eager=False, **kw)
    out_e = eager.generate(ps, sp)
    out_g = graph.generate(ps, sp)
    assert [o["token_ids"] for o in out_e] == [o["token_ids"] for o in out_g]
    assert all(len(o["token_ids"]) == 12 for o in out_g)
    assert graph.stats["decode_steps"] == 11 and graph.stats["prefill_steps"] == 1
    assert graph.scheduler.block_manager.num_free_blocks == 24

    # a second request that shares the first 256 tokens of prompt 3 finds that block in the cache
    from infer_amd.sequence import Sequence
    again = ps[3][:256] + prompts([100], seed=9)[0]
    seq = Sequence(again, SamplingParams(0.0, 3, True))
    graph.scheduler.add(seq)
    batch, is_prefill = graph.scheduler.schedule()
    assert is_prefill and seq.num_cached_tokens == 256
    logits = graph.model_runner.run_model(batch, True)
    reset_context()
    tokens = check_step(graph.model_runner, batch, logits, graph.config.decode_position_offset)
    graph.scheduler.postprocess(batch, tokens)
    while not graph.is_finished():
        graph.step()
    assert seq.num_completion_tokens == 3


def test_preemption_under_a_tiny_pool_still_finishes(gpu):
    from infer_amd.llm_engine import LLMEngine
    engine = LLMEngine(hf_config=ModelConfig(**TINY), num_kvcache_blocks=4, max_model_len=2048,
                       max_num_batched_tokens=4096, max_num_seqs=8, enforce_eager=False, seed=11)
    ps = prompts([250, 251, 252], seed=7)
    outs = engine.generate(ps, SamplingParams(0.0, 10, True))
    assert [len(o["token_ids"]) for o in outs] == [10, 10, 10]
    assert engine.stats["prefill_steps"] > 1                 # somebody was evicted and prefetched again
    assert engine.scheduler.block_manager.num_free_blocks == 4


def test_sampler_temperature(gpu):
    from infer_amd.layers import Sampler
    torch.manual_seed(0)
    logits = torch.full((4, 100), -20.0, device=gpu, dtype=torch.bfloat16)
    logits[:, 7] = 20.0
    temps = torch.tensor([0.0, 1.0, 0.5, 0.0], device=gpu)
    assert Sampler()(logits, temps).tolist() == [7, 7, 7, 7]
    assert Sampler()(logits, temps * 0, all_greedy=True).tolist() == [7, 7, 7, 7]
    # the all-greedy shortcut works on the bf16 logits: same tokens as the float path, ties included
    coarse = (torch.randn((64, 50000), device=gpu) * 4).round().to(torch.bfloat16)   # many exact ties
    zeros = torch.zeros(64, device=gpu)
    assert torch.equal(Sampler()(coarse, zeros, all_greedy=True), Sampler()(coarse, zeros))
    assert torch.equal(Sampler()(coarse, zeros, all_greedy=True), coarse.float().argmax(dim=-1))
    flat = torch.zeros((2000, 4), device=gpu)
    draws = Sampler()(flat, torch.ones(2000, device=gpu))
    counts = torch.bincount(draws, minlength=4).float() / 2000
    assert (counts - 0.25).abs().max() < 0.05                # uniform logits: every token about equally often
