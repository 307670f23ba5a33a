"""``ModelRunner`` with the interface of ``infer/engine/model_runner.py:17-198``: builds the model, sizes
and binds the paged KV cache, turns scheduled sequences into device metadata, runs the step and
samples.

What differs from the reference, by design for this hardware:

* A decode step hands the device ONE staging buffer (last tokens, sequence lengths, block table) in
  one copy; ``positions``, ``slot_mapping`` and ``context_lens`` are derived from it by a kernel that is
  part of the captured graph.  The reference builds five host lists and copies each
  (``model_runner.py:110-126``) and zero-fills its static buffers before every replay (``:144-149``),
  which makes every padding row append to slot 0; here padding rows carry length 0 and get slot -1.
* The metadata kernel is the first node of the captured graph, so a replay needs nothing from the
  host but that one copy.
"""
from __future__ import annotations

import torch

from . import kv_runner, ops
from .config import Config
from .context import reset_context, set_context
from .layers import Sampler
from .qwen3 import QwenForCausalLM, init_random_weights
from .sampling_params import SamplingParams
from .sequence import Sequence


class ModelRunner:

    def __init__(self, config: Config, device: str = "cuda:0"):
        self.config = config
        hf_config = config.hf_config
        self.block_size = config.kvcache_block_size
        self.enforce_eager = config.enforce_eager
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)

        self.model = QwenForCausalLM(hf_config).to(device=self.device, dtype=hf_config.torch_dtype)
        self.load_weights()
        self.sampler = Sampler()
        self.graphs: dict = {}
        self.graph_bs: list[int] = []
        self.graph_pool = None
        self.warmup_model()
        self.allocate_kv_cache()
        self._alloc_step_buffers()
        if not self.enforce_eager:
            self.capture_cudagraph()

    # ------------------------------------------------------------------ set-up
    def load_weights(self):
        from .weight_loader import has_checkpoint, load_model
        if self.config.model and has_checkpoint(self.config.model):
            load_model(self.model, self.config.model)
        else:
            init_random_weights(self.model, self.config.seed)

    def warmup_model(self):
        """One prefill of the largest batch the scheduler may form, so that the peak of everything
        but the KV cache is known before the cache is sized (``model_runner.py:37-45``)."""
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats(self.device)
        max_tokens, max_len = self.config.max_num_batched_tokens, self.config.max_model_len
        num_seqs = max(1, min(max_tokens // max_len, self.config.max_num_seqs))
        seqs = [Sequence([0] * max_len, SamplingParams(temperature=0.7, max_tokens=512)) for _ in range(num_seqs)]
        self.run(seqs, True)
        torch.cuda.empty_cache()
        # what a decode step needs beyond the model is allocated now, before the pool is sized from what
        # is left: the split-KV workspace for the largest batch and the split-K GEMM's partial sums
        hf = self.config.hf_config
        ops.decode_workspace(self.device, min(self.config.max_num_seqs, 512), hf.num_attention_heads,
                             hf.num_key_value_heads, hf.head_dim)
        ops._gemm_workspace(self.device, 64 << 20)

    def allocate_kv_cache(self):
        config, hf = self.config, self.config.hf_config
        if config.num_kvcache_blocks <= 0:
            free, total = torch.cuda.mem_get_info(self.device)
            stats = torch.cuda.memory_stats(self.device)
            block_bytes = kv_runner.kv_block_bytes(hf.num_hidden_layers, self.block_size, hf.num_key_value_heads,
                                                   hf.head_dim, hf.torch_dtype.itemsize)
            config.num_kvcache_blocks = kv_runner.num_kvcache_blocks(
                total, total - free, stats["allocated_bytes.all.peak"], stats["allocated_bytes.all.current"],
                config.gpu_memory_utilization, block_bytes)
        assert config.num_kvcache_blocks > 0
        self.kv_cache = kv_runner.allocate_kv_cache(config.num_kvcache_blocks, hf.num_hidden_layers, self.block_size,
                                                    hf.num_key_value_heads, hf.head_dim, self.device, hf.torch_dtype)
        assert kv_runner.bind_kv_cache(self.model, self.kv_cache) == hf.num_hidden_layers

    def _alloc_step_buffers(self):
        """Static buffers of a decode step.  The staging buffer is one int32 array
        ``[input_ids | seq_lens | block_table]`` that exists twice, pinned on the host and on the device."""
        config = self.config
        self.max_bs = min(config.max_num_seqs, 512)
        self.max_num_blocks = (config.max_model_len + self.block_size - 1) // self.block_size
        n, m = self.max_bs, self.max_num_blocks
        self.stage_host = torch.zeros(n * (2 + m), dtype=torch.int32, pin_memory=True)
        self.stage_dev = torch.zeros(n * (2 + m), dtype=torch.int32, device=self.device)
        host = self.stage_host.numpy()
        self.h_input_ids, self.h_seq_lens = host[:n], host[n:2 * n]
        self.h_block_tables = host[2 * n:].reshape(n, m)
        self._staged_tables = [None] * n        # what each host row of the block table currently holds
        self.d_input_ids, self.d_seq_lens = self.stage_dev[:n], self.stage_dev[n:2 * n]
        self.d_block_tables = self.stage_dev[2 * n:].view(n, m)
        self.d_positions = torch.zeros(n, dtype=torch.int64, device=self.device)
        self.d_slot_mapping = torch.full((n,), -1, dtype=torch.int32, device=self.device)
        self.d_context_lens = torch.zeros(n, dtype=torch.int32, device=self.device)
        # split-KV workspace of the decode kernel for the largest batch, so that no step allocates
        hf = config.hf_config
        ops.decode_workspace(self.device, n, hf.num_attention_heads, hf.num_key_value_heads, hf.head_dim)

    # ------------------------------------------------------------------ per-step metadata
    def prepare_block_tables(self, seqs: list[Sequence]):
        return kv_runner.prepare_block_tables(seqs, self.device)

    def prepare_prefill(self, seqs: list[Sequence]):
        return kv_runner.prepare_prefill(seqs, self.device)

    def prepare_decode(self, seqs: list[Sequence]) -> int:
        """Stages last tokens, lengths and block tables of the batch and returns the batch size the
        step runs at (the captured size that fits, or the exact size when running eagerly)."""
        bs = len(seqs)
        if bs > self.max_bs:
            raise RuntimeError(f"decode batch of {bs} exceeds max_num_seqs={self.max_bs}")
        run_bs = bs if self.enforce_eager or not self.graph_bs else next(x for x in self.graph_bs if x >= bs)
        ids, lens, tables = self.h_input_ids, self.h_seq_lens, self.h_block_tables
        ids[:bs] = [seq.last_token for seq in seqs]
        lens[:bs] = [len(seq) for seq in seqs]
        staged = self._staged_tables
        for i, seq in enumerate(seqs):
            bt = tuple(seq.block_table)
            if staged[i] == bt:          # a row changes once per block of tokens: skip the rewrite otherwise
                continue
            if len(bt) > self.max_num_blocks:
                raise RuntimeError(f"sequence of {len(seq)} tokens exceeds max_model_len={self.config.max_model_len}")
            tables[i, :len(bt)] = bt
            staged[i] = bt
        ids[bs:run_bs] = 0
        lens[bs:run_bs] = 0           # padding rows: no append, no attention
        self.stage_dev.copy_(self.stage_host, non_blocking=True)
        return run_bs

    def _decode_forward(self, run_bs: int) -> torch.Tensor:
        """Metadata kernel + model on the first ``run_bs`` rows of the static buffers; returns the
        final hidden states."""
        positions = self.d_positions[:run_bs]
        slot_mapping = self.d_slot_mapping[:run_bs]
        context_lens = self.d_context_lens[:run_bs]
        block_tables = self.d_block_tables[:run_bs]
        ops.decode_metadata(self.d_seq_lens[:run_bs], block_tables, self.block_size,
                            self.config.decode_position_offset, positions, slot_mapping, context_lens)
        set_context(False, slot_mapping=slot_mapping, context_lens=context_lens, block_tables=block_tables)
        return self.model(self.d_input_ids[:run_bs], positions)

    def prepare_sample(self, seqs: list[Sequence]):
        temps = [seq.temperature for seq in seqs]
        all_greedy = all(t == 0 for t in temps)
        if all_greedy:       # the sampler takes the argmax and never looks at the temperatures
            return None, True
        t = torch.tensor(temps, dtype=torch.float32, pin_memory=True).to(self.device, non_blocking=True)
        return t, all_greedy

    # ------------------------------------------------------------------ the step
    @torch.inference_mode()
    def run_model(self, seqs: list[Sequence], is_prefill: bool) -> torch.Tensor:
        if is_prefill:
            input_ids, positions = self.prepare_prefill(seqs)
            return self.model.compute_logits(self.model(input_ids, positions))
        run_bs = self.prepare_decode(seqs)
        return self.model.compute_logits(self.decode_hidden(run_bs)[:len(seqs)])

    def decode_hidden(self, run_bs: int) -> torch.Tensor:
        """Final hidden states of the staged decode step: the replay of the graph captured for ``run_bs``
        rows, or the eager forward when there is none (``model_runner.py:139-153``)."""
        if self.enforce_eager or run_bs not in self.graphs:
            return self._decode_forward(run_bs)
        self.graphs[run_bs].replay()
        return self.d_outputs

    def run(self, seqs: list[Sequence], is_prefill: bool) -> list[int]:
        temperatures, all_greedy = self.prepare_sample(seqs)
        logits = self.run_model(seqs, is_prefill)
        with torch.inference_mode():
            token_ids = self.sampler(logits, temperatures, all_greedy).tolist()
        reset_context()
        return token_ids

    # ------------------------------------------------------------------ HIP graph capture
    @torch.inference_mode()
    def capture_cudagraph(self):
        """One graph per batch size of ``[1, 2, 4, 8, 16, 32, ...]`` (``model_runner.py:163-198``), largest
        first so that all share one memory pool.  Every kernel of a replay reads the static buffers."""
        self.graph_bs = [b for b in [1, 2, 4, 8] if b <= self.max_bs] + list(range(16, self.max_bs + 1, 16))
        self.d_outputs = torch.zeros(self.max_bs, self.config.hf_config.hidden_size,
                                     dtype=self.config.hf_config.torch_dtype, device=self.device)
        self.h_seq_lens[:] = 0
        self.h_input_ids[:] = 0
        self.stage_dev.copy_(self.stage_host)
        for bs in reversed(self.graph_bs):
            graph = torch.cuda.CUDAGraph()
            self._decode_forward(bs)                       # warm-up: library handles, workspaces
            torch.cuda.synchronize(self.device)
            with torch.cuda.graph(graph, self.graph_pool):
                self.d_outputs[:bs] = self._decode_forward(bs)
            if self.graph_pool is None:
                self.graph_pool = graph.pool()
            self.graphs[bs] = graph
            torch.cuda.synchronize(self.device)
            reset_context()
