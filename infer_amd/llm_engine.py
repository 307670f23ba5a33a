"""``LLMEngine`` with the interface of ``infer/engine/llm_engine.py:12-83``: ``add_request``, ``step``,
``generate``.  A tokenizer is used when the model directory has one; without it prompts are lists of
token ids and the outputs carry token ids only."""
from __future__ import annotations

import os
from dataclasses import fields
from time import perf_counter

from .config import Config
from .model_runner import ModelRunner
from .sampling_params import SamplingParams
from .scheduler import Scheduler
from .sequence import Sequence


class LLMEngine:

    def __init__(self, model: str = "", **kwargs):
        config_fields = {f.name for f in fields(Config)}
        config = Config(model, **{k: v for k, v in kwargs.items() if k in config_fields})
        self.config = config
        self.model_runner = ModelRunner(config)
        self.tokenizer = None
        if model and os.path.exists(os.path.join(model, "tokenizer.json")):
            from transformers import AutoTokenizer
            self.tokenizer = AutoTokenizer.from_pretrained(model, use_fast=True)
            config.eos = self.tokenizer.eos_token_id
        self.scheduler = Scheduler(config)
        self.stats = {"prefill_tokens": 0, "prefill_s": 0.0, "decode_tokens": 0, "decode_s": 0.0,
                      "prefill_steps": 0, "decode_steps": 0}

    def add_request(self, prompt: str | list[int], sampling_params: SamplingParams):
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise RuntimeError("a text prompt needs a tokenizer; pass token ids instead")
            prompt = self.tokenizer.encode(prompt)
        self.scheduler.add(Sequence(prompt, sampling_params))

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    def step(self):
        seqs, is_prefill = self.scheduler.schedule()
        token_ids = self.model_runner.run(seqs, is_prefill)
        self.scheduler.postprocess(seqs, token_ids)
        outputs = [(seq.seq_id, seq.completion_token_ids) for seq in seqs if seq.is_finished]
        # a negative count marks a decode step, as in the reference
        num_tokens = sum(len(seq) for seq in seqs) if is_prefill else -len(seqs)
        return outputs, num_tokens

    def generate(self, prompts: list[str] | list[list[int]], sampling_params: SamplingParams | list[SamplingParams],
                 use_tqdm: bool = False):
        pbar = None
        if use_tqdm:
            from tqdm.auto import tqdm
            pbar = tqdm(total=len(prompts), desc="Generating", dynamic_ncols=True)
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        for prompt, sp in zip(prompts, sampling_params):
            self.add_request(prompt, sp)
        output_dict = {}
        while not self.is_finished():
            t = perf_counter()
            output, num_tokens = self.step()
            dt = perf_counter() - t
            if num_tokens > 0:
                self.stats["prefill_tokens"] += num_tokens
                self.stats["prefill_s"] += dt
                self.stats["prefill_steps"] += 1
            else:
                self.stats["decode_tokens"] += -num_tokens
                self.stats["decode_s"] += dt
                self.stats["decode_steps"] += 1
            for seq_id, token_ids in output:
                output_dict[seq_id] = token_ids
                if pbar is not None:
                    pbar.update(1)
        if pbar is not None:
            pbar.close()
        outputs = [output_dict[seq_id] for seq_id in sorted(output_dict)]
        return [{"text": self.tokenizer.decode(t) if self.tokenizer is not None else None, "token_ids": t}
                for t in outputs]
