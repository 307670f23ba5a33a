"""The request loop: ``LLMEngine.add_request`` / ``step`` / ``generate``.

Interface of the reference's ``infer/engine/llm_engine.py:12-83`` (same call signatures, ``step`` returns the
finished sequences of the step and a token count whose sign tells prefill from decode, ``generate`` returns
one ``{"text", "token_ids"}`` record per prompt in submission order).  A tokenizer is loaded only when the
model directory holds one: without it prompts are lists of token ids and ``text`` is ``None``.  The engine
keeps running totals of tokens and seconds per phase in ``stats`` (the reference prints rates to a progress
bar instead)."""
from __future__ import annotations

import os
from dataclasses import fields
from time import perf_counter

from .config import Config
from .model_runner import ModelRunner
from .sampling_params import SamplingParams
from .scheduler import Scheduler
from .sequence import Sequence


def _load_tokenizer(model_dir: str):
    if not model_dir or not os.path.exists(os.path.join(model_dir, "tokenizer.json")):
        return None
    from transformers import AutoTokenizer
    return AutoTokenizer.from_pretrained(model_dir, use_fast=True)


class LLMEngine:

    def __init__(self, model: str = "", **kwargs):
        known = {f.name for f in fields(Config)}
        self.config = Config(model, **{name: value for name, value in kwargs.items() if name in known})
        self.model_runner = ModelRunner(self.config)          # sizes the KV pool: the scheduler comes after it
        self.tokenizer = _load_tokenizer(model)
        if self.tokenizer is not None:
            self.config.eos = self.tokenizer.eos_token_id
        self.scheduler = Scheduler(self.config)
        self.stats = dict.fromkeys(("prefill_tokens", "prefill_steps", "decode_tokens", "decode_steps"), 0)
        self.stats.update(prefill_s=0.0, decode_s=0.0)

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt: str | list[int], sampling_params: SamplingParams) -> None:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise RuntimeError("a text prompt needs a tokenizer; pass token ids instead")
            prompt = self.tokenizer.encode(prompt)
        self.scheduler.add(Sequence(prompt, sampling_params))

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    # ------------------------------------------------------------------ one step
    def step(self):
        """Runs one scheduled step.  Returns ``(finished, count)``: ``finished`` lists ``(seq_id, completion
        token ids)`` of the sequences that ended in this step; ``count`` is the number of prompt tokens of a
        prefill step, or minus the number of sequences of a decode step."""
        started = perf_counter()
        batch, is_prefill = self.scheduler.schedule()
        sampled = self.model_runner.run(batch, is_prefill)
        self.scheduler.postprocess(batch, sampled)
        count = sum(map(len, batch)) if is_prefill else -len(batch)
        phase = "prefill" if is_prefill else "decode"
        self.stats[phase + "_tokens"] += abs(count)
        self.stats[phase + "_steps"] += 1
        self.stats[phase + "_s"] += perf_counter() - started
        finished = [(seq.seq_id, seq.completion_token_ids) for seq in batch if seq.is_finished]
        return finished, count

    # ------------------------------------------------------------------ batch interface
    def generate(self, prompts: list[str] | list[list[int]], sampling_params: SamplingParams | list[SamplingParams],
                 use_tqdm: bool = False):
        per_prompt = sampling_params if isinstance(sampling_params, list) else [sampling_params] * len(prompts)
        for prompt, params in zip(prompts, per_prompt):
            self.add_request(prompt, params)
        bar = None
        if use_tqdm:
            from tqdm.auto import tqdm
            bar = tqdm(total=len(prompts), desc="Generating", dynamic_ncols=True)
        completions: dict[int, list[int]] = {}
        while not self.is_finished():
            finished, _ = self.step()
            completions.update(finished)
            if bar is not None:
                bar.update(len(finished))
        if bar is not None:
            bar.close()
        decode = self.tokenizer.decode if self.tokenizer is not None else (lambda ids: None)
        # sequence ids grow with submission order
        return [{"text": decode(ids), "token_ids": ids} for _, ids in sorted(completions.items())]
