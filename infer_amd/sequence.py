"""One request as the scheduler, the block pool and the model runner see it.

Interface of the reference's ``infer/engine/sequence.py:8-84`` (attribute and property names, the block
arithmetic, the compact pickled form), written around two counters: how many tokens the sequence holds
and how many of them were the prompt.  ``block_size`` is a class attribute because the reference's block
manager and model runner read it from the class (256 tokens per cache block there)."""
from __future__ import annotations

import itertools
from enum import Enum

from .sampling_params import SamplingParams


class SequenceStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"
    WATING = "waiting"        # alias: the reference spells it this way (``sequence.py:13``)


class Sequence:
    block_size = 256
    counter = itertools.count()

    def __init__(self, token_ids: list[int], sampling_param: SamplingParams | None = None):
        params = sampling_param if sampling_param is not None else SamplingParams()
        prompt = list(token_ids)                 # the caller's list is not aliased
        self.seq_id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = prompt
        self.last_token = prompt[-1]             # IndexError on an empty prompt, as in the reference
        self.num_prompt_tokens = self.num_tokens = len(prompt)
        self.num_cached_tokens = 0               # tokens whose K/V a prefix-cache hit already provides
        self.block_table: list[int] = []         # cache block ids, in sequence order
        self.temperature = params.temperature
        self.max_tokens = params.max_tokens
        self.ignore_eos = params.ignore_eos

    # ------------------------------------------------------------------ tokens
    def __len__(self) -> int:
        return self.num_tokens

    def __getitem__(self, key):
        return self.token_ids[key]

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(token_id)
        self.num_tokens += 1
        self.last_token = token_id

    @property
    def num_completion_tokens(self) -> int:
        return self.num_tokens - self.num_prompt_tokens

    @property
    def prompt_token_ids(self) -> list[int]:
        return self.token_ids[:self.num_prompt_tokens]

    @property
    def completion_token_ids(self) -> list[int]:
        return self.token_ids[self.num_prompt_tokens:]

    @property
    def is_finished(self) -> bool:
        return self.status is SequenceStatus.FINISHED

    # ------------------------------------------------------------------ cache blocks
    @property
    def num_blocks(self) -> int:
        return -(-self.num_tokens // self.block_size)

    @property
    def num_cached_blocks(self) -> int:
        return self.num_cached_tokens // self.block_size

    @property
    def last_block_num_tokens(self) -> int:
        """Tokens in the last, possibly partial block (``block_size`` when it is full)."""
        return self.num_tokens - self.block_size * (self.num_blocks - 1)

    def block(self, i: int) -> list[int]:
        """Token ids of block ``i``."""
        if not 0 <= i < self.num_blocks:
            raise AssertionError(f"block {i} of a sequence of {self.num_blocks} blocks")
        lo = i * self.block_size
        return self.token_ids[lo:lo + self.block_size]

    # ------------------------------------------------------------------ wire form
    # What travels between processes (``sequence.py:75-84``): the three counters, the block table and
    # either all token ids (nothing generated yet: the receiver has to prefill) or the last token alone.
    def __getstate__(self):
        tail = self.last_token if self.num_completion_tokens else self.token_ids
        return (self.num_tokens, self.num_prompt_tokens, self.num_cached_tokens, self.block_table, tail)

    def __setstate__(self, state):
        *head, tail = state
        self.num_tokens, self.num_prompt_tokens, self.num_cached_tokens, self.block_table = head
        if self.num_completion_tokens:
            self.last_token = tail
        else:
            self.token_ids = tail
