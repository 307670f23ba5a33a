"""Sequence geometry of the paged KV cache (mirror of ``infer/engine/sequence.py:8-84``).

Only what the cache path needs: token ids, the block table, how many tokens are already cached,
and the block arithmetic (``block_size`` tokens per block, 256 in the reference)."""
from __future__ import annotations

from copy import copy
from enum import Enum, auto
from itertools import count

from .sampling_params import SamplingParams


class SequenceStatus(Enum):
    RUNNING = auto()
    FINISHED = auto()
    WAITING = auto()
    WATING = WAITING     # the reference's spelling (``sequence.py:13``), kept as an alias


class Sequence:
    block_size = 256
    counter = count()

    def __init__(self, token_ids: list[int], sampling_param: SamplingParams | None = None):
        if sampling_param is None:
            sampling_param = SamplingParams()
        self.seq_id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = copy(token_ids)
        self.last_token = token_ids[-1]
        self.num_tokens = len(token_ids)
        self.num_prompt_tokens = len(token_ids)
        self.num_cached_tokens = 0
        self.block_table: list[int] = []
        self.temperature = sampling_param.temperature
        self.max_tokens = sampling_param.max_tokens
        self.ignore_eos = sampling_param.ignore_eos

    def __len__(self):
        return self.num_tokens

    def __getitem__(self, key):
        return self.token_ids[key]

    @property
    def is_finished(self):
        return self.status == SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self):
        return self.num_tokens - self.num_prompt_tokens

    @property
    def num_cached_blocks(self):
        return self.num_cached_tokens // self.block_size

    @property
    def num_blocks(self):
        return (self.num_tokens + self.block_size - 1) // self.block_size

    @property
    def last_block_num_tokens(self):
        return self.num_tokens - (self.num_blocks - 1) * self.block_size

    def block(self, i):
        assert 0 <= i < self.num_blocks
        return self.token_ids[i * self.block_size:(i + 1) * self.block_size]

    def append_token(self, token_id: int):
        self.token_ids.append(token_id)
        self.last_token = token_id
        self.num_tokens += 1

    @property
    def prompt_token_ids(self):
        return self.token_ids[:self.num_prompt_tokens]

    @property
    def completion_token_ids(self):
        return self.token_ids[self.num_prompt_tokens:]

    # Compact wire form of ``sequence.py:75-84``: once decoding has started only the last token travels.
    def __getstate__(self):
        return (self.num_tokens, self.num_prompt_tokens, self.num_cached_tokens, self.block_table,
                self.token_ids if self.num_completion_tokens == 0 else self.last_token)

    def __setstate__(self, state):
        self.num_tokens, self.num_prompt_tokens, self.num_cached_tokens, self.block_table = state[:-1]
        if self.num_completion_tokens == 0:
            self.token_ids = state[-1]
        else:
            self.last_token = state[-1]
