"""Which sequences run in the next step.

Policy and interface of the reference's ``infer/engine/scheduler.py:6-69``, on the native block pool:
a step is a prefill of as many waiting sequences as fit, in arrival order (a budget of batched tokens,
a cap on sequences, free cache blocks), and only when nothing could be admitted a decode of the running
sequences; a running sequence that needs a cache block when none is free evicts the youngest running
sequence, whose blocks are released and which goes back to the head of the waiting queue."""
from __future__ import annotations

from collections import deque

from .block_manager import BlockManager
from .config import Config
from .sequence import Sequence, SequenceStatus


class Scheduler:

    def __init__(self, config: Config):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        self.block_manager = BlockManager(config.num_kvcache_blocks, config.kvcache_block_size)
        self.waiting: deque[Sequence] = deque()       # arrival order; preempted sequences re-enter at the head
        self.running: deque[Sequence] = deque()       # oldest first

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def is_finished(self) -> bool:
        return len(self.waiting) == 0 and len(self.running) == 0

    def schedule(self) -> tuple[list[Sequence], bool]:
        """Returns (sequences of the step, True for a prefill step)."""
        batch = self._admit_waiting()
        if batch:
            return batch, True
        batch = self._continue_running()
        assert batch, "nothing to schedule: no waiting sequence fits and none is running"
        return batch, False

    def _admit_waiting(self) -> list[Sequence]:
        pool = self.block_manager
        admitted: list[Sequence] = []
        new_tokens = 0
        while self.waiting and len(admitted) < self.max_num_seqs:
            head = self.waiting[0]
            # the budget is tested against the whole length (scheduler.py:31) although a prefix-cache hit
            # then charges only the uncached part
            if new_tokens + len(head) > self.max_num_batched_tokens or not pool.can_allocate(head):
                break
            pool.allocate(head)
            new_tokens += len(head) - head.num_cached_tokens
            head.status = SequenceStatus.RUNNING
            self.running.append(self.waiting.popleft())
            admitted.append(head)
        return admitted

    def _continue_running(self) -> list[Sequence]:
        pool = self.block_manager
        kept: list[Sequence] = []
        while self.running and len(kept) < self.max_num_seqs:
            seq = self.running.popleft()
            has_room = pool.can_append(seq)
            while not has_room and self.running:
                self.preempt(self.running.pop())          # youngest first
                has_room = pool.can_append(seq)
            if not has_room:                              # nobody left to evict but the sequence itself
                self.preempt(seq)
                continue
            pool.may_append(seq)
            kept.append(seq)
        for seq in reversed(kept):                        # back to the head of the queue, order unchanged
            self.running.appendleft(seq)
        return kept

    def preempt(self, seq: Sequence) -> None:
        seq.status = SequenceStatus.WAITING
        self.block_manager.deallocate(seq)
        self.waiting.appendleft(seq)

    def postprocess(self, seqs: list[Sequence], token_ids: list[int]) -> None:
        """Appends the sampled tokens; a sequence that produced EOS (unless told to ignore it) or used up its
        token budget is finished and gives its blocks back."""
        finished = set()
        for seq, token in zip(seqs, token_ids):
            seq.append_token(token)
            hit_eos = token == self.eos and not seq.ignore_eos
            if hit_eos or seq.num_completion_tokens == seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                finished.add(id(seq))
        if finished:
            self.running = deque(s for s in self.running if id(s) not in finished)
