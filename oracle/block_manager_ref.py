"""CPU model of the reference block pool.  TEST INFRASTRUCTURE ONLY (see oracle/paged_ref.py).

Restates ``BlockManager`` of ``infer/engine/block_mannager.py:44-133`` in plain Python on plain
data (lists of token ids and block tables instead of ``Sequence`` objects), written independently
of the C++ pool so that the two can be compared on random workloads:

* ``allocate``   - ``block_mannager.py:79-103``
* ``deallocate`` - ``:105-112``
* ``can_append`` / ``may_append`` - ``:114-133``
* ``block_hash`` - ``compute_hash`` ``:54-60``: xxh64 (seed 0) of the previous block's hash as 8
  little-endian bytes (when there is one) followed by the token ids as little-endian int64.  The
  hash function comes from the third-party ``xxhash`` package (a dependency of the reference,
  un-vendored and unpinned there), not from the reference itself.

Pinned by: the invariants in ``tests/test_block_pool.py`` (free and used partition the pool, a
block is used iff referenced, FIFO reuse, hits only on a common full-block prefix), a brute-force
prefix-tuple model of which blocks may be shared, and the golden trace
``tests/golden/block_manager_trace.json`` recorded from the reference's own class.
"""
from __future__ import annotations

from collections import deque

import numpy as np
import xxhash


def block_hash(token_ids, prefix=-1) -> int:
    h = xxhash.xxh64()
    if prefix != -1:
        h.update(int(prefix).to_bytes(8, "little"))
    h.update(np.asarray(token_ids, dtype=np.int64).tobytes())
    return h.intdigest()


class BlockManagerModel:
    def __init__(self, num_blocks: int, block_size: int):
        self.bs = block_size
        self.refs = [0] * num_blocks
        self.hash = [-1] * num_blocks
        self.tokens = [[] for _ in range(num_blocks)]
        self.by_hash: dict[int, int] = {}
        self.free = deque(range(num_blocks))

    def _take(self, bid):
        assert self.refs[bid] == 0
        self.refs[bid], self.hash[bid], self.tokens[bid] = 1, -1, []
        self.free.remove(bid)

    def num_blocks_for(self, n):
        return -(-n // self.bs)

    def can_allocate(self, n_tokens) -> bool:
        return len(self.free) >= self.num_blocks_for(n_tokens)

    def allocate(self, token_ids) -> tuple[list[int], int]:
        """Returns (block_table, num_cached_tokens)."""
        table, cached, h, missed = [], 0, -1, False
        for i in range(self.num_blocks_for(len(token_ids))):
            chunk = list(token_ids[i * self.bs:(i + 1) * self.bs])
            h = block_hash(chunk, h) if len(chunk) == self.bs else -1
            bid = self.by_hash.get(h, -1)
            if bid == -1 or self.tokens[bid] != chunk:
                missed = True
            if missed:
                bid = self.free[0]
                self._take(bid)
            else:
                cached += self.bs
                if self.refs[bid] > 0:
                    self.refs[bid] += 1
                else:
                    self._take(bid)
            if h != -1:
                self.hash[bid], self.tokens[bid] = h, chunk
                self.by_hash[h] = bid
            table.append(bid)
        return table, cached

    def deallocate(self, table) -> None:
        for bid in reversed(table):
            self.refs[bid] -= 1
            if self.refs[bid] == 0:
                self.free.append(bid)

    def can_append(self, seq_len) -> bool:
        return len(self.free) >= (1 if seq_len % self.bs == 1 else 0)

    def may_append(self, token_ids, table) -> None:
        n = len(token_ids)
        last = table[-1]
        if n % self.bs == 1:
            assert self.hash[last] != -1
            bid = self.free[0]
            self._take(bid)
            table.append(bid)
        elif n % self.bs == 0:
            assert self.hash[last] == -1
            chunk = list(token_ids[-self.bs:])
            prefix = self.hash[table[-2]] if len(table) > 1 else -1
            h = block_hash(chunk, prefix)
            self.hash[last], self.tokens[last] = h, chunk
            self.by_hash[h] = last
        else:
            assert self.hash[last] == -1
