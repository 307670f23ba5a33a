"""``BlockManager`` with the interface of ``infer/engine/block_mannager.py:44-133`` on top of the
native block pool (``infer::BlockPool`` through the C ABI ``infer_pool_*``).

Same method names, same arguments (a ``Sequence``), same side effects on the sequence
(``block_table``, ``num_cached_tokens``), and ``AssertionError`` where the reference asserts."""
from __future__ import annotations

import ctypes

import numpy as np

from . import _lib
from .sequence import Sequence


class BlockManager:

    def __init__(self, num_blocks: int, block_size: int):
        assert num_blocks > 0
        self.block_size = block_size
        self.num_blocks = num_blocks
        self._lib = _lib.load()
        self._pool = self._lib.infer_pool_create(num_blocks, block_size)
        if not self._pool:
            raise RuntimeError(self._lib.infer_pool_last_error().decode())

    def __del__(self):
        pool, self._pool = getattr(self, "_pool", None), None
        if pool:
            self._lib.infer_pool_destroy(pool)

    # ---- helpers
    def _state(self, code):
        if code == -5:
            raise AssertionError(self._lib.infer_pool_last_error().decode())
        if code < 0:
            _lib.check(int(code), "block pool")
        return code

    @staticmethod
    def _ids(token_ids):
        return np.ascontiguousarray(np.asarray(token_ids, dtype=np.int64))

    @classmethod
    def compute_hash(cls, token_ids: list[int], prefix: int = -1) -> int:
        ids = cls._ids(token_ids)
        return int(_lib.load().infer_pool_hash(ids.ctypes.data, ids.size, int(prefix != -1),
                                               ctypes.c_uint64(prefix if prefix != -1 else 0)))

    # ---- state
    @property
    def num_free_blocks(self) -> int:
        return self._lib.infer_pool_num_free(self._pool)

    @property
    def free_block_ids(self) -> list[int]:
        out = np.empty(self.num_blocks, dtype=np.int32)
        n = self._lib.infer_pool_free_ids(self._pool, out.ctypes.data, out.size)
        return out[:n].tolist()

    @property
    def used_block_ids(self) -> set[int]:
        return set(range(self.num_blocks)) - set(self.free_block_ids)

    def ref_count(self, block_id: int) -> int:
        return self._lib.infer_pool_ref_count(self._pool, block_id)

    def block_hash(self, block_id: int) -> int:
        h = ctypes.c_uint64(0)
        has = self._lib.infer_pool_block_hash(self._pool, block_id, ctypes.byref(h))
        return int(h.value) if has == 1 else -1

    # ---- the reference's interface
    def can_allocate(self, seq: Sequence) -> bool:
        return bool(self._lib.infer_pool_can_allocate(self._pool, len(seq)))

    def allocate(self, seq: Sequence):
        assert not seq.block_table
        ids = self._ids(seq.token_ids)
        table = np.empty(seq.num_blocks, dtype=np.int32)
        cached = self._state(self._lib.infer_pool_allocate(self._pool, ids.ctypes.data, ids.size,
                                                           table.ctypes.data, table.size))
        seq.num_cached_tokens += int(cached)
        seq.block_table.extend(table.tolist())

    def deallocate(self, seq: Sequence):
        table = np.asarray(seq.block_table, dtype=np.int32)
        self._state(self._lib.infer_pool_deallocate(self._pool, table.ctypes.data, table.size))
        seq.num_cached_tokens = 0
        seq.block_table.clear()

    def can_append(self, seq: Sequence) -> bool:
        # ``block_manager.py:120-121``: a free block is needed only by the first token of a new block
        if len(seq) % self.block_size != 1:
            return True
        return bool(self._lib.infer_pool_can_append(self._pool, len(seq)))

    def may_append(self, seq: Sequence):
        r = len(seq) % self.block_size
        if r > 1 and seq.block_table:
            return           # mid-block token: the reference only asserts here (``:132-133``)
        # only the block that was just filled has to cross the boundary, not the whole sequence
        ids = self._ids(seq.token_ids[-self.block_size:]) if r == 0 else None
        n = len(seq.block_table)
        table = np.empty(n + 1, dtype=np.int32)
        table[:n] = seq.block_table
        new_n = self._state(self._lib.infer_pool_may_append_block(
            self._pool, ids.ctypes.data if ids is not None else None, len(seq), table.ctypes.data, n, table.size))
        if new_n > n:
            seq.block_table.append(int(table[n]))
