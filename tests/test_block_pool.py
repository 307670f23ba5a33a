"""The native block pool (infer::BlockPool behind infer_pool_*) against: XXH64 known answers, the
third-party xxhash package, the golden trace recorded from the reference's own BlockManager
(tests/golden/block_manager_trace.json), the independent Python model in oracle/, and invariants."""
import json
import os
import random

import numpy as np
import pytest
import xxhash

from infer_amd import _lib
from infer_amd.block_manager import BlockManager
from infer_amd.sequence import Sequence
from oracle.block_manager_ref import BlockManagerModel, block_hash

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(autouse=True)
def small_blocks():
    old = Sequence.block_size
    yield
    Sequence.block_size = old


# ----------------------------------------------------------------------------- hashing

def test_xxh64_known_answers():
    lib = _lib.load()
    # published XXH64 values (xxHash project sanity values; also what `xxhsum -H1` prints)
    assert lib.infer_xxh64(b"", 0, 0) == 0xEF46DB3751D8E999
    assert lib.infer_xxh64(b"a", 1, 0) == 0xD24EC4F1A98C6E5B
    assert lib.infer_xxh64(b"abc", 3, 0) == 0x44BC2CF5AD770999


def test_xxh64_matches_the_xxhash_package_for_every_tail_length_and_seeds():
    lib = _lib.load()
    rng = np.random.default_rng(0)
    for n in list(range(0, 100)) + [255, 256, 257, 2048, 4099]:
        data = rng.integers(0, 256, n, dtype=np.uint8).tobytes()
        for seed in (0, 1, 0x9E3779B185EBCA87):
            assert lib.infer_xxh64(data, n, seed) == xxhash.xxh64(data, seed=seed).intdigest(), (n, seed)


def test_block_hash_chain_matches_the_reference_formula():
    rng = random.Random(1)
    prev = -1
    for _ in range(5):
        toks = [rng.randrange(151936) for _ in range(256)]
        want = xxhash.xxh64((b"" if prev == -1 else prev.to_bytes(8, "little")) + np.array(toks).tobytes()).intdigest()
        assert BlockManager.compute_hash(toks, prev) == want == block_hash(toks, prev)
        prev = want


# ----------------------------------------------------------------------------- golden trace

def _replay(make, trace):
    """Plays the recorded scenario against an implementation; yields (op, observed state)."""
    bs = trace["block_size"]
    Sequence.block_size = bs
    impl = make(trace["num_blocks"], bs)
    seqs = {}
    for op in trace["ops"]:
        if op["op"] == "allocate":
            s = Sequence(op["tokens"])
            ok = impl.can_allocate(s)
            assert ok == op["can_allocate"], op
            if ok:
                impl.allocate(s)
                seqs[op["name"]] = s
        elif op["op"] == "deallocate":
            impl.deallocate(seqs.pop(op["name"]))
        else:
            s = seqs[op["name"]]
            s.append_token(op["token"])
            ok = impl.can_append(s)
            assert ok == op["can_append"], op
            if ok:
                impl.may_append(s)
            else:
                s.token_ids.pop()
                s.num_tokens -= 1
        yield op, impl, seqs


class ModelAdapter:
    """Gives oracle.BlockManagerModel the Sequence-based interface."""
    def __init__(self, n, bs):
        self.m = BlockManagerModel(n, bs)

    def can_allocate(self, s): return self.m.can_allocate(len(s))
    def can_append(self, s): return self.m.can_append(len(s))
    def may_append(self, s): self.m.may_append(s.token_ids, s.block_table)

    def allocate(self, s):
        table, cached = self.m.allocate(s.token_ids)
        s.block_table.extend(table)
        s.num_cached_tokens += cached

    def deallocate(self, s):
        self.m.deallocate(s.block_table)
        s.block_table.clear()
        s.num_cached_tokens = 0

    @property
    def free_block_ids(self): return list(self.m.free)
    def ref_count(self, i): return self.m.refs[i]
    def block_hash(self, i): return self.m.hash[i]


@pytest.mark.parametrize("make", [BlockManager, ModelAdapter], ids=["native", "oracle-model"])
def test_golden_trace_of_the_reference_block_manager(make):
    trace = json.load(open(os.path.join(HERE, "golden", "block_manager_trace.json")))
    n = trace["num_blocks"]
    steps = 0
    for op, impl, seqs in _replay(make, trace):
        assert impl.free_block_ids == op["free"], op
        assert [impl.ref_count(i) for i in range(n)] == op["refs"], op
        assert [impl.block_hash(i) for i in range(n)] == op["hashes"], op
        # (the recorder snapshots a deallocated sequence once more, with an empty table)
        gone = {k for k in op["tables"] if k not in seqs}
        assert all(op["tables"][k] == [] and op["cached"][k] == 0 for k in gone), op
        assert {k: s.block_table for k, s in seqs.items()} == {k: v for k, v in op["tables"].items() if k not in gone}, op
        assert {k: s.num_cached_tokens for k, s in seqs.items()} == {k: v for k, v in op["cached"].items() if k not in gone}, op
        steps += 1
    assert steps == len(trace["ops"]) >= 30


# ----------------------------------------------------------------------------- random workloads

def _check_invariants(bm, n, seqs):
    free = bm.free_block_ids
    assert len(free) == len(set(free)) == bm.num_free_blocks
    used = set(range(n)) - set(free)
    refs = [bm.ref_count(i) for i in range(n)]
    for i in range(n):
        assert (refs[i] >= 1) == (i in used)
    counted = [0] * n
    for s in seqs:
        assert len(s.block_table) == s.num_blocks
        assert s.num_cached_tokens % Sequence.block_size == 0 and s.num_cached_tokens <= len(s)
        for b in s.block_table:
            counted[b] += 1
    assert counted == refs


@pytest.mark.parametrize("seed", range(6))
def test_random_workload_native_equals_model_and_keeps_invariants(seed):
    rng = random.Random(seed)
    bs, n = 4, 24
    Sequence.block_size = bs
    native, model = BlockManager(n, bs), ModelAdapter(n, bs)
    live = []   # pairs (native seq, model seq)
    vocab = 3   # tiny vocabulary so that prefixes collide all the time
    for step in range(400):
        r = rng.random()
        if r < 0.35 or not live:
            toks = [rng.randrange(vocab) for _ in range(rng.randrange(1, 4 * bs + 2))]
            a, b = Sequence(toks), Sequence(toks)
            assert native.can_allocate(a) == model.can_allocate(b)
            if native.can_allocate(a):
                native.allocate(a); model.allocate(b)
                live.append((a, b))
        elif r < 0.55:
            a, b = live.pop(rng.randrange(len(live)))
            native.deallocate(a); model.deallocate(b)
        else:
            a, b = rng.choice(live)
            t = rng.randrange(vocab)
            a.append_token(t); b.append_token(t)
            assert native.can_append(a) == model.can_append(b)
            if native.can_append(a):
                native.may_append(a); model.may_append(b)
            else:
                for s in (a, b):
                    s.token_ids.pop(); s.num_tokens -= 1
        for a, b in live:
            assert a.block_table == b.block_table and a.num_cached_tokens == b.num_cached_tokens
        assert native.free_block_ids == model.free_block_ids
        if step % 20 == 0:
            _check_invariants(native, n, [a for a, _ in live])


def test_sharing_happens_exactly_on_the_common_full_block_prefix():
    """Brute-force statement of the prefix cache: two live sequences share block i iff their first
    (i + 1) * bs tokens are equal (and block i is full in both)."""
    rng = random.Random(3)
    bs, n = 4, 64
    Sequence.block_size = bs
    bm = BlockManager(n, bs)
    seqs = []
    for _ in range(12):
        toks = [rng.randrange(2) for _ in range(rng.randrange(1, 18))]
        s = Sequence(toks)
        if bm.can_allocate(s):
            bm.allocate(s)
            seqs.append(s)
    for x in seqs:
        for y in seqs:
            if x is y:
                continue
            for i in range(min(x.num_blocks, y.num_blocks)):
                full = (i + 1) * bs <= min(len(x), len(y))
                same_prefix = full and x.token_ids[:(i + 1) * bs] == y.token_ids[:(i + 1) * bs]
                assert (x.block_table[i] == y.block_table[i]) == same_prefix
    for s in seqs:   # cached tokens = the longest prefix of full blocks an EARLIER sequence already held
        assert s.num_cached_tokens % bs == 0


def test_exhaustion_and_preemption_path():
    """Two sequences stepping over a block boundary in a pool with no spare block: the second cannot
    append until the first is deallocated (the scheduler's preemption path,
    infer/engine/scheduler.py:44-49,58-61), and the freed blocks are reused in FIFO order."""
    bs = 4
    Sequence.block_size = bs
    bm = BlockManager(3, bs)
    a, b = Sequence([1, 2, 3, 4]), Sequence([5, 6, 7, 8])
    bm.allocate(a); bm.allocate(b)
    a.append_token(9)
    assert bm.can_append(a)
    bm.may_append(a)
    assert a.block_table == [0, 2] and bm.num_free_blocks == 0
    b.append_token(9)
    assert not bm.can_append(b)
    bm.deallocate(a)                    # preempt a
    assert bm.free_block_ids == [2, 0] and a.block_table == [] and a.num_cached_tokens == 0
    assert bm.can_append(b)
    bm.may_append(b)
    assert b.block_table == [1, 2]
    big = Sequence(list(range(100, 109)))
    assert not bm.can_allocate(big)


def test_misuse_raises_like_the_reference_asserts():
    bs = 4
    Sequence.block_size = bs
    bm = BlockManager(4, bs)
    s = Sequence([1, 2, 3, 4, 5])
    bm.allocate(s)
    with pytest.raises(AssertionError):
        bm.allocate(s)                              # assert not seq.block_table
    s.append_token(6)                               # len 6: inside a block, nothing to do
    bm.may_append(s)
    t = Sequence([1, 2, 3, 4])
    bm.allocate(t)                                  # full block is sealed at allocation
    t.append_token(9); t.append_token(9); t.append_token(9); t.append_token(9)   # len 8 without opening a block
    with pytest.raises(AssertionError):
        bm.may_append(t)                            # assert last_block.hash == -1
    with pytest.raises(AssertionError):
        BlockManager(0, 4)
