"""Records a golden trace of the reference's own block pool (run in the build container only).

Imports ``infer.engine.block_mannager.BlockManager`` and ``infer.engine.sequence.Sequence`` from
the reference tree (pure Python; needs only numpy and xxhash), plays a scripted scenario that
exercises the allocation order in the mixed hit/miss cases (a hit on a block that sits in the
free list, a miss after hits, sealing during decode, FIFO reuse after deallocation) and writes
every observable after every operation to ``block_manager_trace.json`` next to this file.

    python tests/golden/make_block_manager_trace.py /root/reference
"""
import json
import os
import random
import sys


def main(ref_root):
    sys.path.insert(0, ref_root)
    from infer.engine.block_mannager import BlockManager      # noqa: E402
    from infer.engine.sequence import Sequence                # noqa: E402
    from infer.sampling_params import SamplingParams          # noqa: E402

    bs = 4
    Sequence.block_size = bs
    bm = BlockManager(12, bs)
    sp = SamplingParams()
    rng = random.Random(7)
    ops = []
    seqs = {}

    def snap(op):
        op["free"] = list(bm.free_block_ids)
        op["refs"] = [b.ref_count for b in bm.blocks]
        op["hashes"] = [b.hash for b in bm.blocks]
        op["tables"] = {k: list(s.block_table) for k, s in seqs.items()}
        op["cached"] = {k: s.num_cached_tokens for k, s in seqs.items()}
        ops.append(op)

    def alloc(name, tokens):
        s = Sequence(tokens, sp)
        ok = bm.can_allocate(s)
        op = {"op": "allocate", "name": name, "tokens": tokens, "can_allocate": ok}
        if ok:
            bm.allocate(s)
            seqs[name] = s
        snap(op)

    def free(name):
        bm.deallocate(seqs[name])
        snap({"op": "deallocate", "name": name})
        del seqs[name]

    def append(name, token):
        s = seqs[name]
        s.append_token(token)
        ok = bm.can_append(s)
        op = {"op": "append", "name": name, "token": token, "can_append": ok}
        if ok:
            bm.may_append(s)
        else:
            s.token_ids.pop()
            s.num_tokens -= 1
        snap(op)

    base = [rng.randrange(1000) for _ in range(14)]
    alloc("a", base[:10])                     # 2 full blocks + partial
    alloc("b", base[:8] + [5, 6])             # shares 2 blocks with a
    alloc("c", base[:4] + [1, 2, 3, 4, 9])    # shares 1 block, then misses
    free("a")
    free("b")                                 # blocks of the shared prefix return to the free list, still hashed
    alloc("d", base[:9])                      # hits on blocks that sit in the free list
    for t in (11, 12, 13, 14, 15, 16, 17):    # decode across two block boundaries (seal + open)
        append("d", t)
    alloc("e", base[:8] + [11, 12, 13, 14])   # a full third block that d sealed during decode? (d has base[8] first)
    free("c")
    alloc("f", [7] * 8)                       # identical blocks inside one sequence
    alloc("g", [7] * 9)
    free("d")
    free("e")
    alloc("h", base[:10])                     # revives base blocks again after more churn
    alloc("i", list(range(100, 100 + 13)))    # takes free blocks in FIFO order
    alloc("j", list(range(200, 200 + 40)))    # does not fit
    for t in range(6):
        append("i", 300 + t)
    free("f"); free("g"); free("h"); free("i")
    alloc("k", [7] * 8)                       # after everything was freed: still a hit

    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "block_manager_trace.json")
    with open(out, "w") as f:
        json.dump({"block_size": bs, "num_blocks": 12, "ops": ops}, f, indent=0)
    print("wrote", out, len(ops), "ops")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
