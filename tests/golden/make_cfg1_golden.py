"""Writes ``cfg1_golden.json``: the reference's CPU-runnable configuration (single-layer
Qwen3-0.6B-shaped decode step, batch 4, lengths {37, 256, 700, 1023}, 64-block pool, seed 0) as a
small fixture: hashes of the seeded inputs, the hash of both caches after the append (bit-exact
data), and the float32 attention output of the CPU oracle (first and last columns of every row plus
row sums).

The numbers come from this repository's own oracle (``oracle/paged_ref.py``), which is pinned
independently in ``tests/test_oracle.py``; the reference's arithmetic for this step lives in the
``flash_attn`` package, which is not available, so nothing of the reference is run here.  The fixture
freezes the configuration across changes of the generator, the oracle and the kernels.

    python tests/golden/make_cfg1_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from infer_amd import workloads  # noqa: E402
from oracle import paged_ref  # noqa: E402
from tests.helpers import bits  # noqa: E402


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def build():
    wl = workloads.cfg1()
    kc, vc = bits(wl.k_cache).copy(), bits(wl.v_cache).copy()
    slots = wl.slot_mapping.numpy()
    paged_ref.append_ref(bits(wl.k_new), bits(wl.v_new), kc, vc, slots)
    out = paged_ref.paged_decode_ref(bits(wl.q), kc, vc, wl.block_table.numpy(), wl.context_lens.numpy(), wl.scale)
    return {
        "config": {"num_q_heads": wl.num_q_heads, "num_kv_heads": wl.num_kv_heads, "head_dim": wl.head_dim,
                   "block_size": wl.block_size, "lengths": list(wl.lengths), "pool_blocks": int(wl.k_cache.shape[0]),
                   "seed": 0},
        "inputs_sha256": {"q": sha(bits(wl.q)), "k_new": sha(bits(wl.k_new)), "v_new": sha(bits(wl.v_new)),
                          "k_cache": sha(bits(wl.k_cache)), "v_cache": sha(bits(wl.v_cache)),
                          "slot_mapping": sha(slots), "block_table": sha(wl.block_table.numpy()),
                          "context_lens": sha(wl.context_lens.numpy())},
        "slot_mapping": slots.tolist(),
        "block_table": wl.block_table.numpy().tolist(),
        "after_append_sha256": {"k_cache": sha(kc), "v_cache": sha(vc)},
        "attention_out": {
            "shape": list(out.shape),
            "first8": np.round(out[:, :, :8].astype(np.float64), 6).tolist(),
            "last8": np.round(out[:, :, -8:].astype(np.float64), 6).tolist(),
            "row_sums": np.round(out.astype(np.float64).sum(axis=-1), 5).tolist(),
        },
    }


if __name__ == "__main__":
    with open(os.path.join(HERE, "cfg1_golden.json"), "w") as f:
        json.dump(build(), f, indent=1)
    print("wrote", os.path.join(HERE, "cfg1_golden.json"))
