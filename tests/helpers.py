"""Shared glue between torch tensors (GPU or CPU) and the numpy oracle."""
import numpy as np
import torch

from oracle import paged_ref


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 numpy array of its bit patterns (on the host)."""
    assert t.dtype == torch.bfloat16
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float32).numpy()


def oracle_decode(wl, k_cache=None, v_cache=None) -> np.ndarray:
    return paged_ref.paged_decode_ref(
        bits(wl.q), bits(wl.k_cache if k_cache is None else k_cache),
        bits(wl.v_cache if v_cache is None else v_cache),
        wl.block_table.cpu().numpy(), wl.context_lens.cpu().numpy(), wl.scale)


# bf16 attention output against the fp32 CPU oracle: the tolerance the reference uses for its
# own attention test (test/op.py:283, atol=2e-2) and the bar set for this path.
ATTN_ATOL = 2e-2


def assert_seeded_inputs(wl, name):
    """The tensors of a named configuration are the ones its seed draws on the CPU: their SHA-256
    equals tests/golden/workload_checksums.json (written by tests/golden/make_workload_checksums.py)."""
    import json
    import os
    from infer_amd import workloads
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "workload_checksums.json")
    want = json.load(open(path))[name]
    assert list(wl.lengths) == want["lengths"]
    got = workloads.checksums(wl)
    assert got == want["sha256"], f"{name}: inputs differ from the committed seeds' checksums"
