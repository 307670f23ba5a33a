"""The named configurations are reproducible from their seeds: the CPU generators give the bits whose
SHA-256 is committed in tests/golden/workload_checksums.json, and the GPU suite moves those same
tensors to the device (tests/test_decode_gpu.py, test_append_gpu.py assert the checksums again at
full size, including the 2 GiB pool of the long-context configuration)."""
import json
import os

import pytest
import torch

from infer_amd import workloads
from tests.helpers import assert_seeded_inputs

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "workload_checksums.json")


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg3"])
def test_generators_reproduce_the_committed_checksums(name):
    assert_seeded_inputs(getattr(workloads, name)(), name)


def test_every_named_configuration_has_checksums_for_every_tensor():
    gold = json.load(open(GOLDEN))
    assert sorted(gold) == ["cfg1", "cfg2", "cfg3", "cfg4"]
    for name in ("cfg1", "cfg3"):
        wl = getattr(workloads, name)()
        tensors = sorted(k for k, v in wl.__dict__.items() if isinstance(v, torch.Tensor))
        assert sorted(gold[name]["sha256"]) == tensors
    assert len(gold["cfg4"]["lengths"]) == 8 and set(gold["cfg4"]["lengths"]) == {32768}


def test_checksum_sees_a_single_flipped_bit():
    wl = workloads.cfg1()
    before = workloads.checksums(wl)
    wl.k_cache.view(torch.int16)[3, 5, 1, 7] ^= 1
    after = workloads.checksums(wl)
    assert after["k_cache"] != before["k_cache"] and after["v_cache"] == before["v_cache"]


def test_device_fill_is_refused_for_nothing_on_cpu():
    """``device_fill`` only changes where the pools are drawn when a device is given; on the CPU it is
    the seeded draw."""
    a = workloads.make_decode_workload("a", [40, 300], 16, 8, seed=3, device_fill=True)
    b = workloads.make_decode_workload("b", [40, 300], 16, 8, seed=3)
    assert workloads.checksums(a) == workloads.checksums(b)
