"""Writes tests/golden/workload_checksums.json: SHA-256 of every input tensor of the named
configurations (cfg1 .. cfg4), drawn on the CPU from their seeds.

    python tests/golden/make_workload_checksums.py

The CPU suite checks that the generators still reproduce these bits; the GPU suite moves the same
CPU-drawn tensors to the device, so the HIP path and the CPU oracle see the inputs named here.
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from infer_amd import workloads  # noqa: E402

SEEDS = {"cfg1": 0, "cfg2": 0, "cfg3": 0, "cfg4": 0}


def main():
    out = {}
    for name in ("cfg1", "cfg2", "cfg3", "cfg4"):
        wl = getattr(workloads, name)()
        out[name] = {"seed": SEEDS[name], "lengths": wl.lengths, "sha256": workloads.checksums(wl)}
        print(name, "done", flush=True)
    path = os.path.join(ROOT, "tests", "golden", "workload_checksums.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", path)


if __name__ == "__main__":
    main()
