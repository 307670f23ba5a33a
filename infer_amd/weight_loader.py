"""Checkpoint loading (the job of ``infer/utils/weight_loader.py:17-57``): every tensor of every
``*.safetensors`` file in a directory is copied into the parameter of the same name; the separate
q/k/v and gate/up projections of a checkpoint land in their slice of the packed parameters as the
model's ``packed_modules_mapping`` says."""
from __future__ import annotations

import os
from glob import glob

from torch import nn


def has_checkpoint(path: str) -> bool:
    return os.path.isdir(path) and bool(glob(os.path.join(path, "*.safetensors")))


def load_model(model: nn.Module, path: str) -> int:
    from safetensors import safe_open

    packed = getattr(model, "packed_modules_mapping", {})
    owners = {f"{m_name}.{p_name}" if m_name else p_name: module
              for m_name, module in model.named_modules()
              for p_name, _ in module.named_parameters(recurse=False)}
    params = dict(model.named_parameters())
    loaded = 0
    for file in sorted(glob(os.path.join(path, "*.safetensors"))):
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                tensor = f.get_tensor(name)
                for key, (target, shard_id) in packed.items():
                    if key in name:
                        pname = name.replace(key, target)
                        owners[pname].weight_loader(params[pname], tensor, shard_id)
                        break
                else:
                    if name not in params:
                        if name == "lm_head.weight":      # tied to the embedding in this model
                            continue
                        raise KeyError(f"checkpoint tensor {name} has no parameter in the model")
                    params[name].data.copy_(tensor)
                loaded += 1
    return loaded
