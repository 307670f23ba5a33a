"""Engine configuration (mirror of ``infer/config.py:5-27``).

The reference reads the model geometry with ``transformers.AutoConfig`` from a checkpoint
directory.  Here ``hf_config`` may also be handed in directly (a ``ModelConfig`` or any object with
the same attributes), which is how a random-initialised model of a published shape is built where
no checkpoint exists; with a directory, its ``config.json`` is parsed."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass

import torch


@dataclass
class ModelConfig:
    """The attributes of a Qwen3 ``config.json`` that the engine reads."""
    vocab_size: int = 151936
    hidden_size: int = 4096
    intermediate_size: int = 12288
    num_hidden_layers: int = 36
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    max_position_embeddings: int = 40960
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1e6
    tie_word_embeddings: bool = False
    torch_dtype: torch.dtype = torch.bfloat16

    @classmethod
    def from_json(cls, path: str) -> "ModelConfig":
        with open(path) as f:
            raw = json.load(f)
        known = {k: raw[k] for k in cls.__dataclass_fields__ if k in raw and k != "torch_dtype"}
        cfg = cls(**known)
        if "head_dim" not in raw:
            cfg.head_dim = cfg.hidden_size // cfg.num_attention_heads
        dtype = raw.get("torch_dtype", raw.get("dtype", "bfloat16"))
        cfg.torch_dtype = getattr(torch, dtype) if isinstance(dtype, str) else dtype
        return cfg


def qwen3_8b() -> ModelConfig:
    return ModelConfig()


def qwen3_0_6b() -> ModelConfig:
    return ModelConfig(hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                       num_key_value_heads=8, tie_word_embeddings=True)


def qwen3_32b() -> ModelConfig:
    return ModelConfig(hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64,
                       num_key_value_heads=8)


@dataclass
class Config:
    model: str = ""
    max_num_batched_tokens: int = 16384
    max_num_seqs: int = 512
    max_model_len: int = 4096
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1
    enforce_eager: bool = False
    hf_config: ModelConfig | None = None
    eos: int = -1
    kvcache_block_size: int = 256
    num_kvcache_blocks: int = -1
    # Decode tokens are fed position len(seq) by the reference (``model_runner.py:117``) while its
    # prefill positions are zero-based (``:84``); 1 reproduces that, 0 makes both zero-based.
    decode_position_offset: int = 1
    seed: int = 0

    def __post_init__(self):
        if self.hf_config is None:
            assert os.path.isdir(self.model)
            self.hf_config = ModelConfig.from_json(os.path.join(self.model, "config.json"))
        assert self.kvcache_block_size % 256 == 0
        assert 1 <= self.tensor_parallel_size <= 8
        self.max_model_len = min(self.max_model_len, self.hf_config.max_position_embeddings)
        assert self.max_num_batched_tokens >= self.max_model_len
