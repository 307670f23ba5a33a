"""Qwen3 decoder with the module tree of ``infer/models/Qwen3.py:59-321`` (same attribute names, so a
checkpoint's tensor names map the same way), built on the paged KV-cache path of this package.

Per layer the step before attention - q_norm, k_norm, the rotary embedding and the KV append, four
launches in the reference (``Qwen3.py:113-131``) - is one fused kernel; attention is the paged decode
kernel or the varlen prefill kernel depending on ``context.is_prefill``."""
from __future__ import annotations

import torch
from torch import nn

from . import ops
from .attention import Attention
from .context import get_context
from .layers import MLP, Embedding, Linear, LMHead, QKVLinear, RMSNorm, cos_sin_table


class QwenAttention(nn.Module):

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, max_position: int = 4096 * 10,
                 head_dim: int = 128, rms_norm_eps: float = 1e-6, rope_theta: float = 100000, layer_idx: int = 0):
        super().__init__()
        self.layer_idx = layer_idx
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.num_kv_heads = num_kv_heads
        self.q_size = num_heads * head_dim
        self.kv_size = num_kv_heads * head_dim
        self.scale = head_dim ** -0.5
        self.max_position = max_position
        self.rope_theta = rope_theta
        self.qkv_proj = QKVLinear(hidden_size, self.q_size, self.kv_size)
        self.o_proj = Linear(self.q_size, hidden_size, False)
        self.attn = Attention(num_heads, head_dim, self.scale, num_kv_heads)
        self.q_norm = RMSNorm(head_dim, rms_norm_eps)
        self.k_norm = RMSNorm(head_dim, rms_norm_eps)
        self._no_cache = None

    def _caches(self, device):
        k_cache, v_cache = self.attn.k_cache, self.attn.v_cache
        if k_cache.numel() and v_cache.numel():
            return k_cache, v_cache, True
        # Before the pool exists (the warm-up pass, ``model_runner.py:37-45``) nothing is stored:
        # the fused kernel gets a one-block stand-in and slots of -1, which it skips.
        if self._no_cache is None or self._no_cache.device != device:
            self._no_cache = torch.zeros(1, 256, self.num_kv_heads, self.head_dim, dtype=torch.bfloat16, device=device)
        return self._no_cache, self._no_cache, False

    def forward(self, positions: torch.Tensor, hidden_states: torch.Tensor) -> torch.Tensor:
        qkv = self.qkv_proj(hidden_states)
        q, k, v = qkv.split([self.q_size, self.kv_size, self.kv_size], dim=-1)
        q = q.view(-1, self.num_heads, self.head_dim)
        k = k.view(-1, self.num_kv_heads, self.head_dim)
        v = v.view(-1, self.num_kv_heads, self.head_dim)
        context = get_context()
        k_cache, v_cache, bound = self._caches(q.device)
        slots = context.slot_mapping
        if bound:
            # with a cache bound every token must come with its slot, as the reference's store_kvcache
            # asserts (infer/ops/attention.py:44): a metadata bug must not silently skip the append
            assert slots is not None and slots.numel() == q.shape[0], "slot_mapping must hold one slot per token"
        else:
            slots = torch.full((q.shape[0],), -1, dtype=torch.int32, device=q.device)
        # keys are read back from the packed rows only by a prefill without a cached prefix
        keys_from_rows = context.is_prefill and context.block_tables is None
        table = cos_sin_table(self.head_dim, self.max_position, self.rope_theta, q.device)
        ops.qk_norm_rope_store_kvcache(q, k, v, positions, self.q_norm.weight, self.k_norm.weight,
                                       self.q_norm.eps, table, k_cache, v_cache, slots, write_key=keys_from_rows)
        o = self.attn(q, k, v, kv_stored=True)
        return self.o_proj(o, defer=True)           # consumed by post_attention_layernorm


class QwenDecoderLayer(nn.Module):

    def __init__(self, config, layer_idx: int):
        super().__init__()
        self.layer_idx = layer_idx
        self.self_attn = QwenAttention(
            hidden_size=config.hidden_size,
            num_heads=config.num_attention_heads,
            num_kv_heads=config.num_key_value_heads,
            max_position=config.max_position_embeddings,
            rms_norm_eps=config.rms_norm_eps,
            head_dim=getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads,
            rope_theta=getattr(config, "rope_theta", 100000),
            layer_idx=layer_idx,
        )
        self.mlp = MLP(hidden_size=config.hidden_size, intermediate_size=config.intermediate_size)
        self.input_layernorm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)
        self.post_attention_layernorm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)

    def forward(self, positions: torch.Tensor, hidden_states: torch.Tensor, residual: torch.Tensor | None):
        if residual is None:
            residual = hidden_states
            hidden_states = self.input_layernorm(hidden_states)
        else:
            hidden_states, residual = self.input_layernorm(hidden_states, residual)
        hidden_states = self.self_attn(positions, hidden_states)
        hidden_states, residual = self.post_attention_layernorm(hidden_states, residual)
        hidden_states = self.mlp(hidden_states)
        return hidden_states, residual


class QwenModel(nn.Module):

    def __init__(self, config):
        super().__init__()
        self.embed_tokens = Embedding(config.vocab_size, config.hidden_size)
        self.layers = nn.ModuleList([QwenDecoderLayer(config, i) for i in range(config.num_hidden_layers)])
        self.norm = RMSNorm(config.hidden_size, eps=config.rms_norm_eps)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        hidden_states = self.embed_tokens(input_ids)
        residual = None
        for layer in self.layers:
            hidden_states, residual = layer(positions, hidden_states, residual)
        hidden_states, _ = self.norm(hidden_states, residual)
        return hidden_states


class QwenForCausalLM(nn.Module):
    packed_modules_mapping = {
        "q_proj": ("qkv_proj", "q"),
        "k_proj": ("qkv_proj", "k"),
        "v_proj": ("qkv_proj", "v"),
        "gate_proj": ("gate_up_proj", 0),
        "up_proj": ("gate_up_proj", 1),
    }

    def __init__(self, config):
        super().__init__()
        self.model = QwenModel(config)
        self.lm_head = LMHead(config.vocab_size, config.hidden_size)
        if config.tie_word_embeddings:
            self.lm_head.weight = self.model.embed_tokens.weight

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        return self.model(input_ids, positions)

    def compute_logits(self, hidden_states: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden_states)


def init_random_weights(model: nn.Module, seed: int = 0, std: float = 0.02) -> None:
    """Projection and embedding weights from N(0, std) with a fixed seed, norm weights left at one:
    the stand-in for a checkpoint where none is available.  Drawn where the parameter lives (an 8B
    model takes seconds on the GPU), one generator for the whole model."""
    gens: dict = {}
    seen = set()
    for name, p in model.named_parameters():
        if id(p) in seen:
            continue
        seen.add(id(p))
        if name.endswith("norm.weight") or "layernorm" in name:
            p.data.fill_(1.0)
            continue
        gen = gens.get(p.device)
        if gen is None:
            gen = gens[p.device] = torch.Generator(device=p.device).manual_seed(seed)
        p.data.normal_(0.0, std, generator=gen)
