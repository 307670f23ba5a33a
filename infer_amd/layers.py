"""The layers of the engine's model around the paged KV-cache path, with the class names and
forward signatures of the reference (``infer/ops/norm.py``, ``MLP.py``, ``embedding.py``, ``rope.py``,
``sampler.py``).  GEMMs go to the vendor library through ``F.linear``, except decode-sized batches over
shapes where this package's split-K weight-streaming kernel measures faster (``ops.linear``);
normalisation, the SwiGLU gate and everything on the cache path are this package's HIP kernels."""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from .context import get_context


class RMSNorm(nn.Module):
    """``infer/ops/norm.py:47-121``: ``forward(x)`` or ``forward(x, residual) -> (out, residual)``."""

    def __init__(self, hidden_size: int, eps: float = 1e-6):
        super().__init__()
        self.hidden_size = hidden_size
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.bfloat16), requires_grad=False)

    def forward(self, x: torch.Tensor, residual: torch.Tensor | None = None):
        return ops.rms_norm(x, self.weight, self.eps, residual)


class Linear(nn.Module):
    """``infer/ops/MLP.py:103-149``: weight ``[out, in]``, ``forward = F.linear``."""

    def __init__(self, in_features: int, out_features: int, bias: bool = False, dtype=torch.bfloat16):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight = nn.Parameter(torch.empty(int(out_features), in_features, dtype=dtype), requires_grad=False)
        if bias:
            self.bias = nn.Parameter(torch.empty(int(out_features), dtype=dtype), requires_grad=False)
        else:
            self.register_parameter("bias", None)

    @staticmethod
    def weight_loader(param: nn.Parameter, loaded_weight: torch.Tensor):
        param.data.copy_(loaded_weight)

    def forward(self, input: torch.Tensor, defer: bool = False):
        """``defer=True`` is for a caller that passes the result straight to an ``RMSNorm``: a split-K
        result may then come back unreduced (``ops.SplitKSum``) and the norm kernel adds the pieces."""
        if self.bias is None and input.dim() == 2 and input.shape[0] <= 128 and input.is_cuda:
            return ops.linear(input, self.weight, defer)    # decode-sized batch: measured choice of kernel
        return F.linear(input, self.weight, self.bias)


class QKVLinear(Linear):
    """``MLP.py:152-184``: q, k, v projections packed along the output dimension."""

    def __init__(self, hidden_size: int, q_size: int, kv_size: int, bias: bool = False):
        self.hidden_size = hidden_size
        self.q_size = q_size
        self.kv_size = kv_size
        super().__init__(hidden_size, q_size + 2 * kv_size, bias=bias)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, shard_id: str):
        assert shard_id in ("q", "k", "v")
        offset = {"q": 0, "k": self.q_size, "v": self.q_size + self.kv_size}[shard_id]
        size = self.q_size if shard_id == "q" else self.kv_size
        param.data.narrow(0, offset, size).copy_(loaded_weight)


class MergeLinear(Linear):
    """``MLP.py:186-198``: gate and up projections packed along the output dimension."""

    def __init__(self, hidden_size: int, output_size: list[int]):
        self.output_size = output_size
        super().__init__(hidden_size, sum(output_size), bias=False)

    def weight_loader(self, param: nn.Parameter, loaded_weight: torch.Tensor, shard_id: int):
        offset = 0 if shard_id == 0 else self.output_size[0]
        param.data.narrow(0, offset, self.output_size[shard_id]).copy_(loaded_weight)


class MLP(nn.Module):
    """SwiGLU feed-forward (``MLP.py:207-226``): ``down(silu(gate(x)) * up(x))``."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        self.intermediate_size = intermediate_size
        self.gate_up_proj = MergeLinear(hidden_size, [intermediate_size] * 2)
        self.down_proj = Linear(intermediate_size, hidden_size)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x = self.gate_up_proj(x)
        act = torch.empty(x.shape[:-1] + (self.intermediate_size,), dtype=x.dtype, device=x.device)
        ops.silu_and_mul(act, x)
        return self.down_proj(act, defer=True)      # consumed by the next RMSNorm (with its residual add)


class Embedding(nn.Module):
    """``infer/ops/embedding.py:7-16``."""

    def __init__(self, num_embeddings: int, embedding_dim: int):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.weight = nn.Parameter(torch.empty(num_embeddings, embedding_dim, dtype=torch.bfloat16),
                                   requires_grad=False)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return F.embedding(input, self.weight)


class LMHead(Embedding):
    """``embedding.py:18-32``: on a prefill step only each sequence's last row is projected."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        context = get_context()
        if context.is_prefill:
            last_indices = context.cu_seqlens_q[1:] - 1
            input = input[last_indices.long()].contiguous()
        return F.linear(input, self.weight)


_cos_sin_tables: dict = {}


def cos_sin_table(rotary_dim: int, max_position: int, base: float, device) -> torch.Tensor:
    """``Rope._compute_cos_sin_cache`` (``infer/ops/rope.py:97-108``): ``[max_position, rotary_dim]`` bf16,
    cos in the first half of a row and sin in the second.  The reference evaluates the inverse
    frequencies, the positions and their product in bf16; the same operations are issued here so
    that the table holds the same values.  One table is shared by all layers of a model."""
    key = (rotary_dim, max_position, float(base), str(device))
    table = _cos_sin_tables.get(key)
    if table is None:
        inv_freq = 1.0 / (base ** (torch.arange(0, rotary_dim, 2, dtype=torch.bfloat16, device=device) / rotary_dim))
        t = torch.arange(max_position, dtype=torch.bfloat16, device=device)
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        table = torch.cat((freqs.cos(), freqs.sin()), dim=-1).contiguous()
        _cos_sin_tables[key] = table
    return table


class Sampler(nn.Module):
    """``infer/ops/sampler.py:4-17``: greedy where the temperature is 0, otherwise a draw from the
    softmax by the exponential-race trick."""

    def forward(self, logits: torch.Tensor, temperatures: torch.Tensor, all_greedy: bool = False) -> torch.Tensor:
        if all_greedy:
            # The caller knows on the host that every temperature is 0.  Widening bf16 to float is exact
            # and order-preserving and argmax breaks ties by the lower index in either type, so the
            # float copy of the [batch, vocab] logits (0.4 ms per decode step at batch 128) is skipped.
            return logits.argmax(dim=-1)
        greedy = logits.argmax(dim=-1)
        # A draw from softmax(logits / T) as a race of exponentials: token i wins with probability p_i when
        # the contestants are p_i / e_i with e_i ~ Exp(1).  Same arithmetic and the same consumption of the
        # random stream as the reference (float32 throughout, 1e-10 added to the noise); rows with T = 0
        # produce NaNs here and take the greedy token below.
        probs = torch.softmax(logits.float() / temperatures.to(torch.float).unsqueeze(1), dim=-1)
        noise = torch.empty_like(probs).exponential_(1.0).add_(1e-10)
        sampled = (probs / noise).argmax(dim=-1)
        return torch.where(temperatures == 0, greedy, sampled)
