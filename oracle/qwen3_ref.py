"""TEST INFRASTRUCTURE ONLY: a float32 CPU restatement of the decoder that the engine runs
(``infer/models/Qwen3.py:59-321``), used by ``tests/`` to check whole steps of the engine (prefill,
decode, graph replay) end to end.  Nothing in the product imports this file.

It evaluates a whole sequence at once with dense causal attention - no cache, no paging, no
prefill/decode split - so it shares no structure with the path under test:

    h   = embed[tokens]
    per layer:  x = rmsnorm(h) ; q,k,v = x Wqkv^T ; q,k = rmsnorm_head(q), rmsnorm_head(k)
                q,k = neox_rope(q,k, positions) ; a = softmax(causal(q k^T / sqrt(D))) v   (GQA)
                h += a Wo^T ; x = rmsnorm(h) ; h += (silu(x Wg^T) * (x Wu^T)) Wd^T
    logits = rmsnorm(h) Wlm^T

``positions`` are explicit because the reference feeds decode tokens position ``len(seq)`` while its
prefill positions are zero-based (``infer/engine/model_runner.py:84,117``), and the rotary table is
an optional input because the reference tabulates cos/sin in bf16 (``infer/ops/rope.py:97-108``):
with ``cos_sin=None`` exact float32 angles are used, which is the textbook model.

Pinned (``tests/test_engine_oracle.py``) against the independent Qwen3 implementation of the
``transformers`` package on a random tiny configuration (logits equal to 1e-4), and against a
per-token scalar loop for the attention core.
"""
from __future__ import annotations

import math

import torch


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps) * w


def rope_angles(positions: torch.Tensor, head_dim: int, theta: float):
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    ang = positions.to(torch.float64)[:, None] * inv[None, :]
    return ang.cos().float(), ang.sin().float()


def neox_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [T, H, D]; cos/sin [T, D/2]; pairs are (i, i + D/2)."""
    x1, x2 = x.chunk(2, dim=-1)
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def forward_full(weights: dict, cfg, tokens, positions, cos_sin: torch.Tensor | None = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` (float32) of one sequence.  ``weights`` uses the engine's parameter names
    (packed ``qkv_proj`` / ``gate_up_proj``); values may be bf16, they are widened to float32."""
    W = {k: v.detach().float().cpu() for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.as_tensor(positions, dtype=torch.long)
    T = tokens.numel()
    Hq, Hkv, D = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    G = Hq // Hkv
    if cos_sin is None:
        cos, sin = rope_angles(positions, D, cfg.rope_theta)
    else:
        rows = cos_sin.detach().float().cpu()[positions]
        cos, sin = rows[:, :D // 2], rows[:, D // 2:]
    h = W["model.embed_tokens.weight"][tokens]
    causal = torch.ones(T, T, dtype=torch.bool).tril()
    for l in range(cfg.num_hidden_layers):
        p = f"model.layers.{l}."
        x = rmsnorm(h, W[p + "input_layernorm.weight"], cfg.rms_norm_eps)
        qkv = x @ W[p + "self_attn.qkv_proj.weight"].T
        q, k, v = qkv.split([Hq * D, Hkv * D, Hkv * D], dim=-1)
        q = rmsnorm(q.view(T, Hq, D), W[p + "self_attn.q_norm.weight"], cfg.rms_norm_eps)
        k = rmsnorm(k.view(T, Hkv, D), W[p + "self_attn.k_norm.weight"], cfg.rms_norm_eps)
        v = v.reshape(T, Hkv, D)
        q, k = neox_rope(q, cos, sin), neox_rope(k, cos, sin)
        out = torch.empty(T, Hq, D)
        for hq in range(Hq):
            s = (q[:, hq] @ k[:, hq // G].T) / math.sqrt(D)
            s = s.masked_fill(~causal, float("-inf"))
            out[:, hq] = torch.softmax(s, dim=-1) @ v[:, hq // G]
        h = h + out.view(T, Hq * D) @ W[p + "self_attn.o_proj.weight"].T
        x = rmsnorm(h, W[p + "post_attention_layernorm.weight"], cfg.rms_norm_eps)
        gu = x @ W[p + "mlp.gate_up_proj.weight"].T
        g, u = gu.chunk(2, dim=-1)
        h = h + (torch.nn.functional.silu(g) * u) @ W[p + "mlp.down_proj.weight"].T
    x = rmsnorm(h, W["model.norm.weight"], cfg.rms_norm_eps)
    lm = W.get("lm_head.weight", W["model.embed_tokens.weight"])
    return x @ lm.T


def engine_positions(num_prompt: int, num_total: int, decode_position_offset: int) -> list[int]:
    """Positions the engine feeds: prompt tokens 0..P-1, the i-th fed completion token
    ``P + i + offset`` (``model_runner.py:84`` and ``:117``)."""
    return list(range(num_prompt)) + [t + decode_position_offset for t in range(num_prompt, num_total)]


def attention_scalar(q, k, v, scale):
    """Per-token scalar loop of causal attention for one head, float64: pins the tensor form above."""
    T, D = q.shape
    out = torch.zeros(T, D, dtype=torch.float64)
    for t in range(T):
        scores = [float((q[t].double() * k[j].double()).sum()) * scale for j in range(t + 1)]
        m = max(scores)
        w = [math.exp(s - m) for s in scores]
        z = sum(w)
        for j in range(t + 1):
            out[t] += (w[j] / z) * v[j].double()
    return out
