"""Pins oracle/rope_norm_ref.py on the CPU against the reference's formulas written with torch's own
bf16 tensor arithmetic, and against closed forms."""
import numpy as np
import torch

from oracle import rope_norm_ref as R
from oracle.paged_ref import bf16_to_f32
from tests.helpers import bits


def from_bits(u):
    return torch.from_numpy(u.view(np.int16).copy()).view(torch.bfloat16)


def rand_bits(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return bits((torch.randn(shape, generator=g) * scale).to(torch.bfloat16))


def test_rope_matches_torch_bf16_arithmetic_bit_for_bit():
    x = rand_bits((33, 5, 128), 0)
    cache = R.cos_sin_cache_ref(512, 128, 1e6)
    pos = np.random.default_rng(0).integers(0, 512, 33)
    got = R.rope_neox_ref(x, cache, pos)
    # infer/ops/rope.py:48-66 with bf16 tensors: every op rounds to bf16
    xt = from_bits(x)
    cs = from_bits(cache)[torch.from_numpy(pos)]
    cos, sin = cs[:, None, :64], cs[:, None, 64:]
    x1, x2 = xt[..., :64], xt[..., 64:]
    want = torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)
    assert np.array_equal(got, bits(want))


def test_rope_closed_forms():
    x = rand_bits((4, 2, 128), 1)
    cache = R.cos_sin_cache_ref(64, 128, 10000.0)
    same = R.rope_neox_ref(x, cache, np.zeros(4, dtype=np.int64))      # position 0: cos 1, sin 0
    assert np.array_equal(same, x)
    rot = bf16_to_f32(R.rope_neox_ref(x, cache, np.array([1, 7, 30, 63])))
    xf = bf16_to_f32(x)
    # a rotation preserves the norm of every (i, i + 64) pair, up to bf16 rounding
    n0 = xf[..., :64] ** 2 + xf[..., 64:] ** 2
    n1 = rot[..., :64] ** 2 + rot[..., 64:] ** 2
    assert np.abs(n1 - n0).max() <= 0.05 * max(1.0, float(n0.max()))
    # and moves things: not the identity
    assert np.abs(rot - xf).max() > 0.1


def test_rms_norm_matches_torch_within_one_ulp_and_closed_forms():
    x = rand_bits((50, 8, 128), 2, scale=3.0)
    w = rand_bits((128,), 3)
    got = bf16_to_f32(R.rms_norm_ref(x, w, 1e-6))
    xt = from_bits(x).float()                                           # infer/ops/norm.py:63-73, eager
    var = xt.pow(2).mean(dim=-1, keepdim=True)
    want = (xt * torch.rsqrt(var + 1e-6)).to(torch.bfloat16).mul_(from_bits(w)).float().numpy()
    ulp = np.maximum(np.abs(want), 2.0 ** -126) * 2.0 ** -7
    assert (np.abs(got - want) <= ulp).all()
    assert (got == want).mean() > 0.99
    # unit weight, constant row c: output is sign(c) (mean square is c^2)
    ones = bits(torch.ones(128, dtype=torch.bfloat16))
    const = bits(torch.full((1, 1, 128), -2.5, dtype=torch.bfloat16))
    assert np.allclose(bf16_to_f32(R.rms_norm_ref(const, ones, 0.0)), -1.0)
    # scale invariance of the normalised direction (power-of-two scale is exact in bf16)
    a = bf16_to_f32(R.rms_norm_ref(x, ones, 0.0))
    b = bf16_to_f32(R.rms_norm_ref(bits(from_bits(x) * 4), ones, 0.0))
    assert np.array_equal(a, b)


def test_fused_sequence_is_norm_then_rope_then_append():
    n, hq, hkv, d = 9, 4, 2, 128
    q, k, v = rand_bits((n, hq, d), 4), rand_bits((n, hkv, d), 5), rand_bits((n, hkv, d), 6)
    wq, wk = rand_bits((d,), 7), rand_bits((d,), 8)
    cache = R.cos_sin_cache_ref(100, d, 1e6)
    pos = np.arange(n) * 3
    kc = np.zeros((2, 8, hkv, d), np.uint16)
    vc = np.zeros_like(kc)
    slots = np.array([0, 3, -1, 5, 9, 15, -1, 1, 2], dtype=np.int32)
    q2, k2 = R.qk_norm_rope_append_ref(q, k, v, pos, wq, wk, 1e-6, cache, kc, vc, slots)
    assert np.array_equal(q2, R.rope_neox_ref(R.rms_norm_ref(q, wq, 1e-6), cache, pos))
    flat_k, flat_v = kc.reshape(-1, hkv, d), vc.reshape(-1, hkv, d)
    for i, s in enumerate(slots):
        if s >= 0:
            assert np.array_equal(flat_k[s], k2[i]) and np.array_equal(flat_v[s], v[i])
    assert not flat_k[4].any() and not flat_k[6].any()
