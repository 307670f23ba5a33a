"""Fused QK-RMSNorm + neox RoPE + KV append on the GPU against oracle/rope_norm_ref.py.

Bar: the V rows are a byte copy (bit-exact); Q and K follow the reference's rounding points, so they
are compared at the tolerance of the reference's own rope test (test/op.py: atol = rtol = 1e-2) and,
more sharply, must be bit-identical on at least 99 % of the elements (the float32 reduction order of
the norm is the only freedom)."""
import numpy as np
import pytest
import torch

from infer_amd import ops
from oracle import rope_norm_ref as R
from oracle.paged_ref import bf16_to_f32
from tests.helpers import bits

pytestmark = pytest.mark.gpu


def make(n, hq, hkv, seed, gpu, nblk=8, bs=64, pad_every=5, max_pos=4096):
    g = torch.Generator().manual_seed(seed)
    d = 128
    qkv = (torch.randn((n, (hq + 2 * hkv) * d), generator=g) * 2).to(torch.bfloat16).to(gpu)
    q, k, v = qkv.split([hq * d, hkv * d, hkv * d], dim=-1)       # strided views, as in Qwen3.py:110-111
    q, k, v = q.view(n, hq, d), k.view(n, hkv, d), v.view(n, hkv, d)
    wq = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16).to(gpu)
    wk = (1 + 0.2 * torch.randn(d, generator=g)).to(torch.bfloat16).to(gpu)
    cache = torch.from_numpy(R.cos_sin_cache_ref(max_pos, d, 1e6).view(np.int16)).view(torch.bfloat16).to(gpu)
    pos = torch.randint(0, max_pos, (n,), generator=g).to(gpu)
    kc = torch.randn((nblk, bs, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    vc = torch.randn((nblk, bs, hkv, d), generator=g).to(torch.bfloat16).to(gpu)
    slots = torch.randperm(nblk * bs, generator=g)[:n].to(torch.int32)
    if pad_every:
        slots[::pad_every] = -1
    return qkv, q, k, v, wq, wk, cache, pos, kc, vc, slots.to(gpu)


def close(got_bits, want_bits):
    got, want = bf16_to_f32(got_bits), bf16_to_f32(want_bits)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= 1e-2 + 1e-2 * np.abs(want).max()
    assert (np.abs(got - want) <= 1e-2 + 1e-2 * np.abs(want)).mean() > 0.9999
    assert (got_bits == want_bits).mean() > 0.99


@pytest.mark.parametrize("n,hq,hkv", [(64, 32, 8), (1, 16, 8), (300, 32, 8), (37, 64, 8), (50, 8, 2), (5, 4, 1)])
def test_against_oracle(gpu, n, hq, hkv):
    qkv, q, k, v, wq, wk, cache, pos, kc, vc, slots = make(n, hq, hkv, n + hq, gpu)
    ek, ev = bits(kc).copy(), bits(vc).copy()
    q2, k2 = R.qk_norm_rope_append_ref(bits(q.contiguous()), bits(k.contiguous()), bits(v.contiguous()),
                                       pos.cpu().numpy(), bits(wq), bits(wk), 1e-6, bits(cache), ek, ev,
                                       slots.cpu().numpy())
    v_before = v.clone()
    ops.qk_norm_rope_store_kvcache(q, k, v, pos, wq, wk, 1e-6, cache, kc, vc, slots)
    torch.cuda.synchronize()
    close(bits(q.contiguous()), q2)
    close(bits(k.contiguous()), k2)
    assert torch.equal(v, v_before)                              # V is only read
    assert np.array_equal(bits(vc), ev)                          # V cache: byte copy, padding rows skipped
    close(bits(kc), ek)
    valid = (slots >= 0).cpu().numpy()
    rows = slots.cpu().numpy()[valid]
    width = hkv * 128
    assert np.array_equal(bits(kc).reshape(-1, width)[rows], bits(k.contiguous()).reshape(n, width)[valid])
    untouched = np.ones(kc.shape[0] * kc.shape[1], bool)
    untouched[rows] = False
    assert np.array_equal(bits(kc).reshape(-1, width)[untouched], ek.reshape(-1, width)[untouched])


def test_rows_of_extreme_magnitude(gpu):
    """Head rows of zeros (variance 0: the norm is eps alone), of very large, very small and alternating
    magnitudes: the sums of squares and the products keep float32 range and the reference's rounding points."""
    n, hq, hkv = 48, 32, 8
    qkv, q, k, v, wq, wk, cache, pos, kc, vc, slots = make(n, hq, hkv, 77, gpu)
    with torch.no_grad():
        q[0::6] = 0
        k[0::6] = 0
        q[1::6] *= 1000.0
        k[1::6] *= 1000.0
        q[2::6] *= 1e-3
        k[2::6] *= 1e-3
        q[3::6, :, ::2] *= 300.0                                   # large and small elements side by side
        k[3::6, :, 1::2] *= 1e-2
    ek, ev = bits(kc).copy(), bits(vc).copy()
    q2, k2 = R.qk_norm_rope_append_ref(bits(q.contiguous()), bits(k.contiguous()), bits(v.contiguous()),
                                       pos.cpu().numpy(), bits(wq), bits(wk), 1e-6, bits(cache), ek, ev,
                                       slots.cpu().numpy())
    ops.qk_norm_rope_store_kvcache(q, k, v, pos, wq, wk, 1e-6, cache, kc, vc, slots)
    torch.cuda.synchronize()
    keep = np.arange(n) % 6 != 0                                   # the zero rows are compared as values: +0 and -0 are both right
    gq, gk = bits(q.contiguous()), bits(k.contiguous())
    close(gq[keep], q2[keep])
    close(gk[keep], k2[keep])
    assert np.array_equal(bits(vc), ev)
    assert (gq[~keep] & 0x7fff == 0).all() and (q2[~keep] & 0x7fff == 0).all()
    assert (gk[~keep] & 0x7fff == 0).all() and (k2[~keep] & 0x7fff == 0).all()
    got_kc, want_kc = bf16_to_f32(bits(kc)), bf16_to_f32(ek)
    assert np.abs(got_kc - want_kc).max() <= 1e-2 + 1e-2 * np.abs(want_kc).max()


def test_key_can_be_left_untouched(gpu):
    qkv, q, k, v, wq, wk, cache, pos, kc, vc, slots = make(20, 16, 8, 3, gpu, pad_every=0)
    k_before = k.clone()
    ops.qk_norm_rope_store_kvcache(q, k, v, pos, wq, wk, 1e-6, cache, kc, vc, slots, write_key=False)
    assert torch.equal(k, k_before)
    assert not torch.equal(kc.view(-1, 8, 128)[slots.long()], k_before)      # the cache holds the rotated rows


def test_equals_the_unfused_sequence_on_the_gpu(gpu):
    """norm -> rope -> store_kvcache done with torch ops and the plain append kernel (the reference's
    order, Qwen3.py:113-131) gives the same caches and the same Q."""
    qkv, q, k, v, wq, wk, cache, pos, kc, vc, slots = make(128, 32, 8, 9, gpu)
    kc2, vc2 = kc.clone(), vc.clone()

    def norm(x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16) * w

    def rope(x):
        cs = cache[pos]
        cos, sin = cs[:, None, :64], cs[:, None, 64:]
        x1, x2 = x[..., :64], x[..., 64:]
        return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)

    q_ref, k_ref = rope(norm(q, wq)), rope(norm(k, wk))
    ops.store_kvcache(k_ref, v.contiguous(), kc2, vc2, slots)
    ops.qk_norm_rope_store_kvcache(q, k, v, pos, wq, wk, 1e-6, cache, kc, vc, slots)
    torch.cuda.synchronize()
    close(bits(q.contiguous()), bits(q_ref))
    close(bits(kc), bits(kc2))
    assert torch.equal(vc, vc2)


def test_position_zero_and_unit_weight_is_plain_normalisation(gpu):
    qkv, q, k, v, wq, wk, cache, pos, kc, vc, slots = make(16, 8, 8, 11, gpu, pad_every=0)
    ones = torch.ones(128, dtype=torch.bfloat16, device=gpu)
    q0 = q.clone()
    ops.qk_norm_rope_store_kvcache(q, k, v, torch.zeros_like(pos), ones, ones, 0.0, cache, kc, vc, slots)
    want = (q0.float() * torch.rsqrt(q0.float().pow(2).mean(-1, keepdim=True))).to(torch.bfloat16)
    close(bits(q.contiguous()), bits(want))
