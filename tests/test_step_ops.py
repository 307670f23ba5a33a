"""The elementwise operators of a decode step (RMSNorm with residual, SwiGLU gate, device-side decode
metadata): oracle pinned on the CPU, HIP kernels checked against the oracle on the GPU.

Bar on the GPU: the residual output and the metadata are exact; normalised values follow the
reference's rounding points, so at least 99 % of the elements are bit-identical to the oracle and all
are within two bf16 steps of it (the float32 reduction order is the only freedom)."""
import numpy as np
import pytest
import torch

from oracle import step_ops_ref as S
from oracle.paged_ref import bf16_to_f32, decode_metadata_ref
from tests.helpers import bits


def _bf16(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_add_rms_norm_oracle_vs_torch_bf16():
    """The same sequence of operations issued with torch tensors (float32 math, ``.to(bfloat16)`` where
    the reference rounds) must give the oracle's bits."""
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(17, 512, generator=g) * 3).to(torch.bfloat16)
    r = torch.randn(17, 512, generator=g).to(torch.bfloat16)
    w = (1 + 0.3 * torch.randn(512, generator=g)).to(torch.bfloat16)
    s = x.float() + r.float()
    res = s.to(torch.bfloat16)
    var = s.pow(2).mean(dim=-1, keepdim=True)
    want = (s * torch.rsqrt(var + 1e-6)).to(torch.bfloat16) * w
    out, new_res = S.add_rms_norm_ref(_bf16(x), _bf16(w), 1e-6, _bf16(r))
    assert np.array_equal(new_res, _bf16(res))
    assert (out == _bf16(want)).mean() > 0.995       # rsqrt vs 1/sqrt may differ in the last float bit
    assert np.abs(bf16_to_f32(out) - want.float().numpy()).max() <= 2 ** -6
    # value check against float64 rms norm
    exact = torch.nn.functional.rms_norm(s.double(), (512,), w.double(), 1e-6)
    assert (np.abs(bf16_to_f32(out) - exact.numpy()) <= 2.0 ** -6 * np.abs(exact.numpy()) + 1e-6).all()


def test_rms_norm_oracle_without_residual_is_the_residual_free_formula():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 256, generator=g).to(torch.bfloat16)
    w = torch.ones(256).to(torch.bfloat16)
    out = S.add_rms_norm_ref(_bf16(x), _bf16(w), 1e-6)
    xf = x.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    assert (out == _bf16(want)).mean() > 0.995


def test_silu_and_mul_oracle_vs_torch_bf16():
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(9, 2 * 384, generator=g) * 4).to(torch.bfloat16)
    gate, up = x[:, :384].float(), x[:, 384:]
    want = (gate / (1 + torch.exp(-gate))).to(torch.bfloat16) * up
    got = S.silu_and_mul_ref(_bf16(x))
    assert (got == _bf16(want)).mean() > 0.995
    exact = torch.nn.functional.silu(gate.double()) * up.double()
    assert (np.abs(bf16_to_f32(got) - exact.numpy()) <= 2.0 ** -6 * np.abs(exact.numpy()) + 1e-6).all()


def _near(got_bits, want_bits, frac=0.99):
    got, want = bf16_to_f32(got_bits), bf16_to_f32(want_bits)
    assert np.isfinite(got).all()
    assert (got_bits == want_bits).mean() >= frac
    # a flip of the first rounding moves the product by one bf16 step and can tip its rounding too
    assert (np.abs(got - want) <= 2.0 ** -6 * np.abs(want) + 1e-30).all()


@pytest.mark.gpu
@pytest.mark.parametrize("n,hidden", [(64, 4096), (1, 1024), (300, 5120), (7, 256), (16, 8192), (3, 136)])
def test_rms_norm_gpu(gpu, n, hidden):
    from infer_amd import ops
    g = torch.Generator().manual_seed(n + hidden)
    x = (torch.randn(n, hidden, generator=g) * 2).to(torch.bfloat16)
    r = torch.randn(n, hidden, generator=g).to(torch.bfloat16)
    w = (1 + 0.3 * torch.randn(hidden, generator=g)).to(torch.bfloat16)
    want_out, want_res = S.add_rms_norm_ref(_bf16(x), _bf16(w), 1e-6, _bf16(r))
    want_plain = S.add_rms_norm_ref(_bf16(x), _bf16(w), 1e-6)
    xd, rd, wd = x.to(gpu), r.to(gpu), w.to(gpu)
    out, res = ops.rms_norm(xd, wd, 1e-6, rd)
    assert res is rd
    torch.cuda.synchronize()
    assert np.array_equal(bits(res), want_res)              # the residual is an exact bf16 sum
    _near(bits(out), want_out)
    _near(bits(ops.rms_norm(xd, wd, 1e-6)), want_plain)
    # in place (out aliases x) and on a strided view
    wide = torch.zeros(n, hidden + 64, dtype=torch.bfloat16, device=gpu)
    view = wide[:, :hidden]
    view.copy_(xd)
    ops.rms_norm(view, wd, 1e-6, out=view)
    torch.cuda.synchronize()
    _near(bits(view.contiguous()), want_plain)
    assert not wide[:, hidden:].any()


@pytest.mark.gpu
def test_rms_norm_rejects_unsupported(gpu):
    from infer_amd import ops
    x = torch.zeros(2, 8200, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(RuntimeError):
        ops.rms_norm(x, torch.ones(8200, dtype=torch.bfloat16, device=gpu), 1e-6)
    x = torch.zeros(2, 132, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(RuntimeError):
        ops.rms_norm(x, torch.ones(132, dtype=torch.bfloat16, device=gpu), 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("n,d", [(64, 12288), (1, 3072), (37, 25600), (5, 8), (128, 512)])
def test_silu_and_mul_gpu(gpu, n, d):
    from infer_amd import ops
    g = torch.Generator().manual_seed(n + d)
    x = (torch.randn(n, 2 * d, generator=g) * 3).to(torch.bfloat16)
    want = S.silu_and_mul_ref(_bf16(x))
    out = torch.empty(n, d, dtype=torch.bfloat16, device=gpu)
    ops.silu_and_mul(out, x.to(gpu))
    torch.cuda.synchronize()
    _near(bits(out), want, frac=0.98)         # expf of the device and of numpy may differ in the last bit


@pytest.mark.gpu
@pytest.mark.parametrize("offset", [0, 1])
def test_decode_metadata_gpu(gpu, offset):
    from infer_amd import ops
    rng = np.random.default_rng(5)
    bs, cols, batch = 256, 16, 48
    lengths = [int(x) for x in rng.integers(1, bs * cols + 1, size=batch)]
    lengths[:4] = [1, 256, 257, 4096]
    tables = [[int(b) for b in rng.permutation(1000)[: (n + bs - 1) // bs]] for n in lengths]
    slots, ctx, padded = decode_metadata_ref(lengths, tables, bs)
    n_pad = 16                                                   # graph padding rows: length 0
    lens_d = torch.tensor(lengths + [0] * n_pad, dtype=torch.int32, device=gpu)
    table_np = np.full((batch + n_pad, cols), 7, dtype=np.int32)         # stale entries in unused cells
    for i, t in enumerate(tables):
        table_np[i, :len(t)] = t
    table_d = torch.from_numpy(table_np).to(gpu)
    pos = torch.full((batch + n_pad,), -9, dtype=torch.int64, device=gpu)
    sm = torch.full((batch + n_pad,), -9, dtype=torch.int32, device=gpu)
    cl = torch.full((batch + n_pad,), -9, dtype=torch.int32, device=gpu)
    ops.decode_metadata(lens_d, table_d, bs, offset, pos, sm, cl)
    torch.cuda.synchronize()
    assert np.array_equal(sm.cpu().numpy()[:batch], slots)
    assert np.array_equal(cl.cpu().numpy()[:batch], ctx)
    assert pos.cpu().tolist()[:batch] == [n - 1 + offset for n in lengths]
    assert (sm.cpu().numpy()[batch:] == -1).all() and (cl.cpu().numpy()[batch:] == 0).all()
    assert (pos.cpu().numpy()[batch:] == 0).all()
    # a negative table entry (unallocated) yields slot -1 instead of a negative address
    table_np[0, 0] = -1
    ops.decode_metadata(lens_d, torch.from_numpy(table_np).to(gpu), bs, offset, pos, sm, cl)
    assert sm.cpu().numpy()[0] == -1
