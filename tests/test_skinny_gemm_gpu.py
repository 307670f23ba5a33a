"""Split-K weight-streaming GEMM (decode-sized batches) against a float32 reference.

Bar: the bf16 result is within two bf16 steps of the float32 product rounded once (the vendor GEMM
meets the same bar: both accumulate in float32, in different orders)."""
import pytest
import torch

from infer_amd import ops

pytestmark = pytest.mark.gpu


def reference(x, w):
    return x.float() @ w.float().T


def close(got, want):
    assert torch.isfinite(got.float()).all()
    err = (got.float() - want).abs()
    assert (err <= 2.0 ** -6 * want.abs() + 2e-2).all(), float(err.max())


@pytest.mark.parametrize("m,n,k", [
    (128, 4096, 12288),      # down_proj of Qwen3-8B: split over K
    (128, 4096, 4096),       # o_proj
    (64, 6144, 4096), (16, 4096, 4096), (1, 4096, 4096), (17, 1024, 1024), (100, 5120, 8192),
    (128, 24576, 4096),      # gate_up: enough tiles, no split
    (33, 136, 128),          # ragged N (not a multiple of the tile), a single chunk
    (128, 264, 384), (5, 8, 128),
])
def test_against_float32(gpu, m, n, k):
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(gpu)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16).to(gpu)
    got = ops.skinny_linear(x, w)
    torch.cuda.synchronize()
    close(got, reference(x, w))
    lib = torch.nn.functional.linear(x, w)
    assert (got.float() - lib.float()).abs().max() <= 2.0 ** -6 * reference(x, w).abs().max() + 2e-2


def test_strided_input_and_output_views(gpu):
    g = torch.Generator().manual_seed(0)
    wide = torch.randn(48, 1024 + 256, generator=g).to(torch.bfloat16).to(gpu)
    x = wide[:, 256:]                                   # row stride 1280, 16-byte aligned start
    w = (torch.randn(512, 1024, generator=g) * 0.05).to(torch.bfloat16).to(gpu)
    out_wide = torch.zeros(48, 512 + 64, dtype=torch.bfloat16, device=gpu)
    ops.skinny_linear(x, w, out_wide[:, :512])
    torch.cuda.synchronize()
    close(out_wide[:, :512], reference(x, w))
    assert not out_wide[:, 512:].any()


def test_exact_small_integers(gpu):
    """Products and sums of small integers are exact in bf16 x bf16 -> float32: any indexing mistake
    (a wrong row, a dropped or doubled K chunk, a misplaced partial sum) changes the result."""
    g = torch.Generator().manual_seed(1)
    x = torch.randint(-1, 2, (77, 1536), generator=g).to(torch.bfloat16).to(gpu)
    w = torch.randint(-1, 2, (4096, 1536), generator=g).to(torch.bfloat16).to(gpu)
    got = ops.skinny_linear(x, w)
    want = reference(x, w)
    assert want.abs().max() < 256                       # representable in bf16 without rounding
    assert torch.equal(got.float(), want)


def test_unsupported_shapes_are_refused(gpu):
    w = torch.zeros(64, 192, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(RuntimeError):
        ops.skinny_linear(torch.zeros(4, 192, dtype=torch.bfloat16, device=gpu), w)        # K % 128 != 0
    w = torch.zeros(64, 256, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(RuntimeError):
        ops.skinny_linear(torch.zeros(129, 256, dtype=torch.bfloat16, device=gpu), w)      # M > 128
    assert not ops.skinny_linear_supported(129, 64, 256)
    assert not ops.skinny_linear_supported(4, 64, 192)


def test_linear_picks_one_kernel_per_shape_and_matches(gpu):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(128, 12288, generator=g).to(torch.bfloat16).to(gpu)
    w = (torch.randn(4096, 12288, generator=g) * 0.02).to(torch.bfloat16).to(gpu)
    a = ops.linear(x, w)
    b = ops.linear(x, w)
    assert torch.equal(a, b)                             # the choice is sticky: same kernel, same bits
    close(a, reference(x, w))
    big = torch.randn(300, 12288, generator=g).to(torch.bfloat16).to(gpu)
    close(ops.linear(big, w), reference(big, w))         # larger batches take the vendor GEMM


@pytest.mark.parametrize("m,n,k,with_residual", [(128, 4096, 12288, True), (40, 4096, 4096, True), (7, 1024, 2048, False)])
def test_rms_norm_adds_unreduced_partial_sums_to_the_same_bits(gpu, m, n, k, with_residual):
    """RMSNorm fed with the unreduced split-K result must give exactly what reducing first gives."""
    g = torch.Generator().manual_seed(m + k)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(gpu)
    w = (torch.randn(n, k, generator=g) * 0.03).to(torch.bfloat16).to(gpu)
    gamma = (1 + 0.2 * torch.randn(n, generator=g)).to(torch.bfloat16).to(gpu)
    res_a = torch.randn(m, n, generator=g).to(torch.bfloat16).to(gpu) if with_residual else None
    res_b = res_a.clone() if with_residual else None
    finished = ops.skinny_linear(x, w)
    want = ops.rms_norm(finished, gamma, 1e-6, res_a)
    deferred = ops.skinny_linear_deferred(x, w)
    assert isinstance(deferred, ops.SplitKSum) and deferred.partial.shape[0] > 1
    assert torch.equal(deferred.materialize(), finished)
    got = ops.rms_norm(deferred, gamma, 1e-6, res_b)
    torch.cuda.synchronize()
    if with_residual:
        assert torch.equal(got[0], want[0]) and torch.equal(res_b, res_a)
    else:
        assert torch.equal(got, want)


def test_partial_sums_cannot_be_used_after_a_later_split_gemm(gpu):
    x = torch.zeros(8, 4096, dtype=torch.bfloat16, device=gpu)
    w = torch.zeros(1024, 4096, dtype=torch.bfloat16, device=gpu)
    first = ops.skinny_linear_deferred(x, w)
    assert isinstance(first, ops.SplitKSum)
    ops.skinny_linear_deferred(x, w)
    with pytest.raises(RuntimeError, match="overwritten"):
        ops.rms_norm(first, torch.ones(1024, dtype=torch.bfloat16, device=gpu), 1e-6)
