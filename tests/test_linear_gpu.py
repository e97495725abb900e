"""The decode step's projections for a few activation rows (daisy_linear_rows_fwd) against the same product in
float64 (models/daisy/attention.py:119-120 and :201 are F.linear on bf16 tensors: fp32 accumulation, one rounding).

Tolerance: the result is one bf16 rounding (relative 2^-9) away from the exact product, plus the error of the fp32
sums, K * 2^-24 of the sum of the absolute terms at most."""
import pytest
import torch

from daisy_amd import _lib, ops
from helpers import say

pytestmark = pytest.mark.gpu


def _check(y, x, w):
    xd, wd = x.double().cpu(), w.double().cpu()
    ref = xd.reshape(-1, xd.shape[-1]) @ wd.t()
    mag = xd.reshape(-1, xd.shape[-1]).abs() @ wd.abs().t()
    got = y.double().cpu().reshape(ref.shape)
    K = w.shape[1]
    tol = ref.abs() * 2.0 ** -8 + mag * (K * 2.0 ** -24) + 1e-30
    bad = (got - ref).abs() > tol
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} outputs off: worst {((got - ref).abs() / tol).max().item():.2f} x tolerance"


@pytest.mark.parametrize("M,N,K", [
    (1, 4608, 1536),     # QKV projection of model_specs/daisy_milli.yml, one sequence
    (1, 1536, 1536),     # its output projection
    (2, 768, 768),
    (3, 100, 64),        # fewer 16-byte pieces per row than lanes
    (4, 1000, 1544),     # N not a multiple of the rows per wavefront, K not a multiple of 512
    (8, 513, 520),
    (5, 7, 8),
    (1, 1, 8),
    (7, 4099, 1024),
    (2, 50304, 768),     # a vocabulary projection
])
def test_linear_rows_matches_the_exact_product(M, N, K):
    say(f"linear rows M{M} N{N} K{K}")
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x = torch.randn(M, K, generator=g).bfloat16().cuda()
    w = (torch.randn(N, K, generator=g) * K ** -0.5).bfloat16().cuda()
    y = ops.linear_rows(x, w)
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    _check(y, x, w)
    # the library's GEMM on the same tensors: equal up to the last bf16 bit of a few outputs
    lib_y = torch.nn.functional.linear(x, w)
    diff = (y.float() - lib_y.float()).abs()
    assert (diff <= lib_y.float().abs() * 2.0 ** -7 + 1e-6).all()
    say(f"  outputs that differ from the library's in the last bit: {int((diff > 0).sum())} of {diff.numel()}")


def test_linear_rows_takes_strided_rows_and_leading_dims():
    """Weight rows that are rows of a wider matrix (a slice of the merged qkvo parameter is contiguous, a column
    block of a bigger one is not), activations [B, 1, K] as a step has them, an output buffer of the caller's."""
    g = torch.Generator().manual_seed(3)
    big = torch.randn(300, 1024, generator=g).bfloat16().cuda()
    w = big[:, 256:768]                       # [300, 512], row stride 1024
    x = torch.randn(4, 1, 512, generator=g).bfloat16().cuda()
    assert ops.linear_rows_ok(x, w)
    y = ops.linear_rows(x, w)
    assert y.shape == (4, 1, 300)
    _check(y, x, w)
    out = torch.full((4, 1, 300), 7.0, dtype=torch.bfloat16, device="cuda")
    assert ops.linear_rows(x, w, out=out) is out and torch.equal(out, y)
    xs = torch.randn(3, 2, 512, generator=g).bfloat16().cuda()[:, 0]      # rows 1024 elements apart
    _check(ops.linear_rows(xs, w), xs, w)


def test_linear_rows_refusals():
    x = torch.zeros(9, 64, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(16, 64, dtype=torch.bfloat16, device="cuda")
    assert not ops.linear_rows_ok(x, w)
    with pytest.raises(RuntimeError, match="at most 8"):
        ops.linear_rows(x, w)
    assert not ops.linear_rows_ok(x[:1, :60], w[:, :60])
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.linear_rows(x[:1, :60].contiguous(), w[:, :60].contiguous())
    with pytest.raises(TypeError):
        ops.linear_rows(x[:1].float(), w)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.linear_rows(x[:1].cpu(), w.cpu())
    assert not ops.linear_rows_ok(x[:1].cpu(), w.cpu())
    assert _lib.LINEAR_MAX_ROWS == 8
