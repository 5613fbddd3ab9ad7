"""The two checks every value comparison of the GPU tests goes through.

1. The mandated tolerance: ``isclose(rtol=1e-2, atol=1e-2)`` against the
   fp32-accumulated oracle, element by element.  On its own it is nearly blind
   where outputs are small: with K = 64 and operands ~ N(0, 0.02) the outputs
   have a standard deviation of 0.0032, a third of ``atol``, and an all-zero
   result trips 0.2 % of the elements.
2. A sharper companion, per 16 x 16 block (the unit one MFMA accumulates):
   ``||got - want||_F <= BLOCK_RTOL * ||want||_F + BLOCK_EPS``.  A 16-bit
   result rounds at 2^-9 (bf16) or 2^-12 (fp16) relative and fp32 summation
   order adds ~1e-6, so 2^-7 leaves a factor of four; a dropped K-substep, a
   zeroed or misplaced fragment, or rows swapped inside a block are off by
   tens of percent of the block's norm whatever the scale of the operands.

``make_ab`` scales its operands so that outputs are O(1) unless a test asks
for a scale of its own.
"""

import torch

RTOL, ATOL = 1e-2, 1e-2
BLOCK = 16
BLOCK_RTOL = 2.0 ** -7
# a block whose expected values are all (near) zero: 256 elements, each within a few fp32 ulps of tiny numbers
BLOCK_EPS = 1e-5


def default_scale(K):
    """Operand scale that gives outputs a standard deviation of about 1:
    sum of K products of two N(0, s) values has deviation s^2 sqrt(K)."""
    return float(max(K, 1)) ** -0.25


def make_ab(M, N, K, dtype, scale=None, seed=123, lda=None, ldb=None):
    """Seeded A [M,K] row-major and B [K,N] K-contiguous (the reference's TN
    layout, benchmark.py:101-102); optional leading dimensions > K give the
    strided K-shard views of 08/09."""
    g = torch.Generator().manual_seed(seed)
    if scale is None:
        scale = default_scale(K)
    lda, ldb = lda or K, ldb or K
    Af = (torch.randn(M, lda, generator=g) * scale).to(dtype)
    Bf = (torch.randn(N, ldb, generator=g) * scale).to(dtype)
    return Af[:, :K], Bf[:, :K].T


def block_errors(got, want):
    """(error norm, reference norm) per BLOCK x BLOCK block of two matrices
    (edges padded with zeros on both sides)."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape and got.dim() == 2
    M, N = got.shape
    pm, pn = (-M) % BLOCK, (-N) % BLOCK
    if pm or pn:
        got = torch.nn.functional.pad(got, (0, pn, 0, pm))
        want = torch.nn.functional.pad(want, (0, pn, 0, pm))
    bm, bn = got.shape[0] // BLOCK, got.shape[1] // BLOCK

    def norms(x):
        return x.double().reshape(bm, BLOCK, bn, BLOCK).pow(2).sum(dim=(1, 3)).sqrt()

    return norms(got - want), norms(want)


def blocks_ok(got, want, block_rtol=BLOCK_RTOL):
    """Boolean matrix: which blocks pass the per-block bound."""
    err, ref = block_errors(got, want)
    return err <= block_rtol * ref + BLOCK_EPS


def check_close(got, want, what="", block_rtol=BLOCK_RTOL):
    """Both checks.  ``block_rtol=None`` skips the second one (results that
    are rounded to 16 bits several times on the way, e.g. 16-bit atomics)."""
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} against {tuple(want.shape)}"
    bad = ~torch.isclose(got, want, rtol=RTOL, atol=ATOL)
    assert not bad.any(), f"{what}: {int(bad.sum())} mismatches, max abs err {(got - want).abs().max().item()}"
    if block_rtol is None or got.numel() == 0:
        return
    if got.dim() != 2:
        got, want = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
    err, ref = block_errors(got, want)
    ok = err <= block_rtol * ref + BLOCK_EPS
    if not bool(ok.all()):
        idx = torch.nonzero(~ok)
        i, j = int(idx[0, 0]), int(idx[0, 1])
        raise AssertionError(
            f"{what}: {int((~ok).sum())} of {ok.numel()} 16x16 blocks are off by more than 2^{torch.log2(torch.tensor(block_rtol)).item():.0f} "
            f"of their norm; first at rows {i * BLOCK}.., columns {j * BLOCK}..: error norm {err[i, j].item():.4g}, "
            f"block norm {ref[i, j].item():.4g}")
