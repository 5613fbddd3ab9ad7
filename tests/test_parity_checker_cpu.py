"""The checker of the GPU parity tests, tested on the CPU: results with one
plausible kernel mistake each must fail it at every shape the scatter tests
run, and a correctly rounded result must pass.

The mandated element-wise tolerance (rtol 1e-2 / atol 1e-2) alone lets most of
these through on small shapes; the per-block bound of ``parity.check_close``
is what catches them.
"""

import pytest
import torch

from oracle import iris_oracle as O
from parity import ATOL, RTOL, blocks_ok, check_close, make_ab
from test_gemm_gpu import SCATTER_CASES

SHAPES = sorted({(M, N, K, dtype) for (M, N, K, _bm, _bn, _g, _grid, dtype) in SCATTER_CASES}, key=str)


def product(A, B, dtype, k_drop=None, block=None):
    """fp32 product rounded to ``dtype``; with ``k_drop`` = (k0, k1) the K range
    [k0, k1) is left out of the 16 x 16 block ``block`` = (i, j)."""
    acc = A.float() @ B.float()
    if k_drop is not None:
        i, j = block
        k0, k1 = k_drop
        rows, cols = slice(16 * i, 16 * i + 16), slice(16 * j, 16 * j + 16)
        acc[rows, cols] -= A[rows, k0:k1].float() @ B[k0:k1, cols].float()
    return acc.to(dtype)


def a_block(M, N):
    """A 16 x 16 block that lies wholly inside the matrix (or the first one)."""
    return (min(1, max(0, M // 16 - 1)), min(2, max(0, N // 16 - 1)))


@pytest.mark.parametrize("M,N,K,dtype", SHAPES)
def test_a_correct_result_passes(M, N, K, dtype):
    A, B = make_ab(M, N, K, dtype)
    want = O.shard_gemm(A, B, dtype)
    # the same sum in another order (two halves of K added afterwards), rounded once
    h = (K // 2) // 8 * 8
    got = (A[:, :h].float() @ B[:h].float() + A[:, h:].float() @ B[h:].float()).to(dtype)
    check_close(got, want, "two halves of K")


@pytest.mark.parametrize("M,N,K,dtype", SHAPES)
def test_a_dropped_k_substep_in_one_block_fails(M, N, K, dtype):
    A, B = make_ab(M, N, K, dtype)
    want = O.shard_gemm(A, B, dtype)
    k1 = min(K, 32)
    got = product(A, B, dtype, k_drop=(0, k1), block=a_block(M, N))
    with pytest.raises(AssertionError):
        check_close(got, want, "dropped substep")
    # ... and exactly that block is named
    ok = blocks_ok(got, want)
    i, j = a_block(M, N)
    assert not bool(ok[i, j]) and int((~ok).sum()) == 1


@pytest.mark.parametrize("M,N,K,dtype", SHAPES)
def test_a_zeroed_block_fails(M, N, K, dtype):
    A, B = make_ab(M, N, K, dtype)
    want = O.shard_gemm(A, B, dtype)
    got = want.clone()
    i, j = a_block(M, N)
    got[16 * i:16 * i + 16, 16 * j:16 * j + 16] = 0
    with pytest.raises(AssertionError):
        check_close(got, want, "zeroed block")


@pytest.mark.parametrize("M,N,K,dtype", SHAPES)
def test_two_rows_swapped_inside_a_block_fail(M, N, K, dtype):
    if M < 2:
        pytest.skip("one row")
    A, B = make_ab(M, N, K, dtype)
    want = O.shard_gemm(A, B, dtype)
    got = want.clone()
    i, j = a_block(M, N)
    r0 = 16 * i
    r1 = min(r0 + 5, M - 1)
    cols = slice(16 * j, 16 * j + 16)
    got[r0, cols], got[r1, cols] = want[r1, cols].clone(), want[r0, cols].clone()
    with pytest.raises(AssertionError):
        check_close(got, want, "swapped rows")


def test_the_element_wise_tolerance_alone_is_blind_at_small_scale():
    """Why the second check exists: with the old operand scale an all-zero
    result of the K = 64 case passes the element-wise tolerance almost
    everywhere; the per-block bound rejects every block."""
    A, B = make_ab(256, 256, 64, torch.bfloat16, scale=0.02)
    want = O.shard_gemm(A, B, torch.bfloat16).float()
    got = torch.zeros_like(want)
    bad = ~torch.isclose(got, want, rtol=RTOL, atol=ATOL)
    assert int(bad.sum()) < want.numel() // 100
    assert not bool(blocks_ok(got, want).any())


def test_edges_and_empty_blocks():
    # ragged edges are padded with zeros on both sides; an all-zero expectation passes only with an all-zero result
    want = torch.zeros(20, 35)
    check_close(torch.zeros(20, 35), want)
    got = want.clone()
    got[19, 34] = 1e-3
    with pytest.raises(AssertionError):
        check_close(got, want, "stray value past the last full block")
    check_close(torch.zeros(0, 8), torch.zeros(0, 8))
