"""GEMM validation of the examples (examples/common/validation.py:7-23)."""

import torch


def validate_gemm(A, B, C, shmem, atol=1):
    """``allclose(C, A @ B, atol)`` at torch's default rtol; logs the first
    mismatch through ``shmem.log``."""
    expected = A @ B
    if torch.allclose(C, expected, atol=atol):
        return True
    shmem.log(f"Max absolute difference: {(C - expected).abs().max().item()}")
    bad = torch.nonzero(~torch.isclose(C, expected, atol=atol), as_tuple=False)
    if bad.numel():
        idx = tuple(bad[0].tolist())
        shmem.log(f"Mismatch at index {idx}: C={C[idx]}, expected={expected[idx]}")
    return False
