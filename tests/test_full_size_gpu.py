"""Parity at the sizes the headline figures are quoted on: the bf16
[8192,1024] x [1024,8192] K-shard GEMM with flag-published 256x256 tiles, and
the one-shot reduce of eight fp32 [8192,8192] partials.

The full fp32 product is too much for the CPU oracle inside a test, so the
GEMM is checked against the oracle on sampled rows and columns (every tile is
crossed by some of them), against a column-sum identity over the whole
matrix, and flag for flag.  The reduce is compared with the oracle bit for
bit over the whole matrix.
"""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O
from test_gemm_gpu import check_close
from test_reduce_gpu import signal_all

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("G", [4, 6])
def test_headline_shard_gemm(shmem, G):
    M = N = 8192
    K, KT, BM, BN = 1024, 8192, 256, 256
    dtype = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(123)
    a_full = shmem.zeros((M, KT), dtype=dtype)
    bt_full = shmem.zeros((N, KT), dtype=dtype)
    a_full.copy_((torch.randn(M, KT, generator=gen, device="cuda") * 0.02).to(dtype))
    bt_full.copy_((torch.randn(N, KT, generator=gen, device="cuda") * 0.02).to(dtype))
    shard = 3  # K-shard views with the full-K leading dimension (benchmark.py:112-118)
    a, b = a_full[:, shard * K:(shard + 1) * K], bt_full[:, shard * K:(shard + 1) * K].T
    assert a.stride() == (KT, 1) and b.stride() == (1, KT)
    cg = shmem.full((M, N), 7, dtype=dtype)
    total = (M // BM) * (N // BN)
    flags = shmem.zeros((total + 1,), dtype=torch.int32)
    ops.gemm_launch(a, b, None, cg, flags, shmem.get_heap_bases(), 0, 1, 256, BM, BN, 64, G, ops.EPI_ALL_SCATTER,
                    num_xcds=8)
    torch.cuda.synchronize()
    assert flags.cpu().tolist() == [1] * total + [0]

    # the oracle on 3 rows and 3 columns of every tile row / tile column
    A, B = a.cpu(), b.cpu()
    g = torch.Generator().manual_seed(7)
    rows = torch.cat([torch.randint(0, BM, (3,), generator=g) + t * BM for t in range(M // BM)])
    cols = torch.cat([torch.randint(0, BN, (3,), generator=g) + t * BN for t in range(N // BN)])
    check_close(cg[rows].cpu(), O.shard_gemm(A[rows], B, dtype), "sampled rows")
    check_close(cg[:, cols].cpu(), O.shard_gemm(A, B[:, cols], dtype), "sampled columns")

    # whole matrix: 1^T C == (1^T A) B up to the rounding of C's 8192 addends per column
    colsum = cg.float().sum(dim=0).cpu()
    want = (A.float().sum(dim=0, keepdim=True) @ B.float()).squeeze(0)
    bound = 8192 ** 0.5 * 2.0 ** -9 * cg.float().abs().max().item() * 6  # 6 sigma of independent bf16 roundings
    assert (colsum - want).abs().max().item() < bound


def test_headline_reduce_of_eight_partials_is_bit_exact(shmem):
    M = N = 8192
    BM = BN = 256
    ws = 8
    c = shmem.zeros((M, N), dtype=torch.float32)
    cg = shmem.zeros((M, N), dtype=torch.bfloat16)
    total = (M // BM) * (N // BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    gen = torch.Generator(device="cuda").manual_seed(321)
    for r in range(ws):
        shmem.on_rank(c, r).copy_(torch.randn(M, N, generator=gen, device="cuda"))
    signal_all(shmem, flags, total, ws)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.one_shot_reduce(c, cg, flags, shmem.get_heap_bases(), 0, ws, BM, BN, 6, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert flags.cpu().tolist() == [0] * total
    # the oracle's loop, one partial at a time (2 GiB of partials never sit on the host together)
    acc = torch.zeros((M, N), dtype=torch.float32)
    for r in range(ws):
        acc = O.one_shot_reduce(torch.stack([acc, shmem.on_rank(c, r).cpu()]), torch.float32)
    assert torch.equal(cg.cpu(), acc.to(torch.bfloat16))
