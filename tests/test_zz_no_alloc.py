"""``iris_gemm_launch_noalloc``: the launch whose split-K / stream-K / few-rows
workspace is a device array inside the library.  Its output must equal, bit
for bit, what ``iris_gemm_launch`` gives with a caller-provided workspace (the
same kernels, the same plan, the same order of fp32 additions), on two calls
in a row, the second with a smaller input (the array keeps the first call's
contents)."""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O

from test_gemm_gpu import check_close, make_ab, to_heap

pytestmark = pytest.mark.gpu


def run_pair(shmem, M, N, K, BM, BN, grid, dtype, split_k, expect_split):
    A, B = make_ab(M, N, K, dtype, seed=7 + M)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    partials = shmem.zeros((grid, BM * BN), dtype=torch.float32)
    locks = shmem.zeros((grid,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    args = lambda cg, flags: (a, b, None, cg, flags, hb, 0, 1, grid, BM, BN, 64, 2, ops.EPI_ALL_SCATTER)
    cg_ws, cg_na = shmem.zeros((M, N), dtype=dtype), shmem.zeros((M, N), dtype=dtype)
    f_ws, f_na = shmem.zeros((total,), dtype=torch.int32), shmem.zeros((total,), dtype=torch.int32)
    got = ops.gemm_split_k(*args(cg_ws, f_ws), partials=partials, locks=locks, split_k=split_k)
    assert got == expect_split, f"the plan under test: split {got}, expected {expect_split}"
    ops.gemm_launch(*args(cg_ws, f_ws), partials=partials, locks=locks, split_k=split_k)
    ops.gemm_launch(*args(cg_na, f_na), split_k=split_k, noalloc=True)
    torch.cuda.synchronize()
    check_close(cg_ws, O.shard_gemm(A, B, dtype), "workspace launch vs oracle")
    assert torch.equal(cg_na.cpu().view(torch.int16), cg_ws.cpu().view(torch.int16)), "no-alloc differs from the workspace launch"
    assert f_na.cpu().tolist() == f_ws.cpu().tolist() == [1] * total


def test_noalloc_allocates_nothing(shmem):
    """The property the entry point exists for: once the first call on the
    device has looked the library's array up, a call leaves the device's free
    memory and torch's allocator exactly as it found them."""
    dtype = torch.bfloat16
    A, B = make_ab(100, 200, 1024, dtype, seed=3)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((100, 200), dtype=dtype)
    flags = shmem.zeros((8,), dtype=torch.int32)
    hb = shmem.get_heap_bases()

    def call():
        ops.gemm_launch(a, b, None, cg, flags, hb, 0, 1, 256, 64, 64, 64, 2, ops.EPI_ALL_SCATTER, split_k=8,
                        noalloc=True)

    call()  # (the symbol lookup, and the kernels' code objects loaded)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    held0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, f"device memory in use changed by {free0 - free1} bytes"
    assert torch.cuda.memory_allocated() == held0 and torch.cuda.memory_reserved() == reserved0
    check_close(cg, O.shard_gemm(A, B, dtype))


def test_noalloc_matches_the_workspace_launch_twice(shmem):
    # split-K 8 on 64 x 64 tiles, then a smaller input with another split
    run_pair(shmem, 100, 200, 1024, 64, 64, 256, torch.bfloat16, 8, 8)
    run_pair(shmem, 40, 72, 512, 64, 64, 256, torch.bfloat16, 2, 2)
    # stream-K on 128 x 128 tiles (the largest slot), then a smaller one
    run_pair(shmem, 512, 768, 2048, 128, 128, 16, torch.bfloat16, ops.SPLIT_STREAM_K, ops.SPLIT_STREAM_K)
    run_pair(shmem, 128, 128, 512, 64, 64, 4, torch.float16, ops.SPLIT_STREAM_K, ops.SPLIT_STREAM_K)


def test_noalloc_last_round_split_matches_the_workspace_launch(shmem):
    # 18 tiles of 128 x 128 on 16 programs, K = 4096: 16 whole tiles, then the last two in two parts each,
    # as two launches; the second one's partials and locks live in the library's array
    dtype, M, N, K, grid = torch.bfloat16, 384, 768, 4096, 16
    A, B = make_ab(M, N, K, dtype, seed=11)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    partials = shmem.zeros((grid, 128 * 128), dtype=torch.float32)
    locks = shmem.zeros((grid,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    args = lambda cg, flags: (a, b, None, cg, flags, hb, 0, 1, grid, 128, 128, 64, 2, ops.EPI_ALL_SCATTER)
    for _ in range(2):
        cg_ws, cg_na = shmem.zeros((M, N), dtype=dtype), shmem.zeros((M, N), dtype=dtype)
        f_ws, f_na = shmem.zeros((18,), dtype=torch.int32), shmem.zeros((18,), dtype=torch.int32)
        assert ops.gemm_plan_name(*args(cg_ws, f_ws), partials=partials, locks=locks).endswith("+last_round_in_2_parts")
        ops.gemm_launch(*args(cg_ws, f_ws), partials=partials, locks=locks)
        ops.gemm_launch(*args(cg_na, f_na), noalloc=True)
        torch.cuda.synchronize()
        check_close(cg_ws, O.shard_gemm(A, B, dtype), "workspace launch vs oracle")
        assert torch.equal(cg_na.cpu().view(torch.int16), cg_ws.cpu().view(torch.int16))
        assert f_na.cpu().tolist() == f_ws.cpu().tolist() == [1] * 18 and int(locks.abs().max().item()) == 0


def test_noalloc_few_rows_counters_and_launcher_choice(shmem):
    # the few-rows kernel counts a tile's arrivals in the same array
    dtype = torch.bfloat16
    for M, N, K in ((16, 1376, 4096), (1, 512, 1376)):
        A, B = make_ab(M, N, K, dtype)
        a, b = to_heap(shmem, A), to_heap(shmem, B)
        total = ops.cdiv(N, 256)
        hb = shmem.get_heap_bases()
        locks = shmem.zeros((256,), dtype=torch.int32)
        cg_ws, cg_na = shmem.zeros((M, N), dtype=dtype), shmem.zeros((M, N), dtype=dtype)
        f_ws, f_na = shmem.zeros((total,), dtype=torch.int32), shmem.zeros((total,), dtype=torch.int32)
        common = lambda cg, f: (a, b, None, cg, f, hb, 0, 1, 256, 256, 256, 64, 4, ops.EPI_ALL_SCATTER)
        assert ops.gemm_plan_name(*common(cg_ws, f_ws), locks=locks) == "few_rows_16xN"
        ops.gemm_launch(*common(cg_ws, f_ws), locks=locks)
        ops.gemm_launch(*common(cg_na, f_na), noalloc=True)
        torch.cuda.synchronize()
        check_close(cg_ws, O.shard_gemm(A, B, dtype))
        assert torch.equal(cg_na.cpu().view(torch.int16), cg_ws.cpu().view(torch.int16))
        assert f_na.cpu().tolist() == f_ws.cpu().tolist() == [1] * total


def test_noalloc_limits_are_errors(shmem):
    dtype = torch.bfloat16
    A, B = make_ab(256, 256, 2048, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((256, 256), dtype=dtype)
    flags = shmem.zeros((16,), dtype=torch.int32)
    with pytest.raises(ValueError, match="at most 256 programs"):  # more programs than the array has slots
        ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 512, 64, 64, 64, 2, ops.EPI_ALL_SCATTER, noalloc=True)
    with pytest.raises(ValueError, match="forced split"):  # a forced split of a tile larger than a slot
        ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 256, 256, 256, 64, 2, ops.EPI_ALL_SCATTER, split_k=2,
                        noalloc=True)
    # the same checks inside the library, past the Python wrapper
    from iris_amd import _native
    import ctypes

    args = ops._fill_gemm_args(a, b, None, cg, flags, None, 0, 1, 256, 64, 64, 64, 2, ops.EPI_ALL_SCATTER,
                               ops.PHASE_FUSED, True, 1, ops.SCOPE_AGENT, 0, None, None, None, 0)
    args.num_sms = 512
    assert _native.lib().iris_gemm_launch_noalloc(ctypes.byref(args), None) == _native.HIP_ERROR_INVALID_VALUE
    args.num_sms, args.block_m, args.block_n, args.split_k = 256, 256, 256, 2
    assert _native.lib().iris_gemm_launch_noalloc(ctypes.byref(args), None) == _native.HIP_ERROR_INVALID_VALUE
    # stream-K forced on a tile larger than a slot: rejected like any forced split, in the wrapper and in the library
    with pytest.raises(ValueError, match="forced split"):
        ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 16, 256, 128, 64, 2, ops.EPI_ALL_SCATTER,
                        split_k=ops.SPLIT_STREAM_K, noalloc=True)
    args.num_sms, args.block_m, args.block_n, args.split_k = 16, 256, 128, ops.SPLIT_STREAM_K
    assert _native.lib().iris_gemm_launch_noalloc(ctypes.byref(args), None) == _native.HIP_ERROR_INVALID_VALUE
    # exactly as many programs as the array has slots is inside the limit
    cg64, f64 = shmem.zeros((256, 256), dtype=dtype), shmem.zeros((16,), dtype=torch.int32)
    ops.gemm_launch(a, b, None, cg64, f64, None, 0, 1, ops.NOALLOC_MAX_PROGRAMS, 64, 64, 64, 2, ops.EPI_ALL_SCATTER,
                    split_k=8, noalloc=True)
    torch.cuda.synchronize()
    check_close(cg64, O.shard_gemm(A, B, dtype), "256 programs, split 8")
    assert f64.cpu().tolist() == [1] * 16
    # without a forced split a large tile simply runs unsplit
    ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 256, 256, 256, 64, 2, ops.EPI_ALL_SCATTER, noalloc=True)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype))
