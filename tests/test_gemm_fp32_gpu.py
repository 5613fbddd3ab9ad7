"""fp32 operands (the reference scripts' ``--datatype fp32``,
examples/09_gemm_one_shot_all_reduce/benchmark.py:41-46,84-96): the shard GEMM
and its three epilogues against the CPU oracle, through the C-ABI.

The kernels multiply fp32 by fp32 and accumulate in fp32
(``v_mfma_f32_16x16x4_f32``), so beside the mandated rtol 1e-2 / atol 1e-2 the
results must agree with the oracle's fp32 product to summation order: every
16 x 16 block within 1e-4 of its norm.  Flags and the reduce: bit-exact.
"""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O
from parity import check_close, make_ab
from test_gemm_gpu import to_heap

pytestmark = pytest.mark.gpu

F32 = torch.float32
TIGHT = 1e-4

CASES = [
    # M, N, K, BLK_M, BLK_N, G, grid, plan the launch must take
    (256, 256, 64, 256, 256, 4, 4, "128x128x32_w2x2_s4_f4_fp32"),
    (512, 768, 256, 256, 256, 4, 256, "128x128x32_w2x2_s4_f4_fp32"),
    (1024, 512, 128, 256, 128, 6, 16, "128x128x32_w2x2_s4_f4_fp32"),
    (640, 384, 96, 128, 128, 3, 32, "128x128x32_w2x2_s4_f4_fp32"),
    (768, 320, 160, 256, 64, 4, 256, "64x64x32_w2x2_s4_fp32"),
    (320, 192, 64, 64, 64, 1, 7, "64x64x32_w2x2_s4_fp32"),
    (300, 200, 72, 256, 256, 4, 8, "128x128x32_w2x2_s4_f4_fp32"),   # ragged M, N; K tail of 8
    (300, 200, 36, 128, 64, 4, 8, "64x64x32_w2x2_s4_fp32"),         # K tail of 4 elements (one 16-byte chunk)
    (300, 200, 70, 128, 64, 4, 8, "64x64x16_w2x2_generic_fp32"),    # K not a multiple of 4: the element-wise loader
    (1, 1376, 256, 256, 256, 4, 256, None),                         # one token
    (16, 1376, 512, 256, 64, 4, 256, None),
    (96, 80, 40, 32, 32, 2, 5, "64x64x16_w2x2_generic_fp32"),       # logical tile smaller than any compute tile
    (200, 136, 264, 96, 72, 2, 8, "64x64x16_w2x2_generic_fp32"),    # logical tile no compute tile divides
]


@pytest.mark.parametrize("M,N,K,BM,BN,G,grid,plan", CASES)
def test_all_scatter_single_rank_fp32(shmem, M, N, K, BM, BN, G, grid, plan):
    A, B = make_ab(M, N, K, F32)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.full((M, N), 7, dtype=F32)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 3,), dtype=torch.int32)
    args = (a, b, None, cg, flags, shmem.get_heap_bases(), 0, 1, grid, BM, BN, 64, G, ops.EPI_ALL_SCATTER)
    kw = dict(num_xcds=ops.default_num_xcds(256, grid))
    if plan is not None:
        assert ops.gemm_plan_name(*args, **kw) == plan
    ops.gemm_launch(*args, **kw)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, F32), "all_scatter fp32", block_rtol=TIGHT)
    assert flags.cpu().tolist() == [1] * total + [0, 0, 0]


def test_every_fp32_variant_and_a_row_major_b(shmem):
    """Each entry of the fp32 table forced by its number, and B given
    N-contiguous (not the scripts' layout), which only the element-wise loader
    takes."""
    M, N, K = 384, 256, 192
    A, B = make_ab(M, N, K, F32)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    want = O.shard_gemm(A, B, F32)
    names = []
    for variant in range(1, 5):
        cg = shmem.zeros((M, N), dtype=F32)
        flags = shmem.zeros((6,), dtype=torch.int32)
        args = (a, b, None, cg, flags, None, 0, 1, 6, 128, 128, 64, 2, ops.EPI_ALL_SCATTER)
        names.append(ops.gemm_plan_name(*args, variant=variant))
        ops.gemm_launch(*args, variant=variant)
        torch.cuda.synchronize()
        check_close(cg, want, names[-1], block_rtol=TIGHT)
        assert flags.cpu().tolist() == [1] * 6
    assert names == ["128x128x32_w2x2_s4_f4_fp32", "128x128x32_w2x2_s4_fp32", "64x64x32_w2x2_s4_fp32",
                     "64x64x16_w2x2_generic_fp32"]
    with pytest.raises(ValueError):
        ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 6, 128, 128, 64, 2, ops.EPI_ALL_SCATTER, variant=5)
    b_rows = shmem.zeros((K, N), dtype=F32)
    b_rows.copy_(B)
    assert b_rows.stride() == (N, 1)
    cg = shmem.zeros((M, N), dtype=F32)
    args = (a, b_rows, None, cg, flags, None, 0, 1, 6, 128, 128, 64, 2, ops.EPI_ALL_SCATTER)
    assert ops.gemm_plan_name(*args) == "64x64x16_w2x2_generic_fp32"
    ops.gemm_launch(*args)
    torch.cuda.synchronize()
    check_close(cg, want, "row-major B", block_rtol=TIGHT)


def test_fp32_operands_need_an_fp32_output(shmem):
    A, B = make_ab(128, 128, 64, F32)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((128, 128), dtype=torch.bfloat16)
    flags = shmem.zeros((1,), dtype=torch.int32)
    with pytest.raises(ValueError):
        ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 4, 128, 128, 64, 2, ops.EPI_ALL_SCATTER)
    # no split-K build of the fp32 tiles: a forced split is refused, the launcher's own choice is "none"
    cg32 = shmem.zeros((128, 128), dtype=F32)
    partials = shmem.zeros((256, 128 * 128), dtype=F32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    with pytest.raises(ValueError):
        ops.gemm_launch(a, b, None, cg32, flags, None, 0, 1, 256, 128, 128, 64, 2, ops.EPI_ALL_SCATTER,
                        partials=partials, locks=locks, split_k=2)
    assert ops.gemm_split_k(a, b, None, cg32, flags, None, 0, 1, 256, 128, 128, 64, 2, ops.EPI_ALL_SCATTER,
                            partials=partials, locks=locks) == 1


@pytest.mark.parametrize("ws", [2, 4])
def test_all_scatter_virtual_ranks_fp32(shmem, ws):
    M, N, K, BM, BN, G = 256, 128 * ws, 128, 128, 64, 4
    A, B = make_ab(M, N, K, F32)
    shards = O.n_shards(A, B, ws)
    a = to_heap(shmem, A)
    bs = [to_heap(shmem, sb) for _, sb in shards]
    cg = shmem.zeros((M, N), dtype=F32)
    n_local = N // ws
    total = ops.cdiv(M, BM) * ops.cdiv(n_local, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    for r in range(ws):
        shmem.on_rank(cg, r).zero_()
        shmem.on_rank(flags, r).zero_()
    for r in range(ws):
        ops.gemm_launch(a, bs[r], None, shmem.on_rank(cg, r), shmem.on_rank(flags, r), shmem.get_heap_bases(), r,
                        ws, 16, BM, BN, 64, G, ops.EPI_ALL_SCATTER)
    torch.cuda.synchronize()
    want = O.all_scatter(shards, F32)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}", block_rtol=TIGHT)
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws] * total


def test_atomics_all_reduce_virtual_ranks_fp32(shmem):
    """K-split over 4 ranks, every rank adds its partial tiles into every
    rank's fp32 C (gemm_atomics_all_reduce.py:206-248)."""
    ws, M, N, K = 4, 256, 192, 512
    A, B = make_ab(M, N, K, F32)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    ks = K // ws
    cg = shmem.zeros((M, N), dtype=F32)
    for r in range(ws):
        shmem.on_rank(cg, r).zero_()
    for r in range(ws):
        ops.gemm_launch(a_full[:, r * ks:(r + 1) * ks], b_full[r * ks:(r + 1) * ks, :], None, shmem.on_rank(cg, r),
                        None, shmem.get_heap_bases(), r, ws, 8, 128, 64, 64, 4, ops.EPI_ATOMIC_ADD)
    torch.cuda.synchronize()
    want = O.atomics_all_reduce(O.k_shards(A, B, ws))
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}", block_rtol=TIGHT)


@pytest.mark.parametrize("phase", [ops.PHASE_FUSED, ops.PHASE_TWO_KERNELS])
def test_one_shot_single_rank_fp32(shmem, phase):
    M, N, K = 384, 320, 192
    A, B = make_ab(M, N, K, F32)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    c = shmem.zeros((M, N), dtype=F32)
    cg = shmem.zeros((M, N), dtype=F32)
    total = ops.cdiv(M, 128) * ops.cdiv(N, 64)
    flags = shmem.zeros((total,), dtype=torch.int32)
    ops.gemm_launch(a, b, c, cg, flags, shmem.get_heap_bases(), 0, 1, 8, 128, 64, 64, 6, ops.EPI_ONE_SHOT, phase=phase)
    torch.cuda.synchronize()
    check_close(c, O.shard_gemm(A, B, F32), "partial", block_rtol=TIGHT)
    assert torch.equal(cg.cpu(), O.one_shot_reduce(c.cpu()[None], F32))
    assert flags.cpu().tolist() == [0] * total


def test_one_shot_all_reduce_virtual_ranks_fp32(shmem):
    """K-split over 4 ranks: every rank produces (partial tile + signal), then
    every rank consumes (wait, reduce in rank order, store); the reduce is
    bit-exact given the partials."""
    ws, M, N, BM, BN, G = 4, 256, 320, 128, 64, 6
    K = 64 * ws
    A, B = make_ab(M, N, K, F32)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    ks = K // ws
    c = shmem.zeros((M, N), dtype=F32)
    cg = shmem.zeros((M, N), dtype=F32)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    for r in range(ws):
        for t in (c, cg, flags):
            shmem.on_rank(t, r).zero_()
    hb = shmem.get_heap_bases()

    def launch(r, phase):
        ops.gemm_launch(a_full[:, r * ks:(r + 1) * ks], b_full[r * ks:(r + 1) * ks, :], shmem.on_rank(c, r),
                        shmem.on_rank(cg, r), shmem.on_rank(flags, r), hb, r, ws, 8, BM, BN, 64, G,
                        ops.EPI_ONE_SHOT, phase=phase, status=status)

    for r in range(ws):
        launch(r, ops.PHASE_PRODUCE)
    torch.cuda.synchronize()
    for r in range(ws):
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total
    partials = torch.stack([shmem.on_rank(c, r).cpu() for r in range(ws)])
    shards = O.k_shards(A, B, ws)
    for r in range(ws):
        check_close(partials[r], O.shard_gemm(*shards[r], F32), f"partial {r}", block_rtol=TIGHT)
    for r in range(ws):
        launch(r, ops.PHASE_CONSUME)
    torch.cuda.synchronize()
    want_bits = O.one_shot_reduce(partials, F32)
    for r in range(ws):
        assert torch.equal(shmem.on_rank(cg, r).cpu(), want_bits), f"rank {r}"
        assert shmem.on_rank(flags, r).cpu().tolist() == [0] * total
    assert int(status.item()) == 0
    check_close(want_bits, O.one_shot_all_reduce(shards, F32, F32), "against the full product", block_rtol=TIGHT)


def test_a_larger_fp32_launch_and_its_rate(shmem):
    """[2048, 1024] x [1024, 2048] in the scripts' 256 x 256 tiles on every CU:
    sampled rows against the oracle (the whole product would take the CPU
    seconds), every flag."""
    M = N = 2048
    K = 1024
    A, B = make_ab(M, N, K, F32)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=F32)
    flags = shmem.zeros((64,), dtype=torch.int32)
    ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 256, 256, 256, 64, 4, ops.EPI_ALL_SCATTER, num_xcds=8)
    torch.cuda.synchronize()
    rows = torch.arange(0, M, 37)
    check_close(cg.cpu()[rows], O.shard_gemm(A[rows], B, F32), "sampled rows", block_rtol=TIGHT)
    assert flags.cpu().tolist() == [1] * 64
