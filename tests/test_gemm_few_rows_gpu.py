"""Parity of the few-rows shard GEMM (at most 32 rows of A, one workgroup per
16 rows x 16 columns of C) against the CPU oracle, through the C-ABI.

Same bar as the persistent kernel: values rtol 1e-2 / atol 1e-2 against the
fp32-accumulated oracle, flags and arrival counters bit-exact.
"""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O
from test_gemm_gpu import check_close, make_ab, to_heap

pytestmark = pytest.mark.gpu

FEW = "few_rows_16xN"


def scatter(shmem, a, b, cg, flags, rank, ws, BM, BN, G, *, locks=None, variant=0, notify=True, grid=256,
            scope=ops.SCOPE_AGENT):
    args = (a, b, None, cg, flags, shmem.get_heap_bases(), rank, ws, grid, BM, BN, 64, G, ops.EPI_ALL_SCATTER)
    name = ops.gemm_plan_name(*args, notify=notify, locks=locks, partials=None, variant=variant)
    ops.gemm_launch(*args, notify=notify, locks=locks, variant=variant, scope=scope)
    return name


CASES = [
    # M, N, K, BLK_M, BLK_N, G, dtype
    (1, 1376, 4096, 256, 256, 4, torch.bfloat16),   # decoder gate/up, one token
    (16, 1376, 4096, 64, 64, 4, torch.bfloat16),
    (16, 4096, 1376, 128, 128, 6, torch.bfloat16),  # decoder down: 21 K blocks and a tail of 32
    (3, 40, 72, 16, 16, 1, torch.bfloat16),         # one workgroup per logical tile; ragged last block; K tail of 8
    (7, 50, 8, 64, 32, 2, torch.float16),           # N not a multiple of 4: element-wise stores; a single 8-k chunk
    (16, 16, 64, 16, 16, 1, torch.float16),
    (5, 272, 9000, 32, 48, 3, torch.bfloat16),      # K range that takes a wave two rounds of fetches
    (12, 2048, 640, 256, 128, 4, torch.float16),
    (17, 1376, 4096, 64, 64, 4, torch.bfloat16),    # two blocks of rows, the second with one row
    (32, 4096, 1376, 32, 128, 6, torch.bfloat16),
    (20, 50, 72, 32, 16, 2, torch.float16),         # one block of columns per flag, two of rows
    # (from five rows and K = 2048 on, A is fetched along its rows and passed through LDS)
    (9, 200, 2120, 64, 64, 2, torch.float16),       # ... with a K tail of 8 and a ragged last block of columns
    (32, 512, 2048, 32, 64, 2, torch.bfloat16),     # ... two blocks of rows
    (4, 1376, 4096, 64, 64, 4, torch.bfloat16),     # (four rows: still fetched in operand layout)
]


@pytest.mark.parametrize("M,N,K,BM,BN,G,dtype", CASES)
def test_scatter_single_rank(shmem, M, N, K, BM, BN, G, dtype):
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.full((M, N), 7, dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 3,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    for launch in (1, 2):
        cg.fill_(7)
        assert scatter(shmem, a, b, cg, flags, 0, 1, BM, BN, G, locks=locks) == FEW
        torch.cuda.synchronize()
        check_close(cg, O.shard_gemm(A, B, dtype), f"launch {launch}")
        # one arrival per tile and launch; the arrival counters are back at zero
        assert flags.cpu().tolist() == [launch] * total + [0, 0, 0]
        assert not locks.any()


MID = "few_rows_32xN"
MID_CASES = [
    # M, N, K, BLK_M, BLK_N, G, dtype: 33 to 64 rows of a K of 2048 or more, one round of workgroups
    (64, 1376, 4096, 64, 64, 4, torch.bfloat16),    # decoder gate/up at 64 tokens: 2 x 86 workgroups
    (33, 1376, 4096, 256, 64, 4, torch.bfloat16),   # the second block of rows holds one row
    (48, 200, 2120, 64, 16, 2, torch.float16),      # K tail of 8, ragged last block of columns, a workgroup a flag
    (50, 272, 9000, 64, 48, 3, torch.bfloat16),     # K range that takes a wave two rounds of fetches
]


@pytest.mark.parametrize("M,N,K,BM,BN,G,dtype", MID_CASES)
def test_scatter_33_to_64_rows(shmem, M, N, K, BM, BN, G, dtype):
    """32 rows x 16 columns a workgroup: the same exchange, with two
    accumulator blocks a wave summed block by block before the stores."""
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.full((M, N), 7, dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 3,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    for launch in (1, 2):
        cg.fill_(7)
        assert scatter(shmem, a, b, cg, flags, 0, 1, BM, BN, G, locks=locks) == MID
        torch.cuda.synchronize()
        check_close(cg, O.shard_gemm(A, B, dtype), f"launch {launch}")
        assert flags.cpu().tolist() == [launch] * total + [0, 0, 0]
        assert not locks.any()


def test_33_to_64_rows_other_epilogues_and_the_launcher_choice(shmem):
    """fp32 partial with the one-shot signal on 4 virtual ranks, atomic add; and
    when the launch stays with the persistent kernels."""
    ws, M, N, K, dtype = 4, 40, 384, 4 * 2048, torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    shards = O.k_shards(A, B, ws)
    ah, bh = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    part = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(N, 128)
    flags = shmem.zeros((total,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        for t in (part, out, flags, locks):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], shmem.on_rank(part, r), shmem.on_rank(out, r),
                shmem.on_rank(flags, r), hb, r, ws, 256, 64, 128, 64, 6, ops.EPI_ONE_SHOT)
        kw = dict(phase=ops.PHASE_PRODUCE, locks=shmem.on_rank(locks, r))
        assert ops.gemm_plan_name(*args, **kw) == MID
        ops.gemm_launch(*args, **kw)
    torch.cuda.synchronize()
    for r in range(ws):
        check_close(shmem.on_rank(part, r), O.shard_gemm(*shards[r], torch.float32), f"partial {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total
        assert not shmem.on_rank(locks, r).any()
    # atomic accumulate of the four K shards into one fp32 C
    c32 = shmem.zeros((M, N), dtype=torch.float32)
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], None, c32, None, None, 0, 1, 256, 64, 128, 64, 6,
                ops.EPI_ATOMIC_ADD)
        assert ops.gemm_plan_name(*args) == MID
        ops.gemm_launch(*args)
    torch.cuda.synchronize()
    check_close(c32, O.atomics_all_reduce(shards))
    # the persistent kernels keep: a short K, more rows, a logical tile that does not cover the rows, more
    # workgroups than CUs, the caller's insistence
    a1 = ah[:, :kk]
    b1 = bh[:kk, :]
    cg = shmem.zeros((M, N), dtype=dtype)
    many_flags = shmem.zeros((1024,), dtype=torch.int32)

    def plan(a_, b_, cg_, BM, BN, **kw):
        return ops.gemm_plan_name(a_, b_, None, cg_, many_flags, None, 0, 1, 256, BM, BN, 64, 4, ops.EPI_ALL_SCATTER,
                                  locks=locks, **kw)

    assert plan(a1, b1, cg, 64, 128) == MID
    assert plan(a1[:, :1024], b1[:1024, :], cg, 64, 128) != MID
    assert plan(a1, b1, cg, 32, 128) != MID
    assert plan(a1, b1, cg, 64, 128, variant=ops.VARIANT_PERSISTENT) != MID
    A2, B2 = make_ab(65, 4096, 2048, dtype)
    a2, b2 = to_heap(shmem, A2), to_heap(shmem, B2)
    cg2 = shmem.zeros((65, 4096), dtype=dtype)
    assert plan(a2, b2, cg2, 128, 128) != MID                    # more than 64 rows
    assert plan(a2[:64], b2, cg2[:64], 64, 128) != MID            # 2 x 256 workgroups: more than one round


def test_strided_operands_and_output(shmem):
    """K-shard views (leading dimensions > K) and an output that is a column
    block of a wider matrix."""
    M, N, K, dtype = 9, 96, 320, torch.bfloat16
    A, B = make_ab(M, N, K, dtype, lda=1024, ldb=2048)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    wide = shmem.full((M, 3 * N), 5, dtype=dtype)
    cg = wide[:, N:2 * N]
    flags = shmem.zeros((2,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    assert scatter(shmem, a, b, cg, flags, 0, 1, 64, 64, 4, locks=locks) == FEW
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype))
    assert (wide[:, :N] == 5).all() and (wide[:, 2 * N:] == 5).all()
    assert flags.cpu().tolist() == [1, 1]


@pytest.mark.parametrize("ws,scope", [(2, ops.SCOPE_AGENT), (8, ops.SCOPE_AGENT), (3, ops.SCOPE_SYSTEM)])
def test_scatter_virtual_ranks(shmem, ws, scope):
    """Rank r's [M, N/ws] block lands at column r*N/ws of c_global on every
    rank (wave w of a workgroup stores on rank w); every rank's flags count ws
    arrivals."""
    M, K, BM, BN, G, dtype = (16 if ws != 2 else 27), 512, 64, 64, 4, torch.bfloat16
    N = 176 * ws
    A, B = make_ab(M, N, K, dtype)
    shards = O.n_shards(A, B, ws)
    a = to_heap(shmem, A)
    bs = [to_heap(shmem, sb) for _, sb in shards]
    cg = shmem.zeros((M, N), dtype=dtype)
    n_local = N // ws
    total = ops.cdiv(n_local, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    for r in range(ws):
        for t in (cg, flags, locks):  # (zeros() clears rank 0's copy only)
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        assert scatter(shmem, a, bs[r], shmem.on_rank(cg, r), shmem.on_rank(flags, r), r, ws, BM, BN, G,
                       locks=shmem.on_rank(locks, r), scope=scope) == FEW
    torch.cuda.synchronize()
    want = O.all_scatter(shards, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws] * total
        assert not shmem.on_rank(locks, r).any()


@pytest.mark.parametrize("pdtype", [torch.float32, torch.bfloat16])
def test_one_shot_producer_and_reduce(shmem, pdtype):
    """K-split over 4 ranks: each rank's partial through the few-rows kernel,
    +1 on every other rank's flag per tile, then the reduce kernel."""
    ws, M, N, K, BM, BN, G, dtype = 4, 16, 384, 4 * 256, 32, 128, 6, torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    shards = O.k_shards(A, B, ws)
    ah, bh = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    part = shmem.zeros((M, N), dtype=pdtype)
    out = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        for t in (part, out, flags, locks):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], shmem.on_rank(part, r), shmem.on_rank(out, r),
                shmem.on_rank(flags, r), hb, r, ws, 256, BM, BN, 64, G, ops.EPI_ONE_SHOT)
        kw = dict(phase=ops.PHASE_PRODUCE, locks=shmem.on_rank(locks, r))
        assert ops.gemm_plan_name(*args, **kw) == FEW
        ops.gemm_launch(*args, **kw)
    torch.cuda.synchronize()
    for r in range(ws):
        check_close(shmem.on_rank(part, r), O.shard_gemm(*shards[r], pdtype), f"partial {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total  # every other rank arrived once
    for r in range(ws):
        ops.one_shot_reduce(shmem.on_rank(part, r), shmem.on_rank(out, r), shmem.on_rank(flags, r), hb, r, ws, BM,
                            BN, G)
    torch.cuda.synchronize()
    want = O.one_shot_all_reduce(shards, pdtype, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(out, r), want, f"reduced on rank {r}")
        assert not shmem.on_rank(flags, r).any()


@pytest.mark.parametrize("phase", [ops.PHASE_TWO_KERNELS, ops.PHASE_FUSED])
@pytest.mark.parametrize("ws", [1, 4])
def test_one_shot_fused_phase(shmem, ws, phase):
    """PHASE_TWO_KERNELS: the few-rows producer and the reduce kernel behind it
    on the same stream.  PHASE_FUSED reduces inside the program, which the
    persistent kernels do: the launch stays with them.  With one GPU playing
    every rank the other ranks' partials and signals are put in place first,
    then the last rank runs both phases."""
    M, N, BM, BN, G, dtype = 9, 272, 16, 64, 3, torch.bfloat16
    K = 192 * ws
    A, B = make_ab(M, N, K, dtype)
    shards = O.k_shards(A, B, ws)
    ah, bh = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    part = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        for t in (part, out, flags, locks):
            shmem.on_rank(t, r).zero_()
    last = ws - 1
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], shmem.on_rank(part, r), shmem.on_rank(out, r),
                shmem.on_rank(flags, r), hb, r, ws, 256, BM, BN, 64, G, ops.EPI_ONE_SHOT)
        kw = dict(phase=phase if r == last else ops.PHASE_PRODUCE, locks=shmem.on_rank(locks, r))
        if r == last and phase == ops.PHASE_FUSED:
            assert ops.gemm_plan_name(*args, **kw).endswith("+reduce")
        else:
            assert ops.gemm_plan_name(*args, **kw) == FEW
        ops.gemm_launch(*args, **kw)
    torch.cuda.synchronize()
    check_close(shmem.on_rank(out, last), O.one_shot_all_reduce(shards, torch.float32, dtype), "fused result")
    assert not shmem.on_rank(flags, last).any()  # consumed


@pytest.mark.parametrize("M,out_dtype", [(16, torch.float32), (24, torch.float32), (7, torch.bfloat16),
                                         (32, torch.bfloat16)])
def test_atomic_accumulate_of_k_shards(shmem, M, out_dtype):
    """08 epilogue: every rank adds its K-shard product into every rank's C."""
    ws, N, K, BM, BN, dtype = 4, 208, 4 * 320, 32, 64, torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    shards = O.k_shards(A, B, ws)
    ah, bh = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    c = shmem.zeros((M, N), dtype=out_dtype)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        shmem.on_rank(c, r).zero_()
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], None, shmem.on_rank(c, r), None, hb, r, ws, 256,
                BM, BN, 64, 4, ops.EPI_ATOMIC_ADD)
        assert ops.gemm_plan_name(*args) == FEW
        ops.gemm_launch(*args)
    torch.cuda.synchronize()
    want = O.atomics_all_reduce(shards)
    for r in range(ws):
        got = shmem.on_rank(c, r).float().cpu()
        if out_dtype == torch.float32:
            check_close(got, want, f"rank {r}")
        else:  # 16-bit accumulation rounds after every add: 4 roundings of half an ulp each
            assert float((got - want).abs().max()) <= 4 * 2.0 ** -8 * float(want.abs().max()) + 1e-2, f"rank {r}"


def test_choice_of_kernel(shmem):
    dtype = torch.bfloat16
    A, B = make_ab(16, 256, 128, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((16, 256), dtype=dtype)
    flags = shmem.zeros((64,), dtype=torch.int32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    hb = shmem.get_heap_bases()

    def plan(a_, b_, cg_, BM, BN, **kw):
        return ops.gemm_plan_name(a_, b_, None, cg_, flags, hb, 0, 1, 256, BM, BN, 64, 4, ops.EPI_ALL_SCATTER, **kw)

    assert plan(a, b, cg, 64, 64, locks=locks) == FEW
    assert plan(a, b, cg, 64, 64, locks=locks, variant=ops.VARIANT_FEW_ROWS) == FEW
    # several workgroups per flag and nowhere to count their arrivals
    assert plan(a, b, cg, 64, 64) != FEW
    # ... unless nothing is published, or a flag belongs to one workgroup
    assert plan(a, b, cg, 64, 64, notify=False) == FEW
    assert plan(a, b, cg, 16, 16) == FEW
    # the persistent kernels on request
    assert plan(a, b, cg, 64, 64, locks=locks, variant=ops.VARIANT_PERSISTENT) == "64x64x128_w2x2_s4_f4"
    names = {}
    v = 1
    while (name := ops.gemm_variant_name(dtype, False, False, v)) is not None:
        names[name] = v
        v += 1
    for name in ("64x64x128_w2x2_s4_f4", "64x64x64_w2x2_s4"):
        assert plan(a, b, cg, 64, 64, locks=locks, variant=names[name]) == name
    # a logical tile that does not cover the rows, or is no multiple of 16 columns
    assert plan(a, b, cg, 8, 64, locks=locks) != FEW
    assert plan(a, b, cg, 64, 40, locks=locks) != FEW
    # up to 32 rows in blocks of 16; no more
    A1, _ = make_ab(32, 256, 128, dtype)
    assert plan(to_heap(shmem, A1), b, shmem.zeros((32, 256), dtype=dtype), 64, 64, locks=locks) == FEW
    assert plan(to_heap(shmem, A1), b, shmem.zeros((32, 256), dtype=dtype), 32, 16) != FEW  # two workgroups a flag
    A2, B2 = make_ab(33, 256, 128, dtype)
    a2, cg2 = to_heap(shmem, A2), shmem.zeros((33, 256), dtype=dtype)
    assert plan(a2, b, cg2, 64, 64, locks=locks) != FEW
    with pytest.raises(ValueError):
        plan(a2, b, cg2, 64, 64, locks=locks, variant=ops.VARIANT_FEW_ROWS)
    # B with N contiguous: no 16-byte fetches along K
    bn = shmem.zeros((128, 256), dtype=dtype)
    assert plan(a, bn, cg, 64, 64, locks=locks) != FEW
    # the atomic epilogue publishes nothing: no counters needed
    assert ops.gemm_plan_name(a, b, None, cg, flags, hb, 0, 1, 256, 64, 64, 64, 4, ops.EPI_ATOMIC_ADD) == FEW


def test_persistent_choice_gives_the_same_result(shmem):
    """The two kernels on one input: same values to the parity tolerance, same flags."""
    M, N, K, dtype = 16, 1376, 1024, torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    locks = shmem.zeros((256,), dtype=torch.int32)
    got = {}
    for variant in (0, ops.VARIANT_PERSISTENT):
        cg = shmem.zeros((M, N), dtype=dtype)
        flags = shmem.zeros((ops.cdiv(N, 128),), dtype=torch.int32)
        name = scatter(shmem, a, b, cg, flags, 0, 1, 128, 128, 4, locks=locks, variant=variant)
        torch.cuda.synchronize()
        got[variant] = (name, cg, flags.cpu().tolist())
    assert got[0][0] == FEW and got[ops.VARIANT_PERSISTENT][0] != FEW
    check_close(got[0][1], got[ops.VARIANT_PERSISTENT][1])
    assert got[0][2] == got[ops.VARIANT_PERSISTENT][2]
