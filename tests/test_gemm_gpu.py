"""Parity of the HIP shard GEMM and its three epilogues against the CPU
oracle, through the C-ABI (``iris_amd.ops`` -> ``libiris_amd.so``).

Values: rtol 1e-2 / atol 1e-2 against the fp32-accumulated oracle (the K-block
order inside the matrix cores is not pinned by the reference).  Flags and
tile indices: bit-exact.
"""

import numpy as np
import pytest
import torch

from iris_amd import ops, testing
from oracle import iris_oracle as O
from parity import ATOL, RTOL, blocks_ok, check_close, make_ab  # noqa: F401  (re-exported to the other GPU test modules)

pytestmark = pytest.mark.gpu


def to_heap(shmem, t):
    """Copy a (possibly strided) host matrix into the heap, keeping its strides."""
    rows, cols = t.shape
    if t.stride(1) == 1:  # row-major view with leading dimension stride(0)
        buf = shmem.zeros((rows, t.stride(0)), dtype=t.dtype)
        buf[:, :cols].copy_(t)
        return buf[:, :cols]
    assert t.stride(0) == 1  # column-major view (B): store the transpose
    buf = shmem.zeros((cols, t.stride(1)), dtype=t.dtype)
    buf[:, :rows].copy_(t.T)
    return buf[:, :rows].T


SCATTER_CASES = [
    # M, N, K, BLK_M, BLK_N, G, grid, dtype
    (256, 256, 64, 256, 256, 4, 4, torch.bfloat16),
    (512, 768, 256, 256, 256, 4, 256, torch.bfloat16),
    (512, 768, 256, 256, 256, 6, 8, torch.float16),
    (1024, 512, 128, 256, 128, 6, 16, torch.bfloat16),
    (512, 1024, 128, 128, 256, 2, 24, torch.bfloat16),
    (640, 384, 96, 128, 128, 3, 32, torch.float16),
    (768, 320, 160, 256, 64, 4, 256, torch.bfloat16),
    (320, 192, 64, 64, 64, 1, 7, torch.bfloat16),
    (300, 200, 72, 256, 256, 4, 8, torch.bfloat16),     # ragged M, N; K not a multiple of 32
    (300, 200, 72, 128, 64, 4, 8, torch.float16),
    (1, 1376, 256, 256, 256, 4, 256, torch.bfloat16),   # decoder shapes: one token, ragged N
    (16, 1376, 512, 256, 64, 4, 256, torch.bfloat16),
    (128, 1376, 1376, 256, 256, 4, 256, torch.bfloat16),  # ragged K tail of 32
    (96, 80, 40, 32, 32, 2, 5, torch.bfloat16),         # logical tile smaller than any compute tile
    (200, 136, 264, 96, 72, 2, 8, torch.bfloat16),      # logical tile no compute tile divides
]


@pytest.mark.parametrize("M,N,K,BM,BN,G,grid,dtype", SCATTER_CASES)
def test_all_scatter_single_rank(shmem, M, N, K, BM, BN, G, grid, dtype):
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.full((M, N), 7, dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 3,), dtype=torch.int32)
    ops.gemm_launch(a, b, None, cg, flags, shmem.get_heap_bases(), 0, 1, grid, BM, BN, 64, G,
                    ops.EPI_ALL_SCATTER, num_xcds=ops.default_num_xcds(256, grid))
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype), "all_scatter")
    # one ready flag per tile, exactly one arrival each; nothing past the last tile
    assert flags.cpu().tolist() == [1] * total + [0, 0, 0]


def test_all_scatter_without_notify_leaves_flags_alone(shmem):
    A, B = make_ab(256, 256, 64, torch.bfloat16)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((256, 256), dtype=torch.bfloat16)
    flags = shmem.zeros((1,), dtype=torch.int32)
    ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 4, 256, 256, 64, 4, ops.EPI_ALL_SCATTER, notify=False)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, torch.bfloat16))
    assert flags.cpu().tolist() == [0]


@pytest.mark.parametrize("ws", [2, 8])
def test_all_scatter_virtual_ranks(shmem, ws):
    """N-split over ws ranks: rank r's [M, N/ws] block lands at column offset
    r*N/ws of c_global on *every* rank; each rank's flags count ws arrivals."""
    M, N, K, BM, BN, G = 256, 128 * ws, 128, 128, 64, 4
    dtype = torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    shards = O.n_shards(A, B, ws)
    a = to_heap(shmem, A)
    bs = [to_heap(shmem, sb) for _, sb in shards]
    cg = shmem.zeros((M, N), dtype=dtype)
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
    want = O.all_scatter(shards, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws] * total


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_k_shard_views_keep_full_k_leading_dimension(shmem, dtype):
    """The 08/09 sharding hands the kernel strided views of the full-K operands."""
    M, N, K, ws = 384, 256, 512, 4
    A, B = make_ab(M, N, K, dtype)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    ks = K // ws
    cg = shmem.zeros((M, N), dtype=dtype)
    flags = shmem.zeros((6,), dtype=torch.int32)
    for r in (0, 3):
        la, lb = a_full[:, r * ks:(r + 1) * ks], b_full[r * ks:(r + 1) * ks, :]
        assert la.stride() == (K, 1) and lb.stride() == (1, K)
        flags.zero_()
        ops.gemm_launch(la, lb, None, cg, flags, None, 0, 1, 6, 128, 128, 64, 2, ops.EPI_ALL_SCATTER)
        torch.cuda.synchronize()
        check_close(cg, O.shard_gemm(A[:, r * ks:(r + 1) * ks], B[r * ks:(r + 1) * ks, :], dtype), f"shard {r}")


def test_operands_the_dma_loader_cannot_take_use_the_generic_loader(shmem):
    dtype = torch.bfloat16
    # K not a multiple of 8
    A, B = make_ab(130, 70, 100, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((130, 70), dtype=dtype)
    ops.gemm_launch(a, b, None, cg, None, None, 0, 1, 4, 64, 64, 64, 2, ops.EPI_ALL_SCATTER, notify=False)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype), "K=100")
    # A stored column-major (stride_ak != 1) and B row-major (stride_bk != 1)
    g = torch.Generator().manual_seed(5)
    At = (torch.randn(64, 96, generator=g) * 0.05).to(dtype)   # [K, M] storage
    Bt = (torch.randn(64, 80, generator=g) * 0.05).to(dtype)   # [K, N] storage, row-major
    a2 = shmem.zeros((64, 96), dtype=dtype)
    a2.copy_(At)
    b2 = shmem.zeros((64, 80), dtype=dtype)
    b2.copy_(Bt)
    cg2 = shmem.zeros((96, 80), dtype=dtype)
    ops.gemm_launch(a2.T, b2, None, cg2, None, None, 0, 1, 4, 64, 64, 64, 2, ops.EPI_ALL_SCATTER, notify=False)
    torch.cuda.synchronize()
    check_close(cg2, O.shard_gemm(At.T, Bt, dtype), "transposed operands")
    # K == 0: the product is all zeros
    cg3 = shmem.full((96, 80), 3, dtype=dtype)
    ops.gemm_launch(a2.T[:, :0], b2[:0, :], None, cg3, None, None, 0, 1, 4, 64, 64, 64, 2, ops.EPI_ALL_SCATTER,
                    notify=False)
    torch.cuda.synchronize()
    assert float(cg3.float().abs().max()) == 0.0


def test_a_launch_without_rows_or_columns_is_a_no_op(shmem):
    """M == 0 or N == 0: nothing is launched, nothing is written, no flag moves (all three epilogues)."""
    dtype = torch.bfloat16
    A, B = make_ab(64, 64, 64, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.full((64, 64), 5, dtype=dtype)
    c = shmem.full((64, 64), 5, dtype=torch.float32)
    flags = shmem.zeros((4,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for av, bv in ((a[:0], b), (a, b[:, :0])):
        ops.gemm_launch(av, bv, None, cg, flags, hb, 0, 1, 4, 64, 64, 64, 1, ops.EPI_ALL_SCATTER)
        ops.gemm_launch(av, bv, None, cg, None, hb, 0, 1, 4, 64, 64, 64, 1, ops.EPI_ATOMIC_ADD)
        ops.gemm_launch(av, bv, c, cg, flags, hb, 0, 1, 4, 64, 64, 64, 1, ops.EPI_ONE_SHOT, phase=ops.PHASE_PRODUCE)
    torch.cuda.synchronize()
    assert float((cg.float() - 5).abs().max()) == 0.0 and float((c - 5).abs().max()) == 0.0
    assert flags.cpu().tolist() == [0] * 4


def test_unaligned_and_strided_output(shmem):
    dtype = torch.bfloat16
    A, B = make_ab(256, 192, 64, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    big = shmem.zeros((256, 200), dtype=dtype)
    cg = big[:, 3:195]  # column offset 3: rows are not 16-byte aligned
    ops.gemm_launch(a, b, None, cg, None, None, 0, 1, 4, 128, 64, 64, 2, ops.EPI_ALL_SCATTER, notify=False)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype))
    assert float(big[:, :3].float().abs().max()) == 0.0 and float(big[:, 195:].float().abs().max()) == 0.0
    cgt = shmem.zeros((192, 256), dtype=dtype).T  # column-major result
    ops.gemm_launch(a, b, None, cgt, None, None, 0, 1, 4, 128, 64, 64, 2, ops.EPI_ALL_SCATTER, notify=False)
    torch.cuda.synchronize()
    check_close(cgt, O.shard_gemm(A, B, dtype))
    c32 = shmem.zeros((256, 192), dtype=torch.float32)  # fp32 destination
    ops.gemm_launch(a, b, None, c32, None, None, 0, 1, 4, 128, 64, 64, 2, ops.EPI_ALL_SCATTER, notify=False)
    torch.cuda.synchronize()
    check_close(c32, O.shard_gemm(A, B, None))


def _variant_names():
    """The compiled kernel variants of the bf16 store path, asked of the
    library (a host-side table: no device is touched)."""
    names, v = [], 1
    while (name := ops.gemm_variant_name(torch.bfloat16, False, False, v)) is not None:
        names.append(name)
        v += 1
    assert len(names) >= 7  # the seven base tiles always exist
    return names


@pytest.mark.parametrize("variant,name", [(i + 1, n) for i, n in enumerate(_variant_names())])
def test_every_tuning_variant_is_correct(shmem, variant, name):
    """Each compiled kernel variant of the bf16 store path, forced on a shape
    with ragged edges and several tiles per program."""
    dtype = torch.bfloat16
    M, N, K = 520, 776, 328
    A, B = make_ab(M, N, K, dtype, lda=336, ldb=344)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, 256) * ops.cdiv(N, 256)
    flags = shmem.zeros((total,), dtype=torch.int32)
    ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 5, 256, 256, 64, 2, ops.EPI_ALL_SCATTER, variant=variant)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype), name)
    assert flags.cpu().tolist() == [1] * total


# --------------------------------------------------------------------------- atomics
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_atomic_accumulate_of_eight_k_shards(shmem, out_dtype):
    """Eight sequential shard GEMMs, each adding its tiles into one shared C."""
    M, N, K, ws = 512, 384, 1024, 8
    dtype = torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=out_dtype)
    ks = K // ws
    for r in range(ws):
        ops.gemm_launch(a_full[:, r * ks:(r + 1) * ks], b_full[r * ks:(r + 1) * ks, :], None, cg, None, None, 0, 1,
                        8, 256, 128, 64, 6, ops.EPI_ATOMIC_ADD)
    torch.cuda.synchronize()
    want = O.atomics_all_reduce(O.k_shards(A, B, ws))
    if out_dtype == torch.float32:
        check_close(cg, want, "fp32 atomics")
    else:
        # 16-bit accumulation rounds after every add: 8 roundings of half an ulp each
        err = (cg.float().cpu() - want).abs()
        assert float(err.max()) <= 8 * 2.0 ** -8 * float(want.abs().max()) + ATOL
        # per 16 x 16 block the eight roundings add up like a random walk: well inside 2^-6 of the block's norm
        assert bool(blocks_ok(cg, want, block_rtol=2.0 ** -6).all())


def test_atomic_add_ragged_and_on_every_rank(shmem):
    M, N, K, ws = 200, 136, 96, 2
    dtype = torch.float16
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=torch.float32)
    for r in range(ws):
        shmem.on_rank(cg, r).fill_(1.0)
    # rank 1 adds its product into c_global of both ranks
    ops.gemm_launch(a, b, None, shmem.on_rank(cg, 1), None, shmem.get_heap_bases(), 1, ws, 4, 128, 64, 64, 2,
                    ops.EPI_ATOMIC_ADD)
    torch.cuda.synchronize()
    want = O.shard_gemm(A, B, None) + 1.0
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}")


# --------------------------------------------------------------------------- one-shot
@pytest.mark.parametrize("phase", [ops.PHASE_FUSED, ops.PHASE_TWO_KERNELS])  # reduce in the program / behind it
@pytest.mark.parametrize("partial_dtype", [torch.bfloat16, torch.float32])
def test_one_shot_fused_single_rank(shmem, partial_dtype, phase):
    """world_size 1: store the tile to C, no flag traffic, c_global = cast(C)."""
    M, N, K = 384, 320, 192
    dtype = torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    c = shmem.zeros((M, N), dtype=partial_dtype)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, 128) * ops.cdiv(N, 64)
    flags = shmem.zeros((total,), dtype=torch.int32)
    ops.gemm_launch(a, b, c, cg, flags, shmem.get_heap_bases(), 0, 1, 8, 128, 64, 64, 6, ops.EPI_ONE_SHOT,
                    phase=phase)
    torch.cuda.synchronize()
    check_close(c, O.shard_gemm(A, B, partial_dtype), "partial")
    assert torch.equal(cg.cpu(), O.one_shot_reduce(c.cpu()[None], dtype))  # bit-exact given the partial
    assert flags.cpu().tolist() == [0] * total  # ws == 1: no flag is ever written


@pytest.mark.parametrize("ws,partial_dtype", [(2, torch.bfloat16), (8, torch.float32), (8, torch.float16)])
def test_one_shot_all_reduce_virtual_ranks(shmem, ws, partial_dtype):
    """K-split over ws ranks on one GPU: every rank produces (partial tile +
    signal), then every rank consumes (wait, reduce, store)."""
    M, N, K, BM, BN, G = 256, 320, 64 * ws, 128, 64, 6
    dtype = torch.float16 if partial_dtype == torch.float16 else torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    ks = K // ws
    c = shmem.zeros((M, N), dtype=partial_dtype)
    cg = shmem.zeros((M, N), dtype=dtype)
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
    fm = O.FlagModel(ws, total)
    for r in range(ws):
        for t in range(total):
            fm.signal(r, t)
    for r in range(ws):  # every producer added +1 on every *other* rank
        assert shmem.on_rank(flags, r).cpu().tolist() == fm.flags[r].tolist() == [ws - 1] * total
    partials = torch.stack([shmem.on_rank(c, r).cpu() for r in range(ws)])
    shards = O.k_shards(A, B, ws)
    for r in range(ws):
        check_close(partials[r], O.shard_gemm(*shards[r], partial_dtype), f"partial {r}")
    for r in range(ws):
        launch(r, ops.PHASE_CONSUME)
    torch.cuda.synchronize()
    want_bits = O.one_shot_reduce(partials, dtype)
    for r in range(ws):
        assert torch.equal(shmem.on_rank(cg, r).cpu(), want_bits), f"rank {r}"  # fixed rank order: bit-exact
        assert shmem.on_rank(flags, r).cpu().tolist() == [0] * total            # the CAS resets every flag
    check_close(cg, O.one_shot_all_reduce(shards, partial_dtype, dtype), "vs closed form")
    assert int(status.item()) == 0


@pytest.mark.parametrize("phase", [ops.PHASE_FUSED, ops.PHASE_TWO_KERNELS])
def test_fused_phase_with_peers_missing_times_out_and_exits(shmem, phase):
    """A rank whose peers never signal: the bounded wait gives up, reports it
    and skips the reduce; the kernel still drains."""
    M, N, K, ws = 128, 128, 64, 2
    dtype = torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    c = shmem.zeros((M, N), dtype=dtype)
    cg = shmem.full((M, N), 5, dtype=dtype)
    flags = shmem.zeros((4,), dtype=torch.int32)
    for r in range(ws):
        shmem.on_rank(flags, r).zero_()
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.gemm_launch(a, b, c, cg, flags, shmem.get_heap_bases(), 0, ws, 4, 64, 64, 64, 1, ops.EPI_ONE_SHOT,
                    phase=phase, status=status, spin_timeout_ticks=2000)  # 20 us
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    assert float((cg.float() - 5).abs().max()) == 0.0  # nothing was reduced
    check_close(c, O.shard_gemm(A, B, dtype))           # the partial was still produced
    assert shmem.on_rank(flags, 1).cpu().tolist() == [1] * 4 and flags.cpu().tolist() == [0] * 4


# --------------------------------------------------------------------------- schedule, timestamps, registers
@pytest.mark.parametrize("M,N,BM,BN,G,num_sms,x", [
    (8192, 8192, 256, 256, 4, 256, 8), (8192, 8192, 256, 256, 6, 256, 1), (4096, 4096, 256, 256, 6, 288, 8),
    (2048, 1376, 256, 64, 4, 304, 8), (1, 1376, 256, 256, 4, 256, 8), (1000, 999, 64, 64, 5, 56, 4),
])
def test_device_tile_schedule_is_bit_exact(M, N, BM, BN, G, num_sms, x):
    got = ops.tile_schedule(M, N, BM, BN, G, num_sms, x).cpu().numpy()
    total = O.cdiv(M, BM) * O.cdiv(N, BN)
    want = np.full((total, 4), -1, dtype=np.int32)
    want[:, :2] = O.tile_map_all(M, N, BM, BN, G)
    for p in range(num_sms):
        for pos, t in enumerate(O.program_tiles(p, total, num_sms, x)):
            want[t, 2:] = (p, pos)
    assert (got == want).all()


def test_tile_timestamps_and_kernel_info(shmem):
    M, N, K = 512, 512, 128
    dtype = torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = 16
    flags = shmem.zeros((total,), dtype=torch.int32)
    begin = torch.full((total,), torch.iinfo(torch.int64).max, dtype=torch.int64, device="cuda")
    end = torch.zeros(total, dtype=torch.int64, device="cuda")
    ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 2, 128, 128, 64, 2, ops.EPI_ALL_SCATTER,
                    mm_begin_timestamp=begin, mm_end_timestamp=end)
    torch.cuda.synchronize()
    bg, en = begin.cpu(), end.cpu()
    assert (bg < torch.iinfo(torch.int64).max).all() and (en > 0).all() and (bg <= en).all()
    # program 0 walks tiles 0, 2, 4, ... in order
    mine = bg[0::2]
    assert (mine[1:] >= mine[:-1]).all()
    check_close(cg, O.shard_gemm(A, B, dtype))
    regs, spills = ops.gemm_kernel_info(a, b, None, cg, flags, None, 0, 1, 2, 128, 128, 64, 2, ops.EPI_ALL_SCATTER)
    assert 0 < regs <= 512 and spills == 0


def test_launcher_rejects_what_the_kernels_do_not_take(shmem):
    A, B = make_ab(64, 64, 64, torch.bfloat16)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((64, 64), dtype=torch.bfloat16)
    with pytest.raises(ValueError):  # c_global too small for two ranks' columns
        ops.gemm_launch(a, b, None, cg, None, shmem.get_heap_bases(), 0, 2, 4, 64, 64, 64, 1, ops.EPI_ALL_SCATTER,
                        notify=False)
    with pytest.raises(ValueError):  # too few flags
        ops.gemm_launch(a, b, None, cg, shmem.zeros((0,), dtype=torch.int32), None, 0, 1, 4, 32, 32, 64, 1,
                        ops.EPI_ALL_SCATTER)
    with pytest.raises(ValueError):  # grid does not split over the XCDs
        ops.gemm_launch(a, b, None, cg, None, None, 0, 1, 12, 64, 64, 64, 1, ops.EPI_ALL_SCATTER, notify=False,
                        num_xcds=8)
    with pytest.raises(ValueError):  # fp16 result from bf16 operands
        ops.gemm_launch(a, b, None, shmem.zeros((64, 64), dtype=torch.float16), None, None, 0, 1, 4, 64, 64, 64, 1,
                        ops.EPI_ALL_SCATTER, notify=False)
    with pytest.raises(ValueError):  # fp32 operands with a 16-bit result
        ops.gemm_launch(a.float(), b.float(), None, cg, None, None, 0, 1, 4, 64, 64, 64, 1, ops.EPI_ALL_SCATTER,
                        notify=False)
    with pytest.raises(TypeError):  # integer operands
        ops.gemm_launch(a.to(torch.int8), b.to(torch.int8), None, cg, None, None, 0, 1, 4, 64, 64, 64, 1,
                        ops.EPI_ALL_SCATTER, notify=False)


def test_small_tiles_get_two_programs_per_cu_when_the_launch_owns_the_device(shmem):
    """64 x 64 tiles take less than half a CU's LDS: a launch with one program
    per CU and two tiles or more per program runs two programs per CU.  Which
    program computes a tile is not observable: values and flags are checked."""
    dtype = torch.bfloat16
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    M, N, K, BM, BN = 2048, 1024, 320, 64, 64
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    args = (a, b, None, cg, flags, None, 0, 1, cus, BM, BN, 64, 4, ops.EPI_ALL_SCATTER)
    assert total >= 2 * cus and ops.gemm_plan_name(*args, num_xcds=8).endswith("+two_per_cu")
    assert not ops.gemm_plan_name(a, b, None, cg, flags, None, 0, 1, cus // 2, BM, BN, 64, 4, ops.EPI_ALL_SCATTER,
                                  num_xcds=8).endswith("+two_per_cu")  # half the device: the grid is the caller's
    ops.gemm_launch(*args, num_xcds=8)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype))
    assert flags.cpu().tolist() == [1] * total


def test_store_probe_writes_every_groups_region(shmem):
    """The store probe (a measurement aid): every wave writes its 16 KiB of
    every tile, whatever the spreading, and nothing outside."""
    groups, tiles = 8, 3
    operands = torch.ones(32768, dtype=torch.bfloat16, device="cuda")
    sink = torch.zeros(groups * 512, dtype=torch.float32, device="cuda")
    for chunk in (16, 4, 1):
        for wt in (True, False):
            out = torch.full((tiles * groups * 131072 + 4096,), 0x5A, dtype=torch.uint8, device="cuda")
            assert testing.store_probe(operands, sink, out[:-4096], tiles, chunk, groups, write_through=wt) == tiles * groups * 131072
            torch.cuda.synchronize()
            body = out[:-4096].view(torch.float32)
            # accumulators of ones x ones products: whole numbers, never the fill pattern
            assert bool((body == body.round()).all()) and bool((body > 0).any())
            assert not bool((out[:-4096] == 0x5A).view(-1, 16).all(dim=1).any()), "a 16-byte unit was not written"
            assert bool((out[-4096:] == 0x5A).all())
    out = torch.full((groups * 131072,), 0x5A, dtype=torch.uint8, device="cuda")
    assert testing.store_probe(operands, sink, out, tiles, 0, groups) == 0
    torch.cuda.synchronize()
    assert bool((out == 0x5A).all()) and bool(torch.isfinite(sink).all())
    with pytest.raises(ValueError):
        testing.store_probe(operands, sink, out[:1000], tiles, 16, groups)
    with pytest.raises(ValueError):
        testing.store_probe(operands, sink, out, tiles, 3, groups)


def _fetching_wave_cases():
    """(epilogue, name with fetching waves, variant, name of the plain build of the same tile and wave layout,
    variant), from the kernel list each epilogue launches from."""
    cases = []
    for epilogue, out_is_f32, atomic in (("scatter16", False, False), ("split_k", False, False),
                                         ("store32", True, False), ("atomic32", True, True)):
        names, v = [], 1
        while (name := ops.gemm_variant_name(torch.bfloat16, out_is_f32, atomic, v)) is not None:
            names.append(name)
            v += 1
        for i, n in enumerate(names):
            if not n.endswith("_f4"):
                continue
            shape, waves = n.split("x")[:2], n.split("_")[1]
            for j, m in enumerate(names):
                if not m.endswith("_f4") and "generic" not in m and m.split("x")[:2] == shape and m.split("_")[1] == waves:
                    cases.append((epilogue, n, i + 1, m, j + 1))
                    break
    assert len(cases) >= 20
    return cases


@pytest.mark.parametrize("epilogue,f4_name,f4_variant,plain_name,plain_variant", _fetching_wave_cases())
def test_build_with_fetching_waves_is_bit_identical_to_the_plain_build(shmem, epilogue, f4_name, f4_variant, plain_name,
                                                                       plain_variant):
    """The multiplying waves of a `_f4` build run the plain build's MFMA sequence
    on the same fragments: whoever issues the loads, and however deep a stage
    is, the accumulators see the same products in the same order.  Ragged
    edges, a K that ends inside a K-step, several tiles per program."""
    dtype = torch.bfloat16
    M, N, K = 520, 392, 1528  # (twelve 128-deep or twenty-four 64-deep steps: three parts cut K at the same places)
    A, B = make_ab(M, N, K, dtype, lda=1536, ldb=1544)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    bm, bn = (int(v) for v in f4_name.split("x")[:2])
    total = ops.cdiv(M, bm) * ops.cdiv(N, bn)
    got = {}
    for variant in (f4_variant, plain_variant):
        flags = shmem.zeros((total,), dtype=torch.int32)
        if epilogue == "scatter16":
            out = shmem.zeros((M, N), dtype=dtype)
            ops.gemm_launch(a, b, None, out, flags, None, 0, 1, 7, bm, bn, 64, 2, ops.EPI_ALL_SCATTER, variant=variant)
        elif epilogue == "store32":
            out = shmem.zeros((M, N), dtype=torch.float32)
            ops.gemm_launch(a, b, None, out, None, None, 0, 1, 7, bm, bn, 64, 2, ops.EPI_ALL_SCATTER, notify=False,
                            variant=variant)
        elif epilogue == "atomic32":
            out = shmem.zeros((M, N), dtype=torch.float32)
            ops.gemm_launch(a, b, None, out, None, None, 0, 1, 7, bm, bn, 64, 2, ops.EPI_ATOMIC_ADD, variant=variant)
        else:
            out = shmem.zeros((M, N), dtype=dtype)
            partials, locks = split_workspace(shmem, 256, bm, bn)
            assert total * 3 <= 256  # a program for every (tile, part) pair
            ops.gemm_launch(a, b, None, out, flags, None, 0, 1, 256, bm, bn, 64, 2, ops.EPI_ALL_SCATTER,
                            partials=partials, locks=locks, split_k=3, split_handover=ops.HANDOVER_SLICED,
                            variant=variant)
            torch.cuda.synchronize()
            assert int(locks.abs().max().item()) == 0
        torch.cuda.synchronize()
        got[variant] = out.cpu().clone()
        if epilogue in ("scatter16", "split_k"):
            assert flags.cpu().tolist() == [1] * total
    check_close(got[f4_variant].to(torch.float32), O.shard_gemm(A, B, None), f4_name)
    width = torch.int16 if got[f4_variant].dtype == dtype else torch.int32
    assert torch.equal(got[f4_variant].view(width), got[plain_variant].view(width)), f"{f4_name} vs {plain_name}"


@pytest.mark.parametrize("M,N,K,BM,BN,grid,ws,suffix", [
    (1024, 640, 256, 256, 64, 2, 1, "+four_tiles_each"),   # 4 x 10 tiles: the last merged tile of a row covers two
    (1024, 640, 256, 256, 64, 16, 2, "+two_tiles_each"),   # 40 tiles on 16 programs: pairs; flags on both ranks
    (520, 392, 328, 256, 128, 3, 1, "+two_tiles_each"),    # 3 x 4 tiles of 256 x 128, ragged edges
    (1024, 640, 256, 256, 64, 32, 1, ""),                  # too few tiles for the programs: as the caller cut them
    (640, 392, 200, 128, 128, 3, 2, "+four_tiles_each"),   # 5 x 4 tiles of 128 x 128 in blocks of 2 x 2, last row 1 x 2
    (640, 392, 200, 128, 128, 8, 1, "+two_tiles_each"),    # ... one above the other
    (640, 200, 136, 128, 64, 3, 1, "+eight_tiles_each"),   # 5 x 4 tiles of 128 x 64 in blocks of 2 x 4
    (640, 200, 136, 128, 64, 6, 1, "+four_tiles_each"),
])
def test_small_tiles_are_computed_several_at_a_time(shmem, M, N, K, BM, BN, grid, ws, suffix):
    """A caller's 256 x 64, 256 x 128, 128 x 128 or 128 x 64 tiles, where there
    are enough of them, are computed a block at a time as one 256 x 128 or
    256 x 256 tile; every one of the caller's flags is raised exactly once,
    on every rank, and nothing else."""
    dtype = torch.bfloat16
    A, B = make_ab(M, N * ws, K, dtype)
    shards = O.n_shards(A, B, ws)
    a = to_heap(shmem, A)
    bs = [to_heap(shmem, sb) for _, sb in shards]
    cg = shmem.zeros((M, N * ws), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 5,), dtype=torch.int32)
    hb = shmem.get_heap_bases() if ws > 1 else None
    for r in range(ws):
        for t in (cg, flags):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        args = (a, bs[r], None, shmem.on_rank(cg, r), shmem.on_rank(flags, r), hb, r, ws, grid, BM, BN, 64, 3,
                ops.EPI_ALL_SCATTER)
        name = ops.gemm_plan_name(*args)
        assert name.endswith(suffix) and (suffix or "tiles_each" not in name), name
        ops.gemm_launch(*args)
    torch.cuda.synchronize()
    want = O.all_scatter(shards, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws] * total + [0] * 5


def test_merged_tiles_with_the_one_shot_producer_and_reduce(shmem):
    """ONE_SHOT over 2 virtual ranks with the reference's default 256 x 64
    tile: the producers compute four tiles at a time and signal each tile's
    flag on the other rank; the reduce waits per tile of the caller's."""
    ws, M, N, K, dtype = 2, 512, 512, 2 * 192, torch.bfloat16
    A, B = make_ab(M, N, K, dtype)
    shards = O.k_shards(A, B, ws)
    ah, bh = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    part = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, 256) * ops.cdiv(N, 64)
    flags = shmem.zeros((total,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        for t in (part, out, flags):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], shmem.on_rank(part, r), shmem.on_rank(out, r),
                shmem.on_rank(flags, r), hb, r, ws, 4, 256, 64, 64, 6, ops.EPI_ONE_SHOT)
        assert ops.gemm_plan_name(*args, phase=ops.PHASE_PRODUCE).endswith("+four_tiles_each")
        ops.gemm_launch(*args, phase=ops.PHASE_PRODUCE)
    torch.cuda.synchronize()
    for r in range(ws):
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total
    for r in range(ws):
        ops.one_shot_reduce(shmem.on_rank(part, r), shmem.on_rank(out, r), shmem.on_rank(flags, r), hb, r, ws, 256, 64,
                            6)
    torch.cuda.synchronize()
    want = O.one_shot_all_reduce(shards, torch.float32, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(out, r), want, f"reduced on rank {r}")
        assert not shmem.on_rank(flags, r).any()


# --------------------------------------------------------------------------- split-K
def split_workspace(shmem, grid, BM, BN):
    return (shmem.zeros((grid, BM * BN), dtype=torch.float32), shmem.zeros((grid,), dtype=torch.int32))


@pytest.mark.parametrize("M,N,K,BM,BN,split_k", [
    (100, 200, 1024, 64, 64, 2),
    (100, 200, 1024, 64, 64, 8),
    (16, 1376, 4096, 64, 64, 8),     # decoder gate/up at 16 tokens
    (128, 512, 1376, 128, 128, 5),   # 22 K-steps (the last one half empty) in 5 uneven parts
    (200, 72, 776, 256, 64, 4),
    (1, 64, 128, 64, 64, 2),         # one K-step per part
    (500, 300, 1024, 256, 256, 7),   # 128-accumulator tiles (sliced hand-over only), ragged edges
    (256, 512, 2048, 256, 128, 16),
    (128, 500, 640, 128, 256, 3),
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_k_all_scatter(shmem, M, N, K, BM, BN, split_k, dtype):
    """A tile's K range shared by several programs: partials through the
    workspace; either the first part adds them, stores and publishes, or every
    part sums and stores its share of the tile's rows and the last one to
    finish publishes.  Twice in a row each way: the locks are left re-armed.
    Both add the partials in part order, so the results are bit-identical."""
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    grid = 256
    partials, locks = split_workspace(shmem, grid, BM, BN)
    want = O.shard_gemm(A, B, dtype)
    got = {}
    launch = 0
    ways = (ops.HANDOVER_OWNER, ops.HANDOVER_SLICED, ops.HANDOVER_AUTO)
    if BM * BN > 128 * 128:
        ways = (ops.HANDOVER_SLICED, ops.HANDOVER_AUTO)
    for handover in ways:
        for again in (1, 2):
            launch += 1
            cg.zero_()
            ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, grid, BM, BN, 64, 2, ops.EPI_ALL_SCATTER,
                            partials=partials, locks=locks, split_k=split_k, split_handover=handover)
            torch.cuda.synchronize()
            check_close(cg, want, f"hand-over {handover}, launch {again}")
            assert flags.cpu().tolist() == [launch] * total
            assert int(locks.abs().max().item()) == 0
        got[handover] = cg.cpu().clone()
    if ops.HANDOVER_OWNER in got:
        assert torch.equal(got[ops.HANDOVER_OWNER].view(torch.int16), got[ops.HANDOVER_SLICED].view(torch.int16))
    assert torch.equal(got[ops.HANDOVER_AUTO].view(torch.int16), got[ops.HANDOVER_SLICED].view(torch.int16))


@pytest.mark.parametrize("M,N,K,BM,BN,ws", [
    (512, 256, 2048, 256, 128, 1),    # 256 x 128 with fetching waves: waves 0-1 are part 0's, 2-3 part 1's
    (500, 300, 1032, 256, 256, 2),    # 256 x 256, eight waves, ragged edges and a ragged last K-step, two ranks
    (256, 500, 640, 128, 256, 1),     # 128 x 256: the halves are column halves
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_split_k_in_two_parts_with_the_pair_hand_over(shmem, M, N, K, BM, BN, ws, dtype):
    """Two parts of a 128-accumulator tile: each part keeps the accumulators of
    the waves it owns and leaves the other half's in its slot, so slots of
    HALF a tile are enough.  Bit-identical with the sliced hand-over (p0 + p1
    either way); twice in a row: the locks are left re-armed."""
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N * ws), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    grid = 16
    full = shmem.zeros((grid, BM * BN), dtype=torch.float32)
    half = shmem.zeros((grid, BM * BN // 2), dtype=torch.float32)  # what a caller with tiles half as wide holds
    locks = shmem.zeros((grid,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        shmem.on_rank(cg, r).zero_()
        shmem.on_rank(flags, r).zero_()
    want = O.shard_gemm(A, B, dtype)
    rank = ws - 1
    args = (a, b, None, shmem.on_rank(cg, rank), shmem.on_rank(flags, rank), hb, rank, ws, grid, BM, BN, 64, 2,
            ops.EPI_ALL_SCATTER)
    got = {}
    launch = 0
    for name, P, handover in (("sliced", full, ops.HANDOVER_SLICED), ("pair", full, ops.HANDOVER_PAIR),
                              ("pair, half slots", half, ops.HANDOVER_PAIR), ("auto, half slots", half, ops.HANDOVER_AUTO)):
        for again in (1, 2):
            launch += 1
            for r in range(ws):
                shmem.on_rank(cg, r).zero_()
            ops.gemm_launch(*args, partials=P, locks=locks, split_k=2, split_handover=handover)
            torch.cuda.synchronize()
            for r in range(ws):
                block = shmem.on_rank(cg, r)[:, rank * N:(rank + 1) * N]
                check_close(block, want, f"{name}, launch {again}, rank {r}")
                assert shmem.on_rank(flags, r).cpu().tolist() == [launch] * total
            assert int(locks.abs().max().item()) == 0
        got[name] = shmem.on_rank(cg, 0)[:, rank * N:(rank + 1) * N].cpu().clone()
    for name in got:
        assert torch.equal(got[name], got["sliced"]), name
    # the sliced hand-over does not fit slots of half a tile, and a pair is two parts
    with pytest.raises(ValueError):
        ops.gemm_launch(*args, partials=half, locks=locks, split_k=2, split_handover=ops.HANDOVER_SLICED)
    with pytest.raises(ValueError):
        ops.gemm_launch(*args, partials=full, locks=locks, split_k=4, split_handover=ops.HANDOVER_PAIR)
    assert ops.gemm_split_k(*args, partials=half, locks=locks, split_k=0) in (1, 2)  # never more with half slots


@pytest.mark.parametrize("M,N,K,BM,BN,grid,kernel", [
    # 2 x 7 tiles of 256 x 64 on 16 programs: 8 blocks of two tiles (the last one a single tile), K in two parts
    (512, 448, 4096, 256, 64, 16, "256x128x64_w2x2_s3_f4+two_tiles_each"),
    # 2 x 4 tiles of 256 x 128 on 8 programs: 4 blocks of two tiles as 256 x 256, K in two parts
    (512, 512, 4096, 256, 128, 8, "256x256x64_w2x4_s2+two_tiles_each"),
    # 2 x 3 tiles of 256 x 64, ragged in M and N, on 8 programs: 2 x 2 blocks, the last column a single narrow tile
    (500, 180, 4096, 256, 64, 8, "256x128x64_w2x2_s3_f4+two_tiles_each"),
    # 2 x 9 tiles of 256 x 64 on 16 programs: the first eight columns as 8 blocks with K in two parts, then the
    # ninth as a launch of its own (2 tiles, K in eight parts), whose flags sit in the caller's ninth column
    (512, 576, 4096, 256, 64, 16, "256x128x64_w2x2_s3_f4+two_tiles_each+last_64_columns_apart"),
])
def test_blocks_of_the_callers_tiles_with_k_in_two_parts(shmem, M, N, K, BM, BN, grid, kernel):
    """Too few blocks of the caller's tiles for every program, but enough for
    every other one: each block's K range is shared by two programs, whose
    hand-over fits the caller's workspace (slots of one of ITS tiles).  Every
    tile of the caller keeps its id and its flag."""
    dtype, ws = torch.bfloat16, 2
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N * ws), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 2,), dtype=torch.int32)
    partials, locks = split_workspace(shmem, grid, BM, BN)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        shmem.on_rank(cg, r).zero_()
        shmem.on_rank(flags, r).zero_()
    args = (a, b, None, shmem.on_rank(cg, 1), shmem.on_rank(flags, 1), hb, 1, ws, grid, BM, BN, 64, 1, ops.EPI_ALL_SCATTER)
    assert ops.gemm_plan_name(*args, partials=partials, locks=locks) == kernel
    assert ops.gemm_split_k(*args, partials=partials, locks=locks) == 2
    assert ops.gemm_split_k(*args) == 1  # no workspace: the caller's tiles, unsplit
    want = O.shard_gemm(A, B, dtype)
    for launch in (1, 2):
        ops.gemm_launch(*args, partials=partials, locks=locks)
        torch.cuda.synchronize()
        for r in range(ws):
            check_close(shmem.on_rank(cg, r)[:, N:], want, f"launch {launch}, rank {r}")
            assert shmem.on_rank(flags, r).cpu().tolist() == [launch] * total + [0, 0]
            assert float(shmem.on_rank(cg, r)[:, :N].float().abs().max()) == 0.0  # rank 0's columns untouched
        assert int(locks.abs().max().item()) == 0


def test_split_k_is_chosen_for_few_tiles_and_long_k_only(shmem):
    dtype = torch.bfloat16
    A, B = make_ab(72, 1376, 4096, dtype)  # (up to 64 rows would go to the few-rows kernel)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((72, 1376), dtype=dtype)
    flags = shmem.zeros((64,), dtype=torch.int32)
    partials, locks = split_workspace(shmem, 256, 64, 64)
    common = (a, b, None, cg, flags, None, 0, 1, 256, 64, 64, 64, 4, ops.EPI_ALL_SCATTER)
    # 44 tiles on 256 programs, K = 4096: 5 parts each
    assert ops.gemm_split_k(*common, partials=partials, locks=locks) == 5
    assert ops.gemm_split_k(*common) == 1                                    # no workspace
    assert ops.gemm_split_k(*common, partials=partials, locks=locks, split_k=1) == 1
    ops.gemm_launch(*common, partials=partials, locks=locks)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype))
    assert flags.cpu().tolist()[:44] == [1] * 44 and int(locks.abs().max().item()) == 0
    # enough tiles to fill the programs: unsplit
    A2, B2 = make_ab(1024, 1024, 512, dtype)
    a2, b2 = to_heap(shmem, A2), to_heap(shmem, B2)
    cg2 = shmem.zeros((1024, 1024), dtype=dtype)
    flags2 = shmem.zeros((256,), dtype=torch.int32)
    assert ops.gemm_split_k(a2, b2, None, cg2, flags2, None, 0, 1, 256, 64, 64, 64, 4, ops.EPI_ALL_SCATTER,
                            partials=partials, locks=locks) == 1
    # a forced split the launch cannot honour is an error, not a silent fallback
    with pytest.raises(ValueError):
        ops.gemm_launch(*common, split_k=4)                                  # no workspace
    with pytest.raises(ValueError):
        ops.gemm_launch(*common, partials=partials, locks=locks, split_k=8)   # 44 * 8 pairs > 256 programs
    # the 128-accumulator tiles split too, with the sliced hand-over only
    big = shmem.zeros((256, 256 * 256), dtype=torch.float32)
    with pytest.raises(ValueError):
        ops.gemm_launch(a2, b2, None, cg2, flags2, None, 0, 1, 256, 256, 256, 64, 4, ops.EPI_ALL_SCATTER,
                        partials=big, locks=locks, split_k=2, split_handover=ops.HANDOVER_OWNER)
    with pytest.raises(ValueError):  # and never stream-K
        ops.gemm_launch(a2, b2, None, cg2, flags2, None, 0, 1, 256, 256, 256, 64, 4, ops.EPI_ALL_SCATTER,
                        partials=big, locks=locks, split_k=ops.SPLIT_STREAM_K)
    for sk in (2, 8):
        cg2.zero_()
        flags2.zero_()
        ops.gemm_launch(a2, b2, None, cg2, flags2, None, 0, 1, 256, 256, 256, 64, 4, ops.EPI_ALL_SCATTER,
                        partials=big, locks=locks, split_k=sk)
        torch.cuda.synchronize()
        check_close(cg2, O.shard_gemm(A2, B2, dtype), f"256 x 256 tiles in {sk} parts")
        assert flags2.cpu().tolist()[:16] == [1] * 16 and int(locks.abs().max().item()) == 0
    # a split 256 x 128 tile runs the build with fetching waves, like an unsplit one; the plain build of the same
    # tile (every wave fetches its share) has a split build too, reached by its variant number
    plain = _variant_names().index("256x128x64_w2x2_s2") + 1
    for K3, variant, name in ((8192, 0, "256x128x64_w2x2_s3_f4"), (4096, 0, "256x128x64_w2x2_s3_f4"),
                              (4096, plain, "256x128x64_w2x2_s2")):
        A3, B3 = make_ab(512, 256, K3, dtype)
        a3, b3 = to_heap(shmem, A3), to_heap(shmem, B3)
        cg3 = shmem.zeros((512, 256), dtype=dtype)
        flags2.zero_()
        args3 = (a3, b3, None, cg3, flags2, None, 0, 1, 16, 256, 128, 64, 4, ops.EPI_ALL_SCATTER)
        assert ops.gemm_split_k(*args3, partials=big, locks=locks, variant=variant) == 4
        assert ops.gemm_plan_name(*args3, partials=big, locks=locks, variant=variant) == name
        ops.gemm_launch(*args3, partials=big, locks=locks, variant=variant)
        torch.cuda.synchronize()
        check_close(cg3, O.shard_gemm(A3, B3, dtype), f"256 x 128 tiles in 4 parts, K = {K3}, {name}")
        assert flags2.cpu().tolist()[:4] == [1] * 4 and int(locks.abs().max().item()) == 0


@pytest.mark.parametrize("M,N,BN,ws,suffix", [
    # 18 tiles on 16 programs: 16 whole, 2 in four parts (the owner's hand-over)
    (1536, 192, 64, 1, "256x64x64_w4x1_s3_f4+last_round_in_4_parts"),
    # 18 tiles: 16 whole, 2 in four parts (the sliced hand-over), on two ranks
    (1536, 384, 128, 2, "256x128x64_w2x2_s3_f4+last_round_in_4_parts"),
    # nine columns of tiles: eight of them in blocks of two tiles with K in two parts, the ninth as a launch of its own
    (512, 576, 64, 1, "256x128x64_w2x2_s3_f4+two_tiles_each+last_64_columns_apart"),
    (512, 1152, 128, 2, "256x256x64_w2x4_s2+two_tiles_each+last_128_columns_apart"),
])
def test_a_short_last_round_of_long_tiles_is_split_over_the_idle_programs(shmem, M, N, BN, ws, suffix):
    """Tiles a few more than a multiple of the programs, K long: the full rounds
    run as they are and a second launch shares K of the last round's tiles
    out; values, every flag once on every rank, workspace left clean."""
    K, grid, dtype = 8192, 16, torch.bfloat16
    A, B = make_ab(M, N * ws, K, dtype)
    shards = O.n_shards(A, B, ws)
    a = to_heap(shmem, A)
    bs = [to_heap(shmem, sb) for _, sb in shards]
    cg = shmem.zeros((M, N * ws), dtype=dtype)
    total = ops.cdiv(M, 256) * ops.cdiv(N, BN)
    flags = shmem.zeros((total + 3,), dtype=torch.int32)
    partials, locks = split_workspace(shmem, grid, 256, BN)
    hb = shmem.get_heap_bases() if ws > 1 else None
    for r in range(ws):
        for t in (cg, flags):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        args = (a, bs[r], None, shmem.on_rank(cg, r), shmem.on_rank(flags, r), hb, r, ws, grid, 256, BN, 64, 4,
                ops.EPI_ALL_SCATTER)
        assert ops.gemm_plan_name(*args, partials=partials, locks=locks) == suffix
        assert "last_" not in ops.gemm_plan_name(*args)                         # no workspace: as before
        ops.gemm_launch(*args, partials=partials, locks=locks)
        torch.cuda.synchronize()
        assert int(locks.abs().max().item()) == 0
    want = O.all_scatter(shards, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws] * total + [0] * 3
    # a shorter K keeps the one launch
    assert "last_" not in ops.gemm_plan_name(a[:, :2048], bs[0][:2048], None, cg, flags, hb, 0, ws, grid, 256, BN, 64,
                                                  4, ops.EPI_ALL_SCATTER, partials=partials, locks=locks)


@pytest.mark.parametrize("M,N,plan", [
    # 16 whole tiles, then the last two in four parts
    (1536, 192, "256x64x64_w4x1_s3_f4+last_round_in_4_parts"),
    # eight columns of tiles in blocks of two with K in two parts, then the ninth column
    (512, 576, "256x128x64_w2x2_s3_f4+two_tiles_each+last_64_columns_apart"),
])
def test_split_last_round_with_the_one_shot_producer_and_reduce(shmem, M, N, plan):
    """K-shards on two ranks, 18 tiles of 256 x 64 on 16 programs, K = 8192 a rank:
    each producer is two launches, the fp32 partials and the flags on the other
    rank are as from one launch, and the reduce gives the oracle's sum."""
    ws, dtype, grid = 2, torch.bfloat16, 16
    K = 8192 * ws
    A, B = make_ab(M, N, K, dtype)
    shards = O.k_shards(A, B, ws)
    ah, bh = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    part = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, 256) * ops.cdiv(N, 64)
    flags = shmem.zeros((total,), dtype=torch.int32)
    partials, locks = split_workspace(shmem, grid, 256, 64)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        for t in (part, out, flags):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        args = (ah[:, r * kk:(r + 1) * kk], bh[r * kk:(r + 1) * kk, :], shmem.on_rank(part, r), shmem.on_rank(out, r),
                shmem.on_rank(flags, r), hb, r, ws, grid, 256, 64, 64, 6, ops.EPI_ONE_SHOT)
        kw = dict(phase=ops.PHASE_PRODUCE, partials=partials, locks=locks)
        assert ops.gemm_plan_name(*args, **kw) == plan
        ops.gemm_launch(*args, **kw)
        torch.cuda.synchronize()
        assert int(locks.abs().max().item()) == 0
        check_close(shmem.on_rank(part, r), O.shard_gemm(*shards[r], torch.float32), f"partial of rank {r}")
    for r in range(ws):
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total
    for r in range(ws):
        ops.one_shot_reduce(shmem.on_rank(part, r), shmem.on_rank(out, r), shmem.on_rank(flags, r), hb, r, ws, 256, 64,
                            6)
    torch.cuda.synchronize()
    want = O.one_shot_all_reduce(shards, torch.float32, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(out, r), want, f"reduced on rank {r}")
        assert not shmem.on_rank(flags, r).any()


STREAM_K_CASES = [
    # M, N, K, BLK_M, BLK_N, grid, dtype
    (2048, 1376, 1024, 128, 128, 256, torch.bfloat16),  # 176 tiles x 16 steps on 256 programs: runs of 11
    (512, 768, 2048, 128, 128, 16, torch.bfloat16),     # 24 x 32 steps on 16 programs: tail, whole tile, head
    (300, 200, 1376, 64, 64, 24, torch.float16),        # ragged M, N and K; 20 x 22 steps = 24 runs of 18 or 19
    (256, 320, 4096, 256, 64, 8, torch.bfloat16),       # 5 x 64 steps on 8 programs
    (64, 128, 8192, 64, 64, 16, torch.bfloat16),        # 2 tiles, 8 runs each: an owner and seven followers
    (128, 128, 512, 64, 64, 4, torch.float16),          # runs that end exactly at tile boundaries
    (256, 384, 512, 64, 64, 5, torch.bfloat16),         # 24 x 8 steps on 5 programs: runs of four and five tiles
]


@pytest.mark.parametrize("M,N,K,BM,BN,grid,dtype", STREAM_K_CASES)
def test_stream_k_all_scatter(shmem, M, N, K, BM, BN, grid, dtype):
    """The launch's K-steps cut into equal runs that cross tile boundaries:
    the program that holds a tile's first step owns it and adds what the
    programs after it hand over.  Twice in a row: the locks are left re-armed."""
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    partials, locks = split_workspace(shmem, grid, BM, BN)
    args = (a, b, None, cg, flags, None, 0, 1, grid, BM, BN, 64, 2, ops.EPI_ALL_SCATTER)
    kw = dict(partials=partials, locks=locks, split_k=ops.SPLIT_STREAM_K, num_xcds=ops.default_num_xcds(256, grid))
    assert ops.gemm_split_k(*args, **kw) == ops.SPLIT_STREAM_K
    assert ops.gemm_plan_name(*args, **kw).endswith("+stream_k")
    want = O.shard_gemm(A, B, dtype)
    for launch in (1, 2):
        cg.zero_()
        ops.gemm_launch(*args, **kw)
        torch.cuda.synchronize()
        check_close(cg, want, f"launch {launch}")
        assert flags.cpu().tolist() == [launch] * total
        assert int(locks.abs().max().item()) == 0


def test_stream_k_is_only_taken_on_request(shmem):
    dtype = torch.bfloat16
    A, B = make_ab(1024, 1376, 2048, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((1024, 1376), dtype=dtype)
    flags = shmem.zeros((128,), dtype=torch.int32)
    partials, locks = split_workspace(shmem, 256, 128, 128)

    def choice(grid, BM, BN, **kw):
        return ops.gemm_split_k(a, b, None, cg, flags, None, 0, 1, grid, BM, BN, 64, 4, ops.EPI_ALL_SCATTER,
                                partials=partials, locks=locks, **kw)

    assert choice(256, 128, 128) == 2                        # 88 tiles on 256 programs: two parts each
    assert choice(256, 128, 128, split_k=ops.SPLIT_STREAM_K) == ops.SPLIT_STREAM_K
    assert choice(64, 128, 128) == 1                         # more tiles than programs
    assert choice(88, 128, 128) == 1                         # one tile each
    assert choice(44, 128, 128) == 1                         # two rounds, both full
    assert choice(256, 128, 128, split_k=1) == 1
    assert choice(256, 256, 256) == 1                        # the workspace's slots are too small for this tile
    ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 256, 128, 128, 64, 4, ops.EPI_ALL_SCATTER, partials=partials,
                    locks=locks)
    torch.cuda.synchronize()
    check_close(cg, O.shard_gemm(A, B, dtype))
    assert flags.cpu().tolist()[:88] == [1] * 88 and int(locks.abs().max().item()) == 0
    with pytest.raises(ValueError):  # no workspace
        ops.gemm_launch(a, b, None, cg, flags, None, 0, 1, 256, 128, 128, 64, 4, ops.EPI_ALL_SCATTER,
                        split_k=ops.SPLIT_STREAM_K)
    with pytest.raises(ValueError):  # runs shorter than four steps
        ops.gemm_launch(a[:, :128], b[:128, :], None, cg, flags, None, 0, 1, 256, 128, 128, 64, 4,
                        ops.EPI_ALL_SCATTER, partials=partials, locks=locks, split_k=ops.SPLIT_STREAM_K)


def test_stream_k_with_the_other_epilogues_and_virtual_ranks(shmem):
    """Atomic accumulate and the one-shot producer behind stream-K runs."""
    dtype = torch.bfloat16
    ws = 4
    M, N, K = 192, 320, 4 * 768
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    hb = shmem.get_heap_bases()
    shards = O.k_shards(A, B, ws)
    kk = K // ws
    grid, BM, BN = 16, 64, 64
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    partials, locks = split_workspace(shmem, grid, BM, BN)
    # 08: every rank adds its shard product into every rank's fp32 C
    cg = shmem.zeros((M, N), dtype=torch.float32)
    for r in range(ws):
        shmem.on_rank(cg, r).zero_()
        shmem.on_rank(locks, r).zero_()  # (zeros() clears rank 0's copy only)
    for r in range(ws):
        ops.gemm_launch(a[:, r * kk:(r + 1) * kk], b[r * kk:(r + 1) * kk, :], None, shmem.on_rank(cg, r), None, hb, r,
                        ws, grid, BM, BN, 64, 4, ops.EPI_ATOMIC_ADD, partials=shmem.on_rank(partials, r),
                        locks=shmem.on_rank(locks, r), split_k=ops.SPLIT_STREAM_K)
    torch.cuda.synchronize()
    want = O.atomics_all_reduce(shards)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"atomic, rank {r}")
    # 09: producers, then the reduce
    part = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    flags = shmem.zeros((total,), dtype=torch.int32)
    for r in range(ws):
        for t in (part, out, flags):
            shmem.on_rank(t, r).zero_()
    for r in range(ws):
        ops.gemm_launch(a[:, r * kk:(r + 1) * kk], b[r * kk:(r + 1) * kk, :], shmem.on_rank(part, r),
                        shmem.on_rank(out, r), shmem.on_rank(flags, r), hb, r, ws, grid, BM, BN, 64, 6,
                        ops.EPI_ONE_SHOT, phase=ops.PHASE_PRODUCE, partials=shmem.on_rank(partials, r),
                        locks=shmem.on_rank(locks, r), split_k=ops.SPLIT_STREAM_K)
    torch.cuda.synchronize()
    for r in range(ws):
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total
        assert not shmem.on_rank(locks, r).any()
    for r in range(ws):
        ops.one_shot_reduce(shmem.on_rank(part, r), shmem.on_rank(out, r), shmem.on_rank(flags, r), hb, r, ws, BM,
                            BN, 6)
    torch.cuda.synchronize()
    want = O.one_shot_all_reduce(shards, torch.float32, dtype)
    for r in range(ws):
        check_close(shmem.on_rank(out, r), want, f"one-shot, rank {r}")


def test_split_k_with_the_other_epilogues_and_virtual_ranks(shmem):
    """Atomic accumulate and the one-shot producer behind a split K loop."""
    dtype = torch.bfloat16
    ws = 4
    M, N, K = 64, 256, 2048
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    hb = shmem.get_heap_bases()
    partials, locks = split_workspace(shmem, 256, 64, 64)
    want32 = O.shard_gemm(A, B, None)
    c32 = shmem.zeros((M, N), dtype=torch.float32)
    for r in range(ws):
        shmem.on_rank(c32, r).zero_()
    for handover in (ops.HANDOVER_OWNER, ops.HANDOVER_SLICED):
        for r in range(ws):
            shmem.on_rank(c32, r).zero_()
        ops.gemm_launch(a, b, None, shmem.on_rank(c32, 1), None, hb, 1, ws, 256, 64, 64, 64, 2, ops.EPI_ATOMIC_ADD,
                        partials=partials, locks=locks, split_k=8, split_handover=handover)
        torch.cuda.synchronize()
        for r in range(ws):
            check_close(shmem.on_rank(c32, r), want32, f"atomic add on rank {r}, hand-over {handover}")
        assert int(locks.abs().max().item()) == 0
    part = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    flags = shmem.zeros((4,), dtype=torch.int32)
    for r in range(ws):
        shmem.on_rank(flags, r).zero_()
    for n, handover in enumerate((ops.HANDOVER_OWNER, ops.HANDOVER_SLICED), start=1):
        shmem.on_rank(part, 2).zero_()
        ops.gemm_launch(a, b, shmem.on_rank(part, 2), shmem.on_rank(out, 2), shmem.on_rank(flags, 2), hb, 2, ws, 256,
                        64, 64, 64, 2, ops.EPI_ONE_SHOT, phase=ops.PHASE_PRODUCE, partials=partials, locks=locks,
                        split_k=4, split_handover=handover)
        torch.cuda.synchronize()
        check_close(shmem.on_rank(part, 2), want32, f"one-shot partial, hand-over {handover}")
        for r in range(ws):  # the producer signals every other rank once per tile
            assert shmem.on_rank(flags, r).cpu().tolist() == [0 if r == 2 else n] * 4
        assert int(locks.abs().max().item()) == 0
