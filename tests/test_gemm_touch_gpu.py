"""The eight-wave 256 x 256 tile's build that touches the operand lines of
K-steps to come (``iris_gemm_args.touch_ahead``): it must give the bits of the
plain build on every shape, and the launcher must take it where a round of
tiles streams its operands from HBM, and only there.

The touches are loads whose data nothing reads; what can go wrong is the
count of loads the hand-over leaves in flight (a stage read before it has
landed) and a touch outside the operand (rows past the matrix edge, K-steps
past the end of a tile), so the cases are ragged in M, N and K, walk several
tiles per program, and run merged tiles and the fp32-output epilogue.
"""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O
from parity import check_close, make_ab
from test_gemm_gpu import to_heap

pytestmark = pytest.mark.gpu

BF16, F16, F32 = torch.bfloat16, torch.float16, torch.float32

CASES = [
    # M, N, K, BLK_M, BLK_N, G, grid, xcds, dtype
    (512, 512, 4096, 256, 256, 4, 256, 8, BF16),     # four tiles on 256 programs: an XCD holds one
    (2048, 2048, 1024, 256, 256, 4, 16, 8, BF16),    # four tiles a program, sixteen K-steps each
    (2048, 1024, 2368, 256, 256, 6, 32, 8, BF16),    # K-steps: 37
    (1000, 700, 2088, 256, 256, 6, 8, 8, BF16),      # ragged M and N, a last K-step of 40
    (1000, 700, 2088, 256, 256, 2, 8, 1, F16),       # one XCD: the share is the whole grid's
    (1024, 1536, 2048, 256, 128, 6, 24, 8, BF16),    # the caller's tiles in twos
    (1024, 1536, 2048, 128, 128, 6, 24, 8, F16),     # ... in fours
    (768, 512, 448, 256, 256, 1, 6, 2, BF16),        # seven K-steps: two lean ones
    (768, 512, 320, 256, 256, 1, 6, 2, BF16),        # five K-steps: none
]


@pytest.mark.parametrize("M,N,K,BM,BN,G,grid,xcds,dtype", CASES)
def test_touching_build_gives_the_plain_builds_bits(shmem, M, N, K, BM, BN, G, grid, xcds, dtype):
    A, B = make_ab(M, N, K, dtype)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    out = {}
    for touch in (ops.TOUCH_OFF, ops.TOUCH_ON):
        cg = shmem.full((M, N), 7, dtype=dtype)
        flags = shmem.zeros((total + 3,), dtype=torch.int32)
        args = (a, b, None, cg, flags, shmem.get_heap_bases(), 0, 1, grid, BM, BN, 64, G, ops.EPI_ALL_SCATTER)
        kw = dict(num_xcds=xcds, touch_ahead=touch)
        name = ops.gemm_plan_name(*args, **kw)
        assert name.startswith("256x256x64_w2x4_s2")
        assert name.endswith("+touch_ahead") == (touch == ops.TOUCH_ON), name
        ops.gemm_launch(*args, **kw)
        torch.cuda.synchronize()
        assert flags.cpu().tolist() == [1] * total + [0, 0, 0]
        out[touch] = cg.clone()
    assert torch.equal(out[ops.TOUCH_ON], out[ops.TOUCH_OFF])
    check_close(out[ops.TOUCH_ON], O.shard_gemm(A, B, dtype), "touching build")


def test_touching_build_with_virtual_ranks_and_fp32_partials(shmem):
    """All-scatter to two ranks, and the one-shot producer's fp32 partial behind
    flags on the other rank, both with the touches forced."""
    ws, M, N, K, BM, BN, G = 2, 1024, 1024, 2304, 256, 256, 4
    A, B = make_ab(M, N, K, BF16)
    shards = O.n_shards(A, B, ws)
    a = to_heap(shmem, A)
    bs = [to_heap(shmem, sb) for _, sb in shards]
    cg = shmem.zeros((M, N), dtype=BF16)
    n_local = N // ws
    total = ops.cdiv(M, BM) * ops.cdiv(n_local, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    for r in range(ws):
        shmem.on_rank(cg, r).zero_()
        shmem.on_rank(flags, r).zero_()
    for r in range(ws):
        args = (a, bs[r], None, shmem.on_rank(cg, r), shmem.on_rank(flags, r), shmem.get_heap_bases(), r, ws, 64, BM,
                BN, 64, G, ops.EPI_ALL_SCATTER)
        assert ops.gemm_plan_name(*args, num_xcds=8, touch_ahead=ops.TOUCH_ON).endswith("+touch_ahead")
        ops.gemm_launch(*args, num_xcds=8, touch_ahead=ops.TOUCH_ON)
    torch.cuda.synchronize()
    want = O.all_scatter(shards, BF16)
    for r in range(ws):
        check_close(shmem.on_rank(cg, r), want, f"rank {r}")
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws] * total

    # the producer of the one-shot all-reduce on rank 0's K shard
    ks = O.k_shards(A, B, ws)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    kk = K // ws
    part = shmem.zeros((M, N), dtype=F32)
    cg2 = shmem.zeros((M, N), dtype=BF16)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags2 = shmem.zeros((total,), dtype=torch.int32)
    got, raised = {}, {}
    for touch in (ops.TOUCH_OFF, ops.TOUCH_ON):
        shmem.on_rank(part, 0).zero_()
        for r in range(ws):
            shmem.on_rank(flags2, r).zero_()
        args = (a_full[:, :kk], b_full[:kk, :], shmem.on_rank(part, 0), shmem.on_rank(cg2, 0),
                shmem.on_rank(flags2, 0), shmem.get_heap_bases(), 0, ws, 64, BM, BN, 64, G, ops.EPI_ONE_SHOT)
        kw = dict(num_xcds=8, phase=ops.PHASE_PRODUCE, touch_ahead=touch)
        assert ops.gemm_plan_name(*args, **kw).endswith("+touch_ahead") == (touch == ops.TOUCH_ON)
        ops.gemm_launch(*args, **kw)
        torch.cuda.synchronize()
        got[touch] = shmem.on_rank(part, 0).clone()
        raised[touch] = [shmem.on_rank(flags2, r).cpu().tolist() for r in range(ws)]
    assert torch.equal(got[ops.TOUCH_ON], got[ops.TOUCH_OFF])
    check_close(got[ops.TOUCH_ON], O.shard_gemm(*ks[0], F32), "producer's partial")
    assert raised[ops.TOUCH_ON] == raised[ops.TOUCH_OFF] and raised[ops.TOUCH_ON][1] == [1] * total


def test_the_launcher_takes_the_touching_build_where_a_round_streams_from_hbm():
    """The choice by shape (no launch): [8192, K] x [K, n] shards of the
    reference's sweep in 256 x 256 tiles on 256 programs and 8 XCDs."""
    dev = torch.device("cuda")

    def plan(n, k, bm=256, bn=256, g=6, touch=ops.TOUCH_AUTO, epilogue=ops.EPI_ALL_SCATTER):
        a = torch.empty((8192, k), dtype=BF16, device=dev)
        bt = torch.empty((n, k), dtype=BF16, device=dev)
        cg = torch.empty((8192, n), dtype=BF16, device=dev)
        flags = torch.zeros((ops.cdiv(8192, bm) * ops.cdiv(n, bn),), dtype=torch.int32, device=dev)
        return ops.gemm_plan_name(a, bt.T, None, cg, flags, None, 0, 1, 256, bm, bn, 64, g, epilogue, num_xcds=8,
                                  touch_ahead=touch)

    assert plan(2048, 14336) == "256x256x64_w2x4_s2+touch_ahead"       # 294 MB in one round
    assert plan(2048, 12288) == "256x256x64_w2x4_s2"                   # 252 MB: stays in the last-level cache
    assert plan(4096, 28672, bn=128) == "256x256x64_w2x4_s2+two_tiles_each+touch_ahead"  # 352 MB a round
    assert plan(4096, 14336, bn=128) == "256x256x64_w2x4_s2+two_tiles_each"              # 176 MB a round
    assert plan(8192, 1024) == "256x256x64_w2x4_s2"                    # the headline launch
    assert plan(4096, 28672, g=2) == "256x256x64_w2x4_s2"              # an XCD's tiles in two rows of sixteen
    assert plan(2048, 14336, touch=ops.TOUCH_OFF) == "256x256x64_w2x4_s2"
    assert plan(2048, 12288, touch=ops.TOUCH_ON) == "256x256x64_w2x4_s2+touch_ahead"
    # a tile without such a build ignores the request
    assert "touch_ahead" not in plan(512, 14336, bn=128, touch=ops.TOUCH_ON)
    with pytest.raises(ValueError):
        plan(2048, 14336, touch=7)


def test_a_streaming_shard_with_the_touches_chosen_by_the_launcher(shmem):
    """[8192, 14336] x [14336, 2048], the sweep's two-GPU all-scatter shard, as
    the launcher runs it by default (touching build), against the plain build's
    bits and, through the product's linearity in A, against itself: C(A) and
    C(2A) differ by exactly a factor of two in bf16."""
    M, N, K = 8192, 2048, 14336
    g = torch.Generator(device="cuda").manual_seed(11)
    a = shmem.zeros((M, K), dtype=BF16)
    bt = shmem.zeros((N, K), dtype=BF16)
    a.copy_(torch.randn((M, K), generator=g, device="cuda", dtype=torch.float32) * 0.02)
    bt.copy_(torch.randn((N, K), generator=g, device="cuda", dtype=torch.float32) * 0.02)
    flags = shmem.zeros((32 * 8,), dtype=torch.int32)
    res = {}
    for key, touch, scale in (("auto", ops.TOUCH_AUTO, 1), ("off", ops.TOUCH_OFF, 1), ("twice", ops.TOUCH_AUTO, 2)):
        cg = shmem.zeros((M, N), dtype=BF16)
        if scale != 1:
            a.mul_(scale)
        flags.zero_()
        args = (a, bt.T, None, cg, flags, shmem.get_heap_bases(), 0, 1, 256, 256, 256, 64, 6, ops.EPI_ALL_SCATTER)
        kw = dict(num_xcds=8, touch_ahead=touch)
        assert ops.gemm_plan_name(*args, **kw).endswith("+touch_ahead") == (touch == ops.TOUCH_AUTO)
        ops.gemm_launch(*args, **kw)
        torch.cuda.synchronize()
        assert flags.cpu().tolist() == [1] * 256
        res[key] = cg
    assert torch.equal(res["auto"], res["off"])
    assert torch.equal(res["twice"].float(), res["auto"].float() * 2)
    # a sample of rows against fp32 arithmetic on the same operands
    rows = torch.arange(0, M, 97, device="cuda")
    want = (a[rows].float() / 2) @ bt.float().T
    check_close(res["auto"][rows].cpu(), want.cpu(), "sampled rows")
