"""The flag protocol with the producer and the consumer resident at the same
time: rank r's shard GEMM publishes tiles from one stream while rank 0's
reduce kernel, enqueued on another stream without any synchronisation in
between, polls the tiles' flags and reads the partials as they arrive.

Every wait is bounded (spin_timeout_ticks), so a scheduling miss shows up as
status 1 and every kernel still exits.  A GEMM workgroup takes a whole CU
(all of its LDS and registers), so the producers run on 128 programs and the
consumer on 128 blocks: both fit the chip at once whichever starts first.
The consumer is enqueued first, so it is polling before the first tile exists.
"""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O

from parity import default_scale
from test_gemm_gpu import check_close, make_ab, to_heap

pytestmark = pytest.mark.gpu

HALF_SECOND = 50_000_000  # ticks of the 100 MHz wall clock


@pytest.fixture(scope="module")
def two_streams(shmem_gpu):
    """Two streams that really run side by side.  HIP maps streams onto a few
    hardware queues, and two streams that share a queue run one after the
    other; so candidates are probed with the protocol itself: a one-tile
    consumer (bounded wait, 20 ms) on one stream, then the signal it waits for
    on the other.  The pair is kept for the whole module."""
    shmem = shmem_gpu
    shmem.heap_offset = 0
    ws = 2
    c = shmem.zeros((64, 64), dtype=torch.float32)
    cg = shmem.zeros((64, 64), dtype=torch.float32)
    flags = shmem.zeros((1,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    streams = [torch.cuda.Stream() for _ in range(4)]
    for s in streams:  # the first submission to a new stream takes milliseconds
        with torch.cuda.stream(s):
            torch.zeros(8, device="cuda").add_(1)
    torch.cuda.synchronize()
    for sb in streams:
        for sa in streams:
            if sa is sb:
                continue
            for r in range(ws):
                shmem.on_rank(flags, r).zero_()
            status.zero_()
            torch.cuda.synchronize()
            with torch.cuda.stream(sb):
                ops.one_shot_reduce(c, cg, flags, hb, 0, ws, 64, 64, 1, num_sms=1, variant=8, status=status,
                                    spin_timeout_ticks=2_000_000)
            with torch.cuda.stream(sa):
                ops.signal_tiles(shmem.on_rank(flags, 1), hb, 1, 1, ws)
            torch.cuda.synchronize()
            if int(status.item()) == 0:
                return sa, sb
    pytest.fail("no two streams of this process run side by side on the device")


# Concurrent passes per parametrisation, each on fresh operands.  Every wait is bounded and every kernel exits;
# the loop stops at the first mismatch or timeout.
ROUNDS = 50


@pytest.mark.parametrize("flag_sem", [ops.FLAG_SEM_WRITE_THROUGH, ops.FLAG_SEM_RELEASE_ACQUIRE])
@pytest.mark.parametrize("scope", [ops.SCOPE_AGENT, ops.SCOPE_SYSTEM])
@pytest.mark.parametrize("variant", [7, 8])  # row bands, tiles
@pytest.mark.parametrize("ws", [2, 4])
def test_one_shot_consumer_polls_while_producers_publish(shmem, two_streams, ws, variant, scope, flag_sem):
    """09 split in two kernels: ranks 1..ws-1 produce (partial tile stores +
    flag +1 on rank 0) while rank 0's consumer is already waiting.  With the
    default flag semantics (write-through stores, relaxed flag) and with the
    reference's release / acquire."""
    M = N = 4096
    K, BM, BN, G = 2048, 128, 128, 6
    dtype = torch.bfloat16
    A, B = make_ab(M, N, K * ws, dtype, seed=ws * 10 + variant)
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    c = shmem.zeros((M, N), dtype=torch.float32)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)  # 1024 tiles
    flags = shmem.zeros((total,), dtype=torch.int32)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    hb = shmem.get_heap_bases()
    on = shmem.on_rank
    scale = float(A.float().std())

    def clear():
        for r in range(ws):
            for t in (c, cg, flags):
                on(t, r).zero_()

    def produce(r, grid):
        ops.gemm_launch(a_full[:, r * K:(r + 1) * K], b_full[r * K:(r + 1) * K, :], on(c, r), on(cg, r),
                        on(flags, r), hb, r, ws, grid, BM, BN, 64, G, ops.EPI_ONE_SHOT, phase=ops.PHASE_PRODUCE,
                        num_xcds=8, scope=scope, status=status, flag_sem=flag_sem)

    def consume():
        ops.one_shot_reduce(c, cg, flags, hb, 0, ws, BM, BN, G, num_sms=128, num_xcds=8, scope=scope,
                            variant=variant, status=status, spin_timeout_ticks=HALF_SECOND, flag_sem=flag_sem)

    sa, sb = two_streams
    zeros = torch.zeros(total, dtype=torch.int32, device="cuda")
    others = torch.full((total,), ws - 1, dtype=torch.int32, device="cuda")
    leads = []
    for it in range(ROUNDS):
        if it > 0:  # fresh operands, drawn on the device
            a_full.normal_(0, scale)
        # one pass in stream order first: the result of these operands is known (and every kernel is loaded)
        clear()
        for r in range(ws):
            produce(r, 128)
        consume()
        torch.cuda.synchronize()
        want = cg.clone()
        assert int(status.item()) == 0 and torch.equal(flags, zeros), f"round {it}, stream order"
        # A consumer that reads a partial before it is complete must find something else there: zeros
        clear()
        # rank 0's own partial is stream-ordered before its consumer, as in the reference program
        produce(0, 256)
        torch.cuda.synchronize()
        cons_begin, cons_end, prod_end = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        # the consumer goes first: its 128 blocks leave at least 128 CUs empty for the producers' 128 programs
        with torch.cuda.stream(sb):
            cons_begin.record()
            consume()
            cons_end.record()
        with torch.cuda.stream(sa):
            for r in range(1, ws):
                produce(r, 128)
            prod_end.record()
        torch.cuda.synchronize()
        assert int(status.item()) == 0, f"round {it}: a flag wait timed out: the kernels did not overlap as planned"
        # the consumer was on the device before the producers were done, and cannot have finished before them
        lead, lag = cons_begin.elapsed_time(prod_end), prod_end.elapsed_time(cons_end)
        leads.append((lead, lag))
        assert lead > 0, f"round {it}: the consumer started after the producers had finished: nothing was polled"
        assert torch.equal(cg, want), f"round {it}: the concurrent pass differs from the pass in stream order"
        assert torch.equal(flags, zeros), f"round {it}: flags not consumed"
        for r in range(1, ws):  # the other ranks' flags: +1 from everyone but themselves, never consumed
            assert torch.equal(on(flags, r), others), f"round {it}: flags of rank {r}"
        if it in (0, ROUNDS - 1):
            # against the oracle: the rank-ordered sum of the partials, bit for bit, and the closed form
            partials = torch.stack([on(c, r).cpu() for r in range(ws)])
            assert torch.equal(cg.cpu(), O.one_shot_reduce(partials, dtype)), "not the rank-ordered sum"
            Ah, Bh = a_full.cpu(), b_full.cpu()
            check_close(cg, O.one_shot_all_reduce(O.k_shards(Ah, Bh, ws), torch.float32, dtype), "vs closed form")
    lead, lag = leads[-1]
    print(f"{ROUNDS} rounds; last: consumer enqueued {lead * 1e3:.0f} us before the producers finished, "
          f"done {lag * 1e3:.0f} us after them")


@pytest.mark.parametrize("scope", [ops.SCOPE_AGENT, ops.SCOPE_SYSTEM])
def test_scatter_ready_flags_gate_a_concurrent_reader(shmem, two_streams, scope):
    """07 with ready flags (flag_mode 1): rank 1 scatters its column block to
    both ranks and raises each tile's flag on both; a reader on rank 0,
    already polling, sums rank 0's and rank 1's copy of each tile as soon as the
    flag is up.  Both copies hold the same tile, so the sum is exactly twice it."""
    ws, M, NL, K, BM, BN, G = 2, 4096, 2048, 2048, 128, 128, 4
    dtype = torch.bfloat16
    A, B = make_ab(M, NL, K, dtype, seed=5)
    a, b = to_heap(shmem, A), to_heap(shmem, B)
    cg = shmem.zeros((M, NL * ws), dtype=dtype)
    out = shmem.zeros((M, NL), dtype=torch.float32)
    total = ops.cdiv(M, BM) * ops.cdiv(NL, BN)  # 512 tiles
    flags = shmem.zeros((total,), dtype=torch.int32)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    hb = shmem.get_heap_bases()
    on = shmem.on_rank
    for r in range(ws):
        on(cg, r).zero_()
        on(flags, r).zero_()
    def produce():
        ops.gemm_launch(a, b, None, on(cg, 1), on(flags, 1), hb, 1, ws, 128, BM, BN, 64, G, ops.EPI_ALL_SCATTER,
                        num_xcds=8, scope=scope)

    def consume():
        # rank 1's block of c_global, as rank 0 sees it; a flag that reads ws-1 == 1 means "tile stored"
        ops.one_shot_reduce(cg[:, NL:], out, flags, hb, 0, ws, BM, BN, G, num_sms=128, num_xcds=8, scope=scope,
                            variant=8, status=status, spin_timeout_ticks=HALF_SECOND)

    produce()  # in stream order first: the kernels are loaded
    consume()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    for r in range(ws):
        on(cg, r).zero_()
        on(flags, r).zero_()
    out.zero_()
    torch.cuda.synchronize()
    sa, sb = two_streams
    cons_begin, prod_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(sb):
        cons_begin.record()
        consume()
    with torch.cuda.stream(sa):
        produce()
        prod_end.record()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert cons_begin.elapsed_time(prod_end) > 0, "the reader started after the producer had finished"
    want = O.shard_gemm(A, B, dtype)
    check_close(cg[:, NL:], want, "scattered block on rank 0")
    assert torch.equal(on(cg, 1)[:, NL:].cpu(), cg[:, NL:].cpu())
    assert torch.equal(out.cpu(), cg[:, NL:].float().cpu() * 2), "reader saw a tile before its stores"
    assert flags.cpu().tolist() == [0] * total and on(flags, 1).cpu().tolist() == [1] * total


@pytest.mark.parametrize("flag_sem", [ops.FLAG_SEM_WRITE_THROUGH, ops.FLAG_SEM_RELEASE_ACQUIRE])
@pytest.mark.parametrize("scope", [ops.SCOPE_AGENT, ops.SCOPE_SYSTEM])
@pytest.mark.parametrize("M,N,K,BM,BN,partial_dtype", [
    (4096, 4096, 512, 256, 256, torch.float32),   # 256 tiles, two per program, one compute tile each
    (4096, 4096, 512, 256, 256, torch.bfloat16),
    (2048, 3072, 1024, 128, 128, torch.float32),  # 384 tiles, three per program
    (1000, 1160, 328, 128, 128, torch.bfloat16),  # ragged M, N and K; 16-byte strips still fit
    (520, 388, 264, 64, 64, torch.float32),       # ragged, 63 tiles on 128 programs
    (300, 250, 136, 128, 64, torch.float32),      # N no multiple of four: the element-wise reduce
])
def test_one_shot_inside_the_program_two_ranks_side_by_side(shmem, two_streams, M, N, K, BM, BN, partial_dtype,
                                                            scope, flag_sem):
    """IRIS_PHASE_FUSED, the reference program's own order
    (gemm_one_shot_all_reduce.py:197-271): each program stores its partial
    tile, signals the other rank, waits for the tile's flag on its own rank,
    sums the tile over both ranks and stores it, tile by tile.  Two ranks of
    128 programs each share the 256 CUs, one stream per rank.  ROUNDS passes,
    each on fresh operands."""
    ws, G = 2, 6
    dtype = torch.bfloat16
    # 16-bit partials round at 2^-9 of their own size, which can be more than the tolerance allows the (smaller)
    # sum when two large partials cancel: those cases keep their partials well below 1
    shrink = 0.3 if partial_dtype != torch.float32 else 1.0
    A, B = make_ab(M, N, K * ws, dtype, seed=M + N, scale=shrink * default_scale(K * ws))
    a_full, b_full = to_heap(shmem, A), to_heap(shmem, B)
    c = shmem.zeros((M, N), dtype=partial_dtype)
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    hb = shmem.get_heap_bases()
    on = shmem.on_rank
    for r in range(ws):
        for t in (c, cg, flags):
            on(t, r).zero_()

    def launch(r):
        args = (a_full[:, r * K:(r + 1) * K], b_full[r * K:(r + 1) * K, :], on(c, r), on(cg, r), on(flags, r), hb, r,
                ws, 128, BM, BN, 64, G, ops.EPI_ONE_SHOT)
        kw = dict(phase=ops.PHASE_FUSED, num_xcds=8)
        assert ops.gemm_plan_name(*args, **kw).endswith("+reduce")
        ops.gemm_launch(*args, status=status, spin_timeout_ticks=HALF_SECOND, scope=scope, flag_sem=flag_sem, **kw)

    scale = float(A.float().std())
    zeros = torch.zeros(total, dtype=torch.int32, device="cuda")
    for it in range(ROUNDS):
        if it > 0:  # fresh operands, drawn on the device; the partials of the round before are still in `c`
            a_full.normal_(0, scale)
        torch.cuda.synchronize()
        for r, s in enumerate(two_streams):
            with torch.cuda.stream(s):
                launch(r)
        torch.cuda.synchronize()
        assert int(status.item()) == 0, f"round {it}: a program gave up waiting for its peer"
        # two ranks: the rank-ordered fp32 sum is one addition, which the device computes to the same bits
        want_dev = (on(c, 0).float() + on(c, 1).float()).to(dtype)
        for r in range(ws):
            assert torch.equal(on(cg, r), want_dev), f"round {it}, rank {r}: not the sum of the partials"
            assert torch.equal(on(flags, r), zeros), f"round {it}, rank {r}: flags"  # up once, consumed
        if it in (0, ROUNDS - 1):
            partials = torch.stack([on(c, r).cpu() for r in range(ws)])
            shards = O.k_shards(a_full.cpu(), b_full.cpu(), ws)
            for r in range(ws):
                check_close(partials[r], O.shard_gemm(*shards[r], partial_dtype), f"partial of rank {r}")
            want = O.one_shot_reduce(partials, dtype)
            for r in range(ws):
                assert torch.equal(on(cg, r).cpu(), want), f"rank {r}: not the rank-ordered sum of the partials"
            check_close(cg, O.one_shot_all_reduce(shards, partial_dtype, dtype), "vs closed form")
