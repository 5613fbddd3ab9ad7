"""The one-shot reduce kernel (consumer half of the 09 epilogue) against the
oracle: bit-exact values for a fixed rank order, bit-exact flags."""

import pytest
import torch

from iris_amd import ops
from oracle import iris_oracle as O

pytestmark = pytest.mark.gpu


def fill_partials(shmem, c, ws, seed=123, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    host = (torch.randn(ws, *c.shape, generator=g) * scale).to(c.dtype)
    for r in range(ws):
        shmem.on_rank(c, r).copy_(host[r])
    return host


def signal_all(shmem, flags, total, ws):
    for r in range(ws):
        shmem.on_rank(flags, r).zero_()
    for r in range(ws):
        ops.signal_tiles(shmem.on_rank(flags, r), shmem.get_heap_bases(), total, r, ws)


@pytest.mark.parametrize("variant", range(0, 9))  # 1-6: tile-kernel tuning points, 7: row bands, 8: tiles
def test_eight_fp32_partials_to_bf16_is_bit_exact(shmem, variant):
    M, N, BM, BN, ws = 1024, 768, 256, 256, 8
    c = shmem.zeros((M, N), dtype=torch.float32)
    cg = shmem.zeros((M, N), dtype=torch.bfloat16)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    host = fill_partials(shmem, c, ws)
    signal_all(shmem, flags, total, ws)
    torch.cuda.synchronize()
    for r in range(ws):
        assert shmem.on_rank(flags, r).cpu().tolist() == [ws - 1] * total
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.one_shot_reduce(c, cg, flags, shmem.get_heap_bases(), 0, ws, BM, BN, 6, variant=variant, status=status)
    torch.cuda.synchronize()
    assert torch.equal(cg.cpu(), O.one_shot_reduce(host, torch.bfloat16))
    assert flags.cpu().tolist() == [0] * total              # consumed: reset to 0
    assert shmem.on_rank(flags, 1).cpu().tolist() == [ws - 1] * total  # other ranks' flags untouched
    assert int(status.item()) == 0


@pytest.mark.parametrize("in_dt,out_dt,ws,M,N,BM,BN,grid", [
    (torch.float32, torch.float16, 4, 300, 264, 128, 64, 0),
    (torch.float32, torch.float32, 2, 130, 72, 64, 64, 3),
    (torch.bfloat16, torch.bfloat16, 8, 512, 256, 256, 64, 256),
    (torch.bfloat16, torch.float32, 3, 96, 40, 32, 32, 0),
    (torch.float16, torch.float16, 5, 257, 136, 256, 128, 2),
    (torch.float32, torch.bfloat16, 8, 77, 50, 64, 64, 0),      # N not a multiple of 8: element-wise kernel
    (torch.float32, torch.bfloat16, 1, 128, 128, 64, 64, 0),    # one rank: plain cast, no flags
    (torch.float16, torch.bfloat16, 2, 64, 64, 64, 64, 0),      # no vector kernel for this pair
])
@pytest.mark.parametrize("variant", [0, 7])
def test_reduce_shapes_types_and_ragged_tiles(shmem, in_dt, out_dt, ws, M, N, BM, BN, grid, variant):
    c = shmem.zeros((M, N), dtype=in_dt)
    cg = shmem.full((M, N), 3, dtype=out_dt)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    host = fill_partials(shmem, c, ws, seed=M * 7 + N)
    signal_all(shmem, flags, total, ws)
    ops.one_shot_reduce(c, cg, flags, shmem.get_heap_bases(), 0, ws, BM, BN, 4, num_sms=grid,
                        num_xcds=8 if grid == 256 else 1, variant=variant)
    torch.cuda.synchronize()
    assert torch.equal(cg.cpu(), O.one_shot_reduce(host, out_dt))
    assert flags.cpu().tolist() == [0] * total


@pytest.mark.parametrize("variant", [0, 7])
def test_reduce_on_a_middle_rank_and_strided_buffers(shmem, variant):
    M, N, ws = 192, 160, 4
    wide = shmem.zeros((M, N + 32), dtype=torch.float32)
    c = wide[:, 16:16 + N]  # a view: row stride N+32, 64-byte column offset
    cg_wide = shmem.zeros((M, N + 8), dtype=torch.bfloat16)
    cg = cg_wide[:, 8:]
    total = ops.cdiv(M, 64) * ops.cdiv(N, 32)
    flags = shmem.zeros((total,), dtype=torch.int32)
    g = torch.Generator().manual_seed(3)
    host = torch.randn(ws, M, N, generator=g)
    for r in range(ws):
        shmem.on_rank(wide, r).zero_()
        shmem.on_rank(c, r).copy_(host[r])
        shmem.on_rank(cg_wide, r).zero_()
    signal_all(shmem, flags, total, ws)
    rank = 2
    ops.one_shot_reduce(shmem.on_rank(c, rank), shmem.on_rank(cg, rank), shmem.on_rank(flags, rank),
                        shmem.get_heap_bases(), rank, ws, 64, 32, 2, variant=variant)
    torch.cuda.synchronize()
    assert torch.equal(shmem.on_rank(cg, rank).cpu(), O.one_shot_reduce(host, torch.bfloat16))
    assert float(shmem.on_rank(cg_wide, rank)[:, :8].float().abs().max()) == 0.0
    assert shmem.on_rank(flags, rank).cpu().tolist() == [0] * total
    assert flags.cpu().tolist() == [ws - 1] * total


@pytest.mark.parametrize("variant", [0, 7])
def test_only_signalled_tiles_are_reduced_and_the_wait_is_bounded(shmem, variant):
    """Flags gate tiles one by one: with every third tile signalled, exactly
    those tiles' regions (per the oracle's tile map) are written; the others
    time out, are reported and are left alone."""
    M, N, BM, BN, G, ws = 512, 384, 128, 64, 3, 2
    c = shmem.zeros((M, N), dtype=torch.float32)
    cg = shmem.full((M, N), -7, dtype=torch.float32)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    host = fill_partials(shmem, c, ws)
    ready = [t for t in range(total) if t % 3 == 0]
    f = torch.zeros(total, dtype=torch.int32)
    f[ready] = ws - 1
    flags.copy_(f)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.one_shot_reduce(c, cg, flags, shmem.get_heap_bases(), 0, ws, BM, BN, G, status=status,
                        spin_timeout_ticks=1000, variant=variant)
    torch.cuda.synchronize()
    want = torch.full((M, N), -7.0)
    full = O.one_shot_reduce(host, torch.float32)
    for t in ready:
        pm, pn = O.tile_map(t, M, N, BM, BN, G)
        want[pm * BM:(pm + 1) * BM, pn * BN:(pn + 1) * BN] = full[pm * BM:(pm + 1) * BM, pn * BN:(pn + 1) * BN]
    assert torch.equal(cg.cpu(), want)
    assert int(status.item()) == 1
    assert flags.cpu().tolist() == [0] * total


def test_reduce_without_flag_wait_is_a_plain_sum(shmem):
    M, N, ws = 256, 256, 8
    c = shmem.zeros((M, N), dtype=torch.float32)
    cg = shmem.zeros((M, N), dtype=torch.bfloat16)
    host = fill_partials(shmem, c, ws)
    ops.one_shot_reduce(c, cg, None, shmem.get_heap_bases(), 0, ws, 256, 256, 1, wait_flags=False)
    torch.cuda.synchronize()
    assert torch.equal(cg.cpu(), O.one_shot_reduce(host, torch.bfloat16))


def test_signal_include_self_and_memset(shmem):
    import iris_amd

    ws, total = 4, 37
    flags = shmem.zeros((total,), dtype=torch.int32)
    for r in range(ws):
        iris_amd.memset_tensor(shmem.on_rank(flags, r), 10 + r)
    ops.signal_tiles(shmem.on_rank(flags, 2), shmem.get_heap_bases(), total, 2, ws, include_self=True)
    ops.signal_tiles(shmem.on_rank(flags, 0), shmem.get_heap_bases(), total - 5, 0, ws)
    torch.cuda.synchronize()
    for r in range(ws):
        want = [10 + r + 1 + (1 if (r != 0 and t < total - 5) else 0) for t in range(total)]
        assert shmem.on_rank(flags, r).cpu().tolist() == want
    big = shmem.zeros((5000,), dtype=torch.int32)
    iris_amd.memset_tensor(big[3:4999], -2)
    torch.cuda.synchronize()
    assert big.cpu().tolist() == [0, 0, 0] + [-2] * 4996 + [0]
