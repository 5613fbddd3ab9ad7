"""Parity at the sizes the figures are quoted on: the bf16 [8192,1024] x
[1024,8192] K-shard GEMM with flag-published 256x256 tiles, the one-shot
reduce of eight fp32 [8192,8192] partials, the eight-shard atomic accumulate
into fp32 [4096,4096], and the decoder-shaped shards for 1 ... 2048 rows.

Every output element is compared with the oracle: the GEMMs within rtol /
atol 1e-2 of the fp32-accumulated product, flags one by one, the reduce bit
for bit.
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

    # the whole [8192, 8192] product against the oracle
    check_close(cg.cpu(), O.shard_gemm(a.cpu(), b.cpu(), dtype), "headline shard GEMM")


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


def test_atomic_accumulate_of_eight_shards_full_size(shmem):
    """Config 4: eight sequential bf16 K-shard GEMMs [4096,512] x [512,4096]
    adding 256 tiles of 256x256 each into one fp32 C; the whole matrix
    against the oracle."""
    M = N = 4096
    ks, shards, dtype = 512, 8, torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(123)
    a_full = shmem.zeros((M, ks * shards), dtype=dtype)
    bt_full = shmem.zeros((N, ks * shards), dtype=dtype)
    a_full.copy_((torch.randn(M, ks * shards, generator=gen, device="cuda") * 0.05).to(dtype))
    bt_full.copy_((torch.randn(N, ks * shards, generator=gen, device="cuda") * 0.05).to(dtype))
    c = shmem.zeros((M, N), dtype=torch.float32)
    for i in range(shards):
        ops.gemm_launch(a_full[:, i * ks:(i + 1) * ks], bt_full[:, i * ks:(i + 1) * ks].T, None, c, None,
                        shmem.get_heap_bases(), 0, 1, 256, 256, 256, 64, 6, ops.EPI_ATOMIC_ADD, num_xcds=8)
    torch.cuda.synchronize()
    A, B = a_full.cpu(), bt_full.cpu().T
    check_close(c.cpu(), O.atomics_all_reduce(O.k_shards(A, B, shards)), "atomic accumulate")


@pytest.mark.parametrize("M", [1, 16, 128, 512, 2048])
def test_decoder_shards_full_size(shmem, M):
    """Config 5: gate/up [M,4096] x [4096,1376] scattered to 8 ranks at column
    rank*1376, down [M,1376] x [1376,4096] as an fp32 partial on each of the 8
    ranks, then the one-shot reduce: against the oracle, whole matrices."""
    ws, hidden, ffn, dtype = 8, 4096, 1376, torch.bfloat16
    BM, BN = (64, 64) if M <= 128 else (128, 128)
    g = torch.Generator().manual_seed(123)
    X = (torch.randn(M, hidden, generator=g) * 0.02).to(dtype)
    Wg = (torch.randn(ws, ffn, hidden, generator=g) * 0.02).to(dtype)   # one shard per rank
    H = (torch.randn(ws, M, ffn, generator=g) * 0.02).to(dtype)
    Wd = (torch.randn(ws, hidden, ffn, generator=g) * 0.02).to(dtype)
    x = shmem.zeros((M, hidden), dtype=dtype)
    wg = shmem.zeros((ffn, hidden), dtype=dtype)
    h = shmem.zeros((M, ffn), dtype=dtype)
    wd = shmem.zeros((hidden, ffn), dtype=dtype)
    gate_all = shmem.zeros((M, ws * ffn), dtype=dtype)
    part = shmem.zeros((M, hidden), dtype=torch.float32)
    out = shmem.zeros((M, hidden), dtype=dtype)
    t_up, t_dn = ops.cdiv(M, BM) * ops.cdiv(ffn, BN), ops.cdiv(M, BM) * ops.cdiv(hidden, BN)
    flags_up = shmem.zeros((t_up,), dtype=torch.int32)
    flags_dn = shmem.zeros((t_dn,), dtype=torch.int32)
    P = shmem.zeros((256, BM * BN), dtype=torch.float32)
    locks = shmem.zeros((256,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    for r in range(ws):
        for t, src in ((x, X), (wg, Wg[r]), (h, H[r]), (wd, Wd[r])):
            shmem.on_rank(t, r).copy_(src)
        for t in (gate_all, part, out, flags_up, flags_dn, P, locks):
            shmem.on_rank(t, r).zero_()
    on = shmem.on_rank
    for r in range(ws):
        ops.gemm_launch(on(x, r), on(wg, r).T, None, on(gate_all, r), on(flags_up, r), hb, r, ws, 256, BM, BN, 64, 4,
                        ops.EPI_ALL_SCATTER, partials=on(P, r), locks=on(locks, r), num_xcds=8)
        ops.gemm_launch(on(h, r), on(wd, r).T, on(part, r), on(out, r), on(flags_dn, r), hb, r, ws, 256, BM, BN, 64, 6,
                        ops.EPI_ONE_SHOT, phase=ops.PHASE_PRODUCE, partials=on(P, r), locks=on(locks, r), num_xcds=8)
    for r in range(ws):
        ops.one_shot_reduce(on(part, r), on(out, r), on(flags_dn, r), hb, r, ws, BM, BN, 6)
    torch.cuda.synchronize()
    up = O.all_scatter([(X, Wg[r].T) for r in range(ws)], dtype)
    dn = O.one_shot_all_reduce([(H[r], Wd[r].T) for r in range(ws)], torch.float32, dtype)
    for r in (0, 5, 7):
        check_close(on(gate_all, r).cpu(), up, f"gate/up on rank {r}")
        check_close(on(out, r).cpu(), dn, f"down + reduce on rank {r}")
        assert on(flags_up, r).cpu().tolist() == [ws] * t_up
        assert on(flags_dn, r).cpu().tolist() == [0] * t_dn
        assert not on(locks, r).any()
