"""Pins of the CPU oracle (oracle/iris_oracle.py).

Each oracle function is checked against something other than its own
formula: invariants, hand-derived values, an independent construction, a
library routine or a higher-precision computation.
"""

import itertools

import numpy as np
import pytest
import torch

from oracle import iris_oracle as O


# --------------------------------------------------------------------------- tile map
def grouped_order_by_enumeration(M, N, BM, BN, G):
    """Independent construction of the grouped tile order: walk groups of G
    block-rows; inside a group go column by column, rows fastest."""
    npm, npn = O.cdiv(M, BM), O.cdiv(N, BN)
    order = []
    for first in range(0, npm, G):
        rows = range(first, min(first + G, npm))
        for pn in range(npn):
            for pm in rows:
                order.append((pm, pn))
    return order


SHAPES = [
    (8192, 8192, 256, 256, 4), (8192, 8192, 256, 256, 6), (768, 512, 256, 128, 6), (4096, 4096, 256, 256, 6),
    (2048, 1376, 256, 256, 4), (1, 1376, 256, 64, 4), (16, 4096, 128, 128, 1), (1000, 999, 64, 64, 8),
    (8192, 4608, 256, 64, 4), (257, 255, 256, 256, 3), (5 * 128, 7 * 64, 128, 64, 2),
]


@pytest.mark.parametrize("M,N,BM,BN,G", SHAPES)
def test_tile_map_matches_enumeration_and_is_bijective(M, N, BM, BN, G):
    total = O.cdiv(M, BM) * O.cdiv(N, BN)
    got = [O.tile_map(t, M, N, BM, BN, G) for t in range(total)]
    assert got == grouped_order_by_enumeration(M, N, BM, BN, G)
    assert len(set(got)) == total
    assert all(0 <= pm < O.cdiv(M, BM) and 0 <= pn < O.cdiv(N, BN) for pm, pn in got)
    assert (O.tile_map_all(M, N, BM, BN, G) == np.array(got, dtype=np.int32)).all()


def test_tile_map_hand_values():
    # hand-derived: 32x32 tile grid, groups of G block-rows, rows cycle fastest
    f = lambda t, g: O.tile_map(t, 8192, 8192, 256, 256, g)
    assert [f(t, 4) for t in range(8)] == [(0, 0), (1, 0), (2, 0), (3, 0), (0, 1), (1, 1), (2, 1), (3, 1)]
    assert [f(t, 6) for t in range(8)] == [(0, 0), (1, 0), (2, 0), (3, 0), (4, 0), (5, 0), (0, 1), (1, 1)]
    # last group of G=6 on 32 block-rows holds 32 - 30 = 2 rows
    assert f(30 * 32, 6) == (30, 0) and f(30 * 32 + 1, 6) == (31, 0) and f(30 * 32 + 2, 6) == (30, 1)
    # fewer block-rows than G: the only group shrinks to num_pid_m
    g = lambda t: O.tile_map(t, 768, 512, 256, 128, 6)
    assert [g(t) for t in range(8)] == [(0, 0), (1, 0), (2, 0), (0, 1), (1, 1), (2, 1), (0, 2), (1, 2)]
    assert O.tile_index_range(5, 768, 512, 256, 128, 6) == (2 * 256, 1 * 128)


@pytest.mark.parametrize("num_sms,x", [(256, 8), (288, 8), (304, 8), (304, 1), (64, 4), (8, 8)])
def test_xcd_remap_is_a_permutation_that_groups_by_xcd(num_sms, x):
    img = [O.xcd_remap(p, num_sms, x) for p in range(num_sms)]
    assert sorted(img) == list(range(num_sms))
    if x > 1:
        per = num_sms // x
        # hardware deals workgroup p to XCD p % x: every XCD gets one contiguous block of remapped ids
        for xcd in range(x):
            ids = sorted(img[p] for p in range(num_sms) if p % x == xcd)
            assert ids == list(range(xcd * per, (xcd + 1) * per))


@pytest.mark.parametrize("total,num_sms,x", [(1024, 256, 8), (1024, 288, 8), (1000, 304, 8), (7, 256, 8), (300, 256, 1)])
def test_program_tiles_partition_all_tiles(total, num_sms, x):
    seen = list(itertools.chain.from_iterable(O.program_tiles(p, total, num_sms, x) for p in range(num_sms)))
    assert sorted(seen) == list(range(total))
    for p in range(num_sms):
        t = O.program_tiles(p, total, num_sms, x)
        assert t == sorted(t) and all(b - a == num_sms for a, b in zip(t, t[1:]))


def test_num_xcds_rule_and_streamk_bookkeeping():
    assert O.num_xcds_rule(304) == 8 and O.num_xcds_rule(256) == 1 and O.num_xcds_rule(104) == 1
    s = O.streamk_bookkeeping(8192, 8192, 1024, 256, 256, 64, 256)
    assert s["total_tiles"] == 1024 and s["iters_per_tile"] == 16 and s["even_k"]
    assert s["total_tiles_streamk"] == 0 and s["total_blocking_tiles"] == 1024
    s = O.streamk_bookkeeping(8192, 4608, 36864, 256, 64, 64, 288)
    assert s["total_tiles"] == 32 * 72 and s["total_tiles_streamk"] == 0
    s = O.streamk_bookkeeping(1000, 1000, 100, 256, 256, 64, 7)
    assert s["total_tiles"] == 16 and s["total_tiles_streamk"] == 2 and s["total_iters_streamk"] == 4
    assert s["total_full_tiles_streamk"] == 0 and s["total_partial_tiles_streamk"] == 4 and not s["even_k"]


# --------------------------------------------------------------------------- values
def test_round_to_bf16_bits_matches_torch_bit_for_bit():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(1 << 16, generator=g) * torch.logspace(-20, 20, 1 << 16)
    special = torch.tensor([0.0, -0.0, 1.0, -1.0, float("inf"), -float("inf"), 3.3895314e38, 1e-40, -1e-45,
                            1.00390625, 1.01171875, 1.005859375])  # ties and near-overflow
    x = torch.cat([x, special])
    want = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.round_to_bf16_bits(x.numpy())
    assert (got == want).all()
    # a tie rounds to the even mantissa: 1 + 2^-8 -> 1.0 ; 1 + 3*2^-8 -> 1 + 2^-6
    assert O.round_to_bf16_bits(np.float32([1.00390625]))[0] == 0x3F80
    assert O.round_to_bf16_bits(np.float32([1.01171875]))[0] == 0x3F82
    assert (O.round_to_bf16_bits(np.float32([np.nan])) & 0x7FC0 == 0x7FC0).all()


def test_shard_gemm_against_float64():
    g = torch.Generator().manual_seed(123)
    A = (torch.randn(96, 200, generator=g) * 0.02).to(torch.bfloat16)
    B = (torch.randn(72, 200, generator=g) * 0.02).to(torch.bfloat16).T
    ref64 = A.double() @ B.double()
    acc = O.shard_gemm(A, B, None)
    assert acc.dtype == torch.float32
    assert torch.allclose(acc.double(), ref64, rtol=1e-5, atol=1e-7)
    out = O.shard_gemm(A, B, torch.bfloat16)
    assert out.dtype == torch.bfloat16 and torch.equal(out, acc.to(torch.bfloat16))


@pytest.mark.parametrize("K,BK", [(64, 64), (96, 64), (1376, 64), (100, 32), (7, 64), (129, 64)])
def test_blocked_k_loop_with_ragged_tail_equals_plain_product(K, BK):
    rng = np.random.default_rng(K * 131 + BK)
    A = rng.standard_normal((33, K)).astype(np.float32)
    B = rng.standard_normal((K, 17)).astype(np.float32)
    got = O.blocked_k_gemm(A, B, BK)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-4)
    # a dropped or doubled tail block would change the sum by O(1)
    if K % BK:
        body = O.blocked_k_gemm(A[:, : (K // BK) * BK], B[: (K // BK) * BK], BK) if K >= BK else 0
        assert not np.allclose(body, want, rtol=1e-3, atol=1e-2)


def test_sharding_helpers_and_collective_closed_forms():
    g = torch.Generator().manual_seed(123)
    A = torch.randn(64, 96, generator=g)
    B = torch.randn(80, 96, generator=g).T
    full = A.double() @ B.double()
    ks = O.k_shards(A, B, 4)
    assert all(a.shape == (64, 24) and b.shape == (24, 80) for a, b in ks)
    assert ks[1][0].stride() == (96, 1) and ks[1][1].stride() == (1, 96)  # views keep the full-K leading dimension
    assert torch.allclose(O.atomics_all_reduce(ks).double(), full, atol=1e-4)
    assert torch.allclose(O.one_shot_all_reduce(ks, torch.float32, torch.float32).double(), full, atol=1e-4)
    ns = O.n_shards(A, B, 4)
    assert all(a.shape == (64, 96) and b.shape == (96, 20) and b.stride() == (1, 96) for a, b in ns)
    assert torch.allclose(O.all_scatter(ns, torch.float32).double(), full, atol=1e-4)


def test_one_shot_reduce_order_and_rounding():
    g = torch.Generator().manual_seed(5)
    parts = torch.randn(8, 40, 24, generator=g)
    got = O.one_shot_reduce(parts, torch.bfloat16)
    # explicit sequential loop in rank order, fp32, starting from +0
    acc = np.zeros((40, 24), dtype=np.float32)
    for r in range(8):
        acc = acc + parts[r].numpy()
    assert (got.view(torch.int16).numpy().view(np.uint16) == O.round_to_bf16_bits(acc)).all()
    assert torch.allclose(got.double(), parts.double().sum(0), rtol=1e-2, atol=1e-2)
    # rank order matters at the bit level: a reversed sum differs somewhere in fp32
    rev = np.zeros((40, 24), dtype=np.float32)
    for r in reversed(range(8)):
        rev = rev + parts[r].numpy()
    assert (rev != acc).any()
    # one rank: the result is the cast of the partial itself
    assert torch.equal(O.one_shot_reduce(parts[:1], torch.bfloat16), parts[0].to(torch.bfloat16))


# --------------------------------------------------------------------------- flags
@pytest.mark.parametrize("ws", [1, 2, 8])
def test_flag_protocol_invariants(ws):
    tiles = 12
    fm = O.FlagModel(ws, tiles)
    for r in range(ws):
        for t in range(tiles):
            fm.signal(r, t)
    # every producer added exactly +1 to every *other* rank
    assert (fm.flags == ws - 1).all()
    for r in range(ws):
        for t in range(tiles):
            assert fm.try_consume(r, t)
    assert (fm.flags == 0).all()  # the CAS resets the flag
    if ws > 1:
        assert not fm.try_consume(0, 0)  # not signalled again: the wait would spin
        fm.signal(1, 0)
        assert fm.try_consume(0, 0) == (ws == 2)
    # scatter's ready flag: every destination (self included) counts one arrival per producer
    fm2 = O.FlagModel(ws, tiles)
    for r in range(ws):
        for t in range(tiles):
            fm2.arrive(r, t)
    assert (fm2.flags == ws).all()


# --------------------------------------------------------------------------- heap
def test_heap_model_and_translate():
    h = O.HeapModel(1 << 20)
    sizes = [(4096, 4), (1, 2), (1025, 1), (0, 4), (256, 8)]
    offs = [h.allocate(n, es)[0] for n, es in sizes]
    want, cur = [], 0
    for n, es in sizes:
        want.append(cur)
        cur += -(-(n * es) // 1024) * 1024
    assert offs == want and all(o % 1024 == 0 for o in offs) and h.heap_offset == cur
    with pytest.raises(MemoryError, match="Heap out of memory"):
        h.allocate(1 << 20, 1)
    h2 = O.HeapModel(2048)
    h2.allocate(2048, 1)  # exactly full is fine
    with pytest.raises(MemoryError):
        h2.allocate(1, 1)
    bases = [0x7F0000000000, 0x7F0040000000, 0x7E0000000000]
    p = bases[0] + 12345
    assert O.translate(p, 0, 0, bases) == p
    assert O.translate(p, 0, 1, bases) - p == bases[1] - bases[0]
    assert O.translate(O.translate(p, 0, 2, bases), 2, 0, bases) == p
    assert O.translate(p, 0, 2, bases) == bases[2] + 12345  # target base below the source base


# --------------------------------------------------------------------------- bench statistics
def test_quantile_is_numpy_linear():
    rng = np.random.default_rng(0)
    for n in (1, 2, 5, 100):
        a = rng.random(n).tolist()
        q = [0.0, 0.2, 0.5, 0.8, 1.0, 0.33]
        assert np.allclose(O.quantile(a, q), np.quantile(a, q, method="linear"))
    with pytest.raises(ValueError):
        O.quantile([1.0, 2.0], [1.5])
    t = [3.0, 1.0, 2.0, 10.0]
    assert O.summarize_statistics(t, None, "mean") == 4.0
    assert O.summarize_statistics(t, None, "median") == 2.5
    assert O.summarize_statistics(t, None, "min") == 1.0 and O.summarize_statistics(t, None, "max") == 10.0
    assert O.summarize_statistics(t, None, "all") is t
    assert O.summarize_statistics(t, [0.5], None) == 2.5


def test_validate_gemm_is_allclose():
    A = torch.eye(4)
    B = torch.arange(16.0).reshape(4, 4)
    assert O.validate_gemm(A, B, B.clone(), atol=1)
    C = B.clone()
    C[2, 3] += 0.9
    assert O.validate_gemm(A, B, C, atol=1)
    C[2, 3] += 0.2
    assert not O.validate_gemm(A, B, C, atol=1)
