"""Host logic of the Iris context, the bench helpers and the launch-argument
checks, on a machine without a GPU (the heap is host memory injected through
the test seam; no kernel is launched)."""

import numpy as np
import pytest
import torch

import iris_amd
from iris_amd import ops, util
from oracle import iris_oracle as O


@pytest.fixture()
def ctx(host_pool_factory):
    return iris_amd.Iris(1 << 20, virtual_ranks=4, cur_rank=1, _pool_factory=host_pool_factory)


def test_exports():
    for name in ("Iris", "iris", "do_bench", "memset_tensor"):
        assert hasattr(iris_amd, name)


def test_bump_allocator_matches_oracle_model(ctx):
    model = O.HeapModel(1 << 20)
    base = ctx.memory_pool.data_ptr()
    for n, dt in [(100, torch.int32), (1, torch.float16), (513, torch.bfloat16), (1024, torch.int8), (7, torch.float64)]:
        t = ctx.allocate(n, dt)
        start, nbytes = model.allocate(n, t.element_size())
        assert t.data_ptr() - base == start and t.numel() == n and t.dtype == dt
        assert t.numel() * t.element_size() == nbytes
    assert ctx.heap_offset == model.heap_offset
    with pytest.raises(MemoryError, match="Heap out of memory"):
        ctx.allocate(1 << 20, torch.int8)


def test_factories_defaults_and_shapes(ctx):
    z = ctx.zeros(4096)
    assert z.dtype == torch.int32 and z.shape == (4096,) and int(z.abs().sum()) == 0
    z2 = ctx.zeros((3, 5), dtype=torch.bfloat16, device="cuda")  # device= is accepted and ignored
    assert z2.shape == (3, 5) and z2.dtype == torch.bfloat16
    assert ctx.zeros(2, 3, dtype=torch.float32).shape == (2, 3)
    o = ctx.ones(2, 3)
    assert o.dtype == torch.get_default_dtype() and torch.equal(o, torch.ones(2, 3))
    f = ctx.full((4,), 7)
    assert f.dtype == torch.int32 and f.tolist() == [7] * 4
    assert ctx.empty((2, 2)).dtype == torch.float32
    u = ctx.uniform((1000,), 2.0, 3.0)
    assert 2.0 <= float(u.min()) and float(u.max()) <= 3.0
    g = torch.Generator().manual_seed(123)
    r = ctx.randn(8, 4, generator=g)
    assert torch.equal(r, torch.randn(32, generator=torch.Generator().manual_seed(123)).reshape(8, 4))
    assert ctx.arange(5).tolist() == [0, 1, 2, 3, 4] and ctx.arange(5).dtype == torch.int64
    assert ctx.arange(1, 2.5, 0.5).dtype == torch.get_default_dtype()
    assert torch.allclose(ctx.linspace(0, 1, 5), torch.linspace(0, 1, 5))
    ri = ctx.randint((3, 4), 0, 10)
    assert ri.shape == (3, 4) and ri.dtype == torch.int32 and 0 <= int(ri.min()) and int(ri.max()) < 10
    zl = ctx.zeros_like(r)
    assert zl.numel() == r.numel() and zl.dtype == r.dtype
    for t in (z, z2, o, f, u, r, zl):
        assert (t.data_ptr() - ctx.memory_pool.data_ptr()) % 1024 == 0


def test_out_tensor_validation(ctx):
    good = ctx.zeros(6, dtype=torch.float32)
    assert ctx.ones(6, out=good, dtype=torch.float32) is good or torch.equal(good, torch.ones(6))
    with pytest.raises(RuntimeError, match="not on the symmetric heap"):
        ctx.ones(6, out=torch.zeros(6), dtype=torch.float32)
    with pytest.raises(RuntimeError, match="elements"):
        ctx.ones(5, out=good, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="dtype"):
        ctx.ones(6, out=good, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="elements"):
        ctx.arange(4, out=good, dtype=torch.float32)


def test_heap_bases_and_virtual_ranks(ctx):
    hb = ctx.get_heap_bases()
    assert hb.dtype == torch.uint64 and hb.numel() == 4
    bases = hb.view(torch.int64).tolist()
    assert bases == [ctx._pool_all.data_ptr() + r * (1 << 20) for r in range(4)]
    assert ctx.get_rank() == 1 and ctx.get_num_ranks() == 4
    t = ctx.zeros((4, 6), dtype=torch.int32)
    view = t[:, 2:5]  # strided view inside the heap
    for r in range(4):
        peer = ctx.on_rank(view, r)
        assert peer.shape == view.shape and peer.stride() == view.stride() and peer.dtype == view.dtype
        assert peer.data_ptr() == O.translate(view.data_ptr(), 1, r, bases)
    assert ctx.on_rank(t, 1).data_ptr() == t.data_ptr()
    ctx.on_rank(t, 3).fill_(9)  # symmetric: same offset, different sub-heap
    assert int(t.sum()) == 0 and int(ctx.on_rank(t, 3).sum()) == 9 * 24
    with pytest.raises(RuntimeError):
        ctx.on_rank(torch.zeros(3), 0)
    with pytest.raises(ValueError):
        ctx.on_rank(t, 4)
    assert ctx.broadcast(3.5, 0) == 3.5  # callers pass (value, rank)
    with pytest.raises(ValueError):
        iris_amd.Iris(1024, virtual_ranks=2, cur_rank=2, _pool_factory=lambda n: torch.zeros(n, dtype=torch.int8))


def test_logging_flags(ctx, capsys):
    ctx.log("hello")
    ctx.log_stats("stats")
    ctx.log_debug("hidden")
    out = capsys.readouterr().out
    assert "[Iris] [1/4] hello" in out and "[Iris] [1/4] stats" in out and "hidden" not in out


def test_quantile_and_summary_match_numpy_and_oracle():
    rng = np.random.default_rng(1)
    a = rng.random(37).tolist()
    q = [0.0, 0.1, 0.5, 0.9, 1.0]
    assert np.allclose(util._quantile(a, q), np.quantile(a, q, method="linear"))
    assert util._quantile(a, q) == O.quantile(a, q)
    with pytest.raises(ValueError):
        util._quantile(a, [-0.1])
    for mode in ("min", "max", "mean", "median", "all"):
        assert util._summarize_statistics(a, None, mode) == O.summarize_statistics(a, None, mode)
    assert util._summarize_statistics(a, [0.5], "mean") == O.summarize_statistics(a, [0.5], "mean")


def test_memset_tensor_contract():
    with pytest.raises(AssertionError, match="int32"):
        util.memset_tensor(torch.zeros(4, dtype=torch.int64), 0)
    with pytest.raises(AssertionError, match="contiguous"):
        util.memset_tensor(torch.zeros(4, 4, dtype=torch.int32)[:, 1], 0)
    with pytest.raises(RuntimeError, match="device tensor"):
        util.memset_tensor(torch.zeros(4, dtype=torch.int32), 0)


def test_xcd_choice():
    assert ops.default_num_xcds(304, 304) == 8 and ops.default_num_xcds(304, 288) == 8
    assert ops.default_num_xcds(256, 256) == 8
    assert ops.default_num_xcds(256, 250) == 1  # the remap needs a grid that splits evenly
    assert ops.default_num_xcds(120, 120) == 1


def test_launch_argument_checks_fire_before_any_launch():
    a = torch.zeros(64, 32, dtype=torch.bfloat16)
    b = torch.zeros(32, 48, dtype=torch.bfloat16)
    cg = torch.zeros(64, 48, dtype=torch.bfloat16)
    common = dict(tile_completed=None, heap_bases=None, rank=0, world_size=1, num_sms=4, BLK_M=64, BLK_N=64,
                  BLK_K=32, gsize_m=1, epilogue=ops.EPI_ALL_SCATTER)
    with pytest.raises(AssertionError, match="incompatible dimensions"):
        ops.gemm_launch(a, torch.zeros(31, 48, dtype=torch.bfloat16), None, cg, **common)
    with pytest.raises(RuntimeError, match="must be on"):
        ops.gemm_launch(a, b, None, cg, **common)  # host tensors never reach a kernel
    with pytest.raises(RuntimeError, match="must be on"):
        ops.one_shot_reduce(cg, cg, None, None, 0, 1, 64, 64, 1)
