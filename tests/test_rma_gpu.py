"""Device-side remote access (include/iris_device.hpp) against the
expectations of the reference's unit tests (tests/unittests/test_*.py), with
the ranks played by sub-heaps of the one GPU.

Every rank runs the test kernel in turn on its own copy of the buffers, as the
MPI ranks of the reference each do; afterwards every rank's result must hold
what the reference expects on every rank.
"""

import pytest
import torch

import iris_amd
from iris_amd import ops, testing

pytestmark = pytest.mark.gpu

RANKS = [1, 2, 4]
BLOCKS = [1, 8, 16, 32]  # tests/unittests/test_load.py:43-50
SEMS = ["acquire", "release", "acq_rel"]  # tests/unittests/test_atomic_add.py:44-51
SCOPES = ["cta", "gpu", "sys"]  # tests/unittests/test_atomic_add.py:52-60


@pytest.fixture(scope="module", params=RANKS)
def heap(request):
    return iris_amd.iris(1 << 20, virtual_ranks=request.param)


def fresh(heap, block, dtype, fill):
    """(data, results) at a fresh heap offset, data filled with `fill` and results zeroed on every rank."""
    heap.heap_offset = 0
    data = heap.zeros(block, dtype=dtype)
    results = heap.zeros(block, dtype=dtype)
    for r in range(heap.get_num_ranks()):
        heap.on_rank(data, r).fill_(fill)
        heap.on_rank(results, r).zero_()
    return data, results


def run_all_ranks(heap, op, data, results, block, **kw):
    n = heap.get_num_ranks()
    hb = heap.get_heap_bases()
    for r in range(n):
        testing.rma_selftest(op, None if data is None else heap.on_rank(data, r), heap.on_rank(results, r), hb, r, n, block,
                         **kw)
    torch.cuda.synchronize()


def check_every_rank(heap, results, expected_value):
    for r in range(heap.get_num_ranks()):
        got = heap.on_rank(results, r)
        expected = torch.full_like(got, expected_value)
        torch.testing.assert_close(got, expected, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", [torch.int8, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("block", BLOCKS)
def test_load(heap, dtype, block):
    """Sum of ones loaded from every rank == num_ranks (tests/unittests/test_load.py:52-70)."""
    data, results = fresh(heap, block, dtype, 1)
    run_all_ranks(heap, "load", data, results, block)
    check_every_rank(heap, results, heap.get_num_ranks())


@pytest.mark.parametrize("dtype", [torch.int8, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("block", BLOCKS)
def test_store(heap, dtype, block):
    """Ones stored to every rank (tests/unittests/test_store.py:51-69)."""
    data, results = fresh(heap, block, dtype, 1)
    run_all_ranks(heap, "store", data, results, block)
    check_every_rank(heap, results, 1)


@pytest.mark.parametrize("dtype", [torch.int8, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("block", BLOCKS)
def test_get(heap, dtype, block):
    """Ones fetched from every rank and accumulated == num_ranks (tests/unittests/test_get.py:53-71)."""
    data, results = fresh(heap, block, dtype, 1)
    run_all_ranks(heap, "get", data, results, block)
    check_every_rank(heap, results, heap.get_num_ranks())


@pytest.mark.parametrize("dtype", [torch.int8, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("block", BLOCKS)
def test_put(heap, dtype, block):
    """Ones put to every rank (tests/unittests/test_put.py:48-66)."""
    data, results = fresh(heap, block, dtype, 1)
    run_all_ranks(heap, "put", data, results, block)
    check_every_rank(heap, results, 1)


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("sem", SEMS + ["relaxed"])
@pytest.mark.parametrize("scope", SCOPES)
@pytest.mark.parametrize("block", BLOCKS)
def test_atomic_add(heap, dtype, sem, scope, block):
    """Every rank adds 1 on every rank == num_ranks (tests/unittests/test_atomic_add.py:66-83)."""
    _, results = fresh(heap, block, dtype, 1)
    run_all_ranks(heap, "atomic_add", None, results, block, sem=sem, scope=scope)
    check_every_rank(heap, results, heap.get_num_ranks())


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.float16, torch.float32])
@pytest.mark.parametrize("sem", ["acq_rel"])
@pytest.mark.parametrize("scope", SCOPES)
def test_atomic_sub(heap, dtype, sem, scope):
    """iris/iris.py:452-473 has no reference test: start at 2*num_ranks, every
    rank subtracts 1 on every rank, num_ranks is left."""
    n = heap.get_num_ranks()
    _, results = fresh(heap, 16, dtype, 1)
    for r in range(n):
        heap.on_rank(results, r).fill_(2 * n)
    run_all_ranks(heap, "atomic_sub", None, results, 16, sem=sem, scope=scope)
    check_every_rank(heap, results, n)


@pytest.mark.parametrize("dtype", [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize("sem", SEMS)
@pytest.mark.parametrize("scope", SCOPES)
def test_atomic_cas(heap, dtype, sem, scope):
    """CAS(0 -> num_ranks) on every rank (tests/unittests/test_atomic_cas.py:50-67)."""
    _, results = fresh(heap, 1, dtype, 1)
    run_all_ranks(heap, "atomic_cas", None, results, 1, sem=sem, scope=scope)
    check_every_rank(heap, results, heap.get_num_ranks())


@pytest.mark.parametrize("dtype", [torch.int32, torch.int64, torch.float32])
@pytest.mark.parametrize("sem", SEMS)
@pytest.mark.parametrize("scope", SCOPES)
def test_atomic_xchg(heap, dtype, sem, scope):
    """Exchange in num_ranks on every rank (tests/unittests/test_atomic_xchg.py:49-66)."""
    _, results = fresh(heap, 1, dtype, 1)
    run_all_ranks(heap, "atomic_xchg", None, results, 1, sem=sem, scope=scope)
    check_every_rank(heap, results, heap.get_num_ranks())


def test_cas_only_swaps_on_a_match_and_masked_lanes_do_nothing(heap):
    n = heap.get_num_ranks()
    _, results = fresh(heap, 8, torch.int32, 1)
    for r in range(n):
        heap.on_rank(results, r).fill_(7)  # not the compare value: CAS must leave it
    run_all_ranks(heap, "atomic_cas", None, results, 1)
    check_every_rank(heap, results, 7)
    # block_size 3 of 8 elements: lanes 3.. are masked off
    _, results = fresh(heap, 8, torch.float32, 1)
    run_all_ranks(heap, "atomic_add", None, results, 3)
    for r in range(n):
        assert heap.on_rank(results, r).tolist() == [float(n)] * 3 + [0.0] * 5


def test_selftest_launcher_rejects_bad_arguments(heap):
    _, results = fresh(heap, 8, torch.int8, 1)
    with pytest.raises(RuntimeError):  # int8 has no atomics
        testing.rma_selftest("atomic_add", None, results, heap.get_heap_bases(), 0, heap.get_num_ranks(), 8)
    with pytest.raises(ValueError):
        testing.rma_selftest("load", results, results, heap.get_heap_bases(), 0, heap.get_num_ranks(), 65)
