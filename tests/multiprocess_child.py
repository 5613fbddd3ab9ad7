"""One rank of the multi-process GPU test (started by test_multiprocess_gpu.py
with RANK / WORLD_SIZE / IRIS_AMD_RENDEZVOUS set).  Every rank is a process of
its own on the one GPU: ``iris_amd.iris(heap_size)`` allocates its heap, swaps
IPC handles with the others and maps their heaps, so ``heap_bases`` holds real
mapped addresses.  Checks, with the expectations of the reference's unit
tests (tests/unittests/test_*.py) and of the one-shot example:

* the seven device-side remote-access kernels against the mapped heaps,
* all-scatter of N-shards with ready flags,
* 09 as PRODUCE -> barrier -> CONSUME, bit-exact against the oracle.
"""

import os
import sys

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
sys.path.insert(0, ROOT)

import torch  # noqa: E402

import iris_amd  # noqa: E402
from iris_amd import ops, testing  # noqa: E402
from oracle import iris_oracle as O  # noqa: E402


def say(*a):
    print(f"[rank {os.environ.get('RANK')}]", *a, flush=True)


def main():
    shmem = iris_amd.iris(96 << 20)
    rank, ws = shmem.get_rank(), shmem.get_num_ranks()
    assert ws == int(os.environ["WORLD_SIZE"]) and rank == int(os.environ["RANK"])
    hb = shmem.get_heap_bases()
    bases = hb.cpu().view(torch.int64).tolist()
    assert len(bases) == ws and bases[rank] == shmem.memory_pool.data_ptr() and len(set(bases)) == ws
    assert int(shmem.broadcast(1000 + rank, 1)) == 1001  # (value, root): iris/iris.py:93-94
    say("heap bases", [hex(b) for b in bases])

    # ---- the unit tests' kernels against the real mapped heaps
    def fresh(block, dtype, fill_data, fill_results):
        shmem.heap_offset = 0
        data, results = shmem.zeros(block, dtype=dtype), shmem.zeros(block, dtype=dtype)
        data.fill_(fill_data)
        results.fill_(fill_results)
        shmem.barrier()  # every rank's buffers are in place before anyone touches a peer's
        return data, results

    def check(results, value, what):
        shmem.barrier()  # every rank's kernel has run
        want = torch.full_like(results, value)
        assert torch.equal(results, want), f"{what}: {results.tolist()} != {value}"
        shmem.barrier()  # nobody re-fills the buffers while a peer still reads them

    for dtype in (torch.int8, torch.float16, torch.bfloat16, torch.float32):
        for block in (1, 8, 32):
            for op, expect in (("load", ws), ("store", 1), ("get", ws), ("put", 1)):
                data, results = fresh(block, dtype, 1, 0)
                testing.rma_selftest(op, data, results, hb, rank, ws, block)
                check(results, expect, f"{op} {dtype} block {block}")
    for dtype in (torch.int32, torch.int64, torch.float16, torch.bfloat16, torch.float32):
        for sem, scope in (("relaxed", "gpu"), ("release", "sys"), ("acq_rel", "sys"), ("acquire", "gpu")):
            _, results = fresh(16, dtype, 1, 0)
            testing.rma_selftest("atomic_add", None, results, hb, rank, ws, 16, sem=sem, scope=scope)
            check(results, ws, f"atomic_add {dtype} {sem} {scope}")
    _, results = fresh(16, torch.int32, 1, 2 * ws)
    testing.rma_selftest("atomic_sub", None, results, hb, rank, ws, 16)
    check(results, ws, "atomic_sub")
    for dtype in (torch.int32, torch.int64):
        _, results = fresh(1, dtype, 1, 0)
        testing.rma_selftest("atomic_cas", None, results, hb, rank, ws, 1, sem="acq_rel", scope="sys")
        check(results, ws, f"atomic_cas {dtype}")
        _, results = fresh(1, dtype, 1, 0)
        testing.rma_selftest("atomic_xchg", None, results, hb, rank, ws, 1, sem="acq_rel", scope="sys")
        check(results, ws, f"atomic_xchg {dtype}")
    say("remote-access kernels ok")

    # ---- GEMM + all-scatter: rank r's N-shard lands at column r*N_local on every rank, flags count ws arrivals
    shmem.heap_offset = 0
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(123)
    M, N, K, BM, BN, G = 384, 256 * ws, 512, 128, 64, 4
    A = (torch.randn(M, K, generator=g) * 0.05).to(dtype)
    B = (torch.randn(N, K, generator=g) * 0.05).to(dtype).T
    n_local = N // ws
    a = shmem.zeros((M, K), dtype=dtype)
    a.copy_(A)
    bt = shmem.zeros((n_local, K), dtype=dtype)
    bt.copy_(B.T[rank * n_local:(rank + 1) * n_local])
    cg = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(n_local, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    shmem.barrier()
    ops.gemm_launch(a, bt.T, None, cg, flags, hb, rank, ws, 64, BM, BN, 64, G, ops.EPI_ALL_SCATTER, num_xcds=8,
                    scope=ops.SCOPE_SYSTEM)
    shmem.barrier()
    want = O.all_scatter(O.n_shards(A, B, ws), dtype)
    assert torch.allclose(cg.float().cpu(), want.float(), rtol=1e-2, atol=1e-2), "all-scatter result"
    assert flags.cpu().tolist() == [ws] * total, "ready flags"
    shmem.barrier()
    say("all-scatter ok")

    # ---- 09: PRODUCE -> barrier -> CONSUME over K-shards; partials fp32
    shmem.heap_offset = 0
    M, N, K, BM, BN, G = 512, 384, 256 * ws, 256, 128, 6
    A = (torch.randn(M, K, generator=g) * 0.05).to(dtype)
    B = (torch.randn(N, K, generator=g) * 0.05).to(dtype).T
    ks = K // ws
    a = shmem.zeros((M, ks), dtype=dtype)
    a.copy_(A[:, rank * ks:(rank + 1) * ks])
    bt = shmem.zeros((N, ks), dtype=dtype)
    bt.copy_(B.T[:, rank * ks:(rank + 1) * ks])
    c = shmem.zeros((M, N), dtype=torch.float32)
    out = shmem.zeros((M, N), dtype=dtype)
    total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
    flags = shmem.zeros((total,), dtype=torch.int32)
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    shmem.barrier()
    ops.gemm_launch(a, bt.T, c, out, flags, hb, rank, ws, 64, BM, BN, 64, G, ops.EPI_ONE_SHOT,
                    phase=ops.PHASE_PRODUCE, num_xcds=8, scope=ops.SCOPE_SYSTEM)
    shmem.barrier()
    assert flags.cpu().tolist() == [ws - 1] * total, "every other rank has signalled every tile"
    ops.one_shot_reduce(c, out, flags, hb, rank, ws, BM, BN, G, scope=ops.SCOPE_SYSTEM, status=status,
                        spin_timeout_ticks=50_000_000)
    shmem.barrier()
    assert int(status.item()) == 0
    partials = torch.stack([shmem.on_rank(c, r).cpu() for r in range(ws)])  # the peers' partials, through the mappings
    assert torch.equal(out.cpu(), O.one_shot_reduce(partials, dtype)), "reduce is not the rank-ordered sum"
    full = O.one_shot_all_reduce(O.k_shards(A, B, ws), torch.float32, dtype)
    assert torch.allclose(out.float().cpu(), full.float(), rtol=1e-2, atol=1e-2), "all-reduce result"
    assert flags.cpu().tolist() == [0] * total, "flags consumed"
    shmem.barrier()
    say("one-shot all-reduce ok")

    # ---- 09 inside the program (PHASE_FUSED): the ranks' kernels wait for each other on the device, so they
    # must share it: at most two ranks of 128 programs on the 256 CUs
    if ws == 2:
        for t in (c, out, flags):
            t.zero_()
        status.zero_()
        shmem.barrier()
        ops.gemm_launch(a, bt.T, c, out, flags, hb, rank, ws, 128, BM, BN, 64, G, ops.EPI_ONE_SHOT,
                        phase=ops.PHASE_FUSED, num_xcds=8, scope=ops.SCOPE_SYSTEM, status=status,
                        spin_timeout_ticks=50_000_000)
        shmem.barrier()
        assert int(status.item()) == 0, "a program gave up waiting for the other process's rank"
        partials = torch.stack([shmem.on_rank(c, r).cpu() for r in range(ws)])
        assert torch.equal(out.cpu(), O.one_shot_reduce(partials, dtype)), "in-program reduce"
        assert flags.cpu().tolist() == [0] * total
        shmem.barrier()
        say("in-program one-shot across two processes ok")
    print(f"RANK {rank} OK", flush=True)
    shmem.barrier()


if __name__ == "__main__":
    main()
