#!/usr/bin/env python3
"""Headline benchmark of the fused GEMM + tile-publishing path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one batch of synthetic input:
the bf16 shard GEMM A[8192,1024] x B[1024,8192] (one rank's K-shard of
K=8192) with 256x256 output tiles stored as bf16 into the fine-grained heap
and one uint32 ready flag published per tile.  Prints ONE JSON line.

Also measured and reported inside that line: the one-shot reduce of 8 fp32
partial-C buffers [8192,8192] -> bf16 (the reduce phase, HBM-bound), the same
GEMM under the reference's cold-cache ``do_bench`` protocol, and a CPU
baseline of the same math on the host cores.
"""

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
PEAK_HBM_GBPS = 8000.0     # MI355X HBM3E, published

# HBM-side bytes per launch of the default kernels on this workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script, each scaled by what the same counter reads for the --copy-calibration
# kernel (profiles/gemm_all_scatter_bf16_8192x8192x1024.txt, profiles/one_shot_reduce_fp32x8_8192x8192.txt).
# Counters cannot be read from inside a run, so these are carried here and dropped for non-default variants.
GEMM_TRAFFIC_BYTES = 332877946
REDUCE_TRAFFIC_BYTES = 2281385094

M, N, K_SHARD, K_TOTAL = 8192, 8192, 1024, 8192
BLK_M, BLK_N, BLK_K, GSIZE_M, GRID = 256, 256, 64, 4, 256


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed launches of the same step before the warm-up, until this much time has passed: after "
                         "an idle period the GPU's power management first overshoots and then clamps the clocks for "
                         "~10 ms, which a short run would measure instead of the steady state")
    ap.add_argument("--variant", type=int, default=0, help="GEMM kernel tuning variant (0 = default)")
    ap.add_argument("--reduce-variant", type=int, default=0)
    ap.add_argument("--gsize_m", type=int, default=GSIZE_M)
    ap.add_argument("--no-reduce", action="store_true", help="skip the reduce-phase measurement")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-coldcache", action="store_true", help="skip the cold-cache do_bench protocol run")
    ap.add_argument("--offheap-operands", action="store_true", help="keep A and B outside the fine-grained heap")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain fp32 copy of [8192,8192] (256 MiB in, 256 MiB out): the kernel of known "
                         "size that scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    return ap.parse_args()


def timed_steps(fn, steps, warmup):
    """(wall seconds for `steps` calls, mean per-launch device ms).

    The device time comes from one pair of HIP events on the launch stream
    around the `steps` back-to-back launches: an event between every two
    launches would insert a ~11 us idle gap and a cache write-back before each
    kernel, which is not how the path runs.
    """
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, start.elapsed_time(end) / steps


def cpu_baseline():
    """The oracle's shard GEMM (fp32 matmul + bf16 downcast) on the host cores,
    on a bounded sample: the first 2048 rows of A against all of B."""
    import torch

    from oracle import iris_oracle as O

    rows = 2048
    g = torch.Generator().manual_seed(123)
    A = (torch.randn(rows, K_SHARD, generator=g) * 0.02).to(torch.bfloat16)
    B = (torch.randn(N, K_SHARD, generator=g) * 0.02).to(torch.bfloat16).T
    O.shard_gemm(A, B, torch.bfloat16)  # warm-up
    times = []
    t_end = time.perf_counter() + 12.0
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 20):
        t0 = time.perf_counter()
        O.shard_gemm(A, B, torch.bfloat16)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    # the reduce phase of the same math: 8 fp32 partials [1024, 8192] summed in rank order -> bf16
    parts = torch.randn(8, 1024, N, generator=g)
    O.one_shot_reduce(parts, torch.bfloat16)
    rtimes = []
    for _ in range(3):
        t0 = time.perf_counter()
        O.one_shot_reduce(parts, torch.bfloat16)
        rtimes.append(time.perf_counter() - t0)
    rmed = statistics.median(rtimes)
    return {
        "reduce_GBps": round((parts.numel() * 4 + 1024 * N * 2) / rmed / 1e9, 2),
        "reduce_sample": "oracle one_shot_reduce of 8 fp32 partials [1024,8192] -> bf16, 3 runs, median",
        "value": 2.0 * rows * N * K_SHARD / med / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle shard_gemm (torch fp32 matmul + bf16 cast) on A[:{rows}] x B, {len(times)} runs, median; "
                  f"os.cpu_count()={os.cpu_count()}",
    }


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU's share of the path; --gpus {args.gpus} is not supported "
              "(no collectives or multi-GPU runs are part of this build).", file=sys.stderr)
        sys.exit(2)

    import torch

    import iris_amd
    from iris_amd import ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)

    ws = 8
    # per-rank heap: full-K operands 2 x 128 MiB, bf16 results 2 x 128 MiB, fp32 partial 256 MiB, flags
    shmem = iris_amd.iris(1 << 30, virtual_ranks=ws)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(123)
    # one rank's K-shard as a strided view of the full-K operands (the 08/09 sharding)
    A_full = (torch.randn(M, K_TOTAL, generator=g) * 0.02).to(dtype)
    B_full = (torch.randn(N, K_TOTAL, generator=g) * 0.02).to(dtype)
    if args.offheap_operands:
        a_full, bt_full = A_full.cuda(), B_full.cuda()
    else:
        a_full = shmem.zeros((M, K_TOTAL), dtype=dtype)
        a_full.copy_(A_full)
        bt_full = shmem.zeros((N, K_TOTAL), dtype=dtype)
        bt_full.copy_(B_full)
    a = a_full[:, :K_SHARD]
    b = bt_full[:, :K_SHARD].T
    del A_full, B_full
    c_global = shmem.zeros((M, N), dtype=dtype)
    total_tiles = ops.cdiv(M, BLK_M) * ops.cdiv(N, BLK_N)
    flags = shmem.zeros((total_tiles,), dtype=torch.int32)
    hb = shmem.get_heap_bases()
    num_xcds = ops.default_num_xcds(shmem.get_cu_count(), GRID)

    def gemm_step():
        ops.gemm_launch(a, b, None, c_global, flags, hb, 0, 1, GRID, BLK_M, BLK_N, BLK_K, args.gsize_m,
                        ops.EPI_ALL_SCATTER, notify=True, num_xcds=num_xcds, variant=args.variant)

    flops = 2.0 * M * N * K_SHARD
    settle_launches = 0
    t_end = time.perf_counter() + args.settle_ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(20):
            gemm_step()
        torch.cuda.synchronize()
        settle_launches += 20
    wall, kernel_ms = timed_steps(gemm_step, args.steps, args.warmup)
    ms_per_step = wall / args.steps * 1e3
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    kernel_tflops = flops / (kernel_ms * 1e-3) / 1e12
    assert int(flags.min().item()) == args.steps + args.warmup + settle_launches, "every tile publishes once per step"
    regs, spills = ops.gemm_kernel_info(a, b, None, c_global, flags, hb, 0, 1, GRID, BLK_M, BLK_N, BLK_K,
                                        args.gsize_m, ops.EPI_ALL_SCATTER, num_xcds=num_xcds, variant=args.variant)

    result = {
        "metric": "fused GEMM+reduce TFLOP/s (% bf16 MFMA peak); reduce-phase HBM GB/s",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "single-shard fused GEMM + flag-published epilogue: bf16 A[8192,1024] x B[1024,8192] "
                        "(K-shard views, lda=ldb=8192), fp32 accumulate, 256x256 tiles -> bf16 in the fine-grained "
                        "heap, one uint32 ready flag per tile",
            "M": M, "N": N, "K_shard": K_SHARD, "BLK_M": BLK_M, "BLK_N": BLK_N, "gsize_m": args.gsize_m,
            "grid": GRID, "num_xcds": num_xcds, "variant": args.variant,
            "operands": "device memory outside the heap" if args.offheap_operands else "fine-grained heap",
        },
        "pct_of_bf16_peak": round(100.0 * tflops / PEAK_BF16_TFLOPS, 2),
        "gemm_kernel": {"registers": regs, "spill_bytes": spills, "mean_ms": round(kernel_ms, 5)},
        "roofline": {
            "bound": "mfma",
            "achieved": round(kernel_tflops, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(kernel_tflops / PEAK_BF16_TFLOPS, 4),
            "traffic": GEMM_TRAFFIC_BYTES if args.variant == 0 and args.gsize_m == GSIZE_M else None,
        },
    }

    if not args.no_coldcache:
        cold_ms = iris_amd.do_bench(gemm_step, shmem.barrier, lambda: None, n_warmup=5, n_repeat=20)
        result["gemm_cold_cache"] = {"protocol": "do_bench: 256 MiB cache flush before every repetition, mean",
                                     "ms": round(cold_ms, 5),
                                     "tflops": round(flops / (cold_ms * 1e-3) / 1e12, 2)}

    if not args.no_reduce:
        # reduce phase: 8 fp32 partials [8192,8192] (one per virtual rank) -> bf16
        c = shmem.zeros((M, N), dtype=torch.float32)
        out = shmem.zeros((M, N), dtype=dtype)
        for r in range(ws):
            part = shmem.on_rank(c, r)
            part.normal_(generator=None)
            shmem.on_rank(flags, r).zero_()
        torch.cuda.synchronize()

        def arm():
            for r in range(ws):  # the producers' signals: +1 on every other rank's tile flags
                ops.signal_tiles(shmem.on_rank(flags, r), hb, total_tiles, r, ws)

        red_ms = []
        steps = max(5, min(args.steps, 30))
        for i in range(3 + steps):
            arm()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            ops.one_shot_reduce(c, out, flags, hb, 0, ws, BLK_M, BLK_N, args.gsize_m, variant=args.reduce_variant)
            e.record()
            torch.cuda.synchronize()
            if i >= 3:
                red_ms.append(s.elapsed_time(e))
        assert int(flags.abs().max().item()) == 0, "the reduce consumes every flag"
        rbytes = ws * M * N * 4 + M * N * 2
        rms = statistics.mean(red_ms)
        gbps = rbytes / (rms * 1e-3) / 1e9
        result["reduce"] = {
            "workload": "one-shot reduce of 8 fp32 partial-C [8192,8192] -> bf16, gated by per-tile flags",
            "mean_ms": round(rms, 5), "min_ms": round(min(red_ms), 5), "GBps": round(gbps, 1),
            "pct_of_hbm_peak": round(100.0 * gbps / PEAK_HBM_GBPS, 2), "variant": args.reduce_variant,
            "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                         "frac": round(gbps / PEAK_HBM_GBPS, 4),
                         "traffic": REDUCE_TRAFFIC_BYTES if args.reduce_variant == 0 else None},
        }

    if args.copy_calibration:
        # ws=1, fp32 -> fp32: the reduce kernel degenerates to a plain tiled copy
        src = torch.randn((M, N), dtype=torch.float32, device="cuda")
        dst = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        for _ in range(3):
            ops.one_shot_reduce(src, dst, flags, hb, 0, 1, BLK_M, BLK_N, args.gsize_m, wait_flags=False)
        torch.cuda.synchronize()
        assert torch.equal(src, dst)
        result["copy_calibration"] = {"kernel": "reduce_tiles_vec_kernel<fp32, fp32, ws=1>",
                                      "read_bytes": M * N * 4, "write_bytes": M * N * 4, "launches": 3}

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()

    print(json.dumps(result))


if __name__ == "__main__":
    main()
