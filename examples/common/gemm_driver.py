"""Shared driver of the three GEMM + communication examples.

One ``main(algorithm)`` stands in for the reference's three near-identical
``benchmark.py`` scripts (examples/07_gemm_all_scatter/benchmark.py,
examples/08_gemm_atomics_all_reduce/benchmark.py,
examples/09_gemm_one_shot_all_reduce/benchmark.py): same command-line flags,
same buffers, same warm-up / validate / benchmark / JSON flow.

Differences, all forced by the hardware this runs on:

* ``--gemm_sms`` defaults to 256, one persistent program per MI355X CU;
* ``--virtual_ranks P`` (new) lets the one GPU play P ranks: the heap is
  carved into P symmetric sub-heaps and every rank's launch runs in turn.
  With the one-shot algorithm all producers run before the consumers, since
  P programs that wait for each other cannot share one GPU from one stream.
* Started once per rank instead (``torchrun --nproc-per-node P``, or ``RANK``
  / ``WORLD_SIZE`` with ``IRIS_AMD_RENDEZVOUS``; the reference uses
  ``mpirun -np P``), every process is one rank with its own heap, mapped by
  its peers over IPC, as in the reference.  The one-shot algorithm then runs
  the reference's program as it is (produce, signal, wait, reduce, tile by
  tile); on one GPU the ranks' kernels must be resident together, so
  ``--gemm_sms`` is capped at the CU count divided by the ranks.
"""

import argparse
import os
import random
import sys

import torch

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

import iris_amd as iris  # noqa: E402
from iris_amd import matmul as _matmul  # noqa: E402
from iris_amd import ops  # noqa: E402
from examples.common.utils import JSONWriter, Timestamps  # noqa: E402
from examples.common.validation import validate_gemm  # noqa: E402

ALGORITHMS = {
    # name: (matmul class, per-script defaults, K-split?, validation atol)
    "all_scatter": (_matmul.matmul_all_scatter, dict(BLK_N=64, gsize_m=4, num_stages=2, kpack=1), False, 1),
    "atomics_all_reduce": (_matmul.matmul_atomics_all_reduce, dict(BLK_N=128, gsize_m=6, num_stages=1, kpack=2),
                           True, 2),
    "one_shot_all_reduce": (_matmul.matmul_one_shot_all_reduce, dict(BLK_N=64, gsize_m=6, num_stages=1, kpack=2),
                            True, 2),
}

DATATYPES = {"fp16": torch.float16, "fp32": torch.float32, "int8": torch.int8, "bf16": torch.bfloat16}


def parse_args(defaults, argv=None):
    parser = argparse.ArgumentParser(
        description="Parse matrix dimensions and configuration.",
        formatter_class=argparse.ArgumentDefaultsHelpFormatter,
    )
    parser.add_argument("-m", type=int, default=8192, help="Number of rows in matrix A")
    parser.add_argument("-n", type=int, default=4608, help="Number of columns in matrix B")
    parser.add_argument("-k", type=int, default=36864, help="Common dimension between matrices A and B")
    parser.add_argument("-d", "--debug", action="store_true", help="Enable debug mode")
    parser.add_argument("-v", "--validate", action="store_true", help="Enable validation mode")
    parser.add_argument("-t", "--trace_tiles", action="store_true", help="Enable tile-tracing mode")
    parser.add_argument("-b", "--benchmark", action="store_true", help="Enable benchmarking mode")
    parser.add_argument("--datatype", type=str, default="fp16", choices=list(DATATYPES), help="Datatype of computation")
    parser.add_argument("--algorithm", type=str, default=None, help="Accepted for compatibility; ignored")
    parser.add_argument("--output_file", type=str, default="log.json", help="Output file")
    parser.add_argument("--BLK_M", type=int, default=256, help="Block size M")
    parser.add_argument("--BLK_N", type=int, default=defaults["BLK_N"], help="Block size N")
    parser.add_argument("--BLK_K", type=int, default=64, help="Block size K")
    parser.add_argument("--gsize_m", type=int, default=defaults["gsize_m"], help="Grid size M")
    parser.add_argument("--two_tiles", type=str, default="True", help="Use two tiles")
    parser.add_argument("--num_stages", type=int, default=defaults["num_stages"], help="Number of stages")
    parser.add_argument("--num_warps", type=int, default=8, help="Number of warps")
    parser.add_argument("--waves_per_eu", type=int, default=0, help="Waves per execution unit")
    parser.add_argument("--mfmaInstrSize", type=int, default=16, help="MFMA instruction size")
    parser.add_argument("--kpack", type=int, default=defaults["kpack"], help="K packing size")
    parser.add_argument("--heap_size", type=int, default=None,
                        help="Iris heap size (default: 1 << 33; with one process per rank, whose heaps are mapped "
                             "through IPC, the largest size such a mapping takes here, just under 2 GiB)")
    parser.add_argument("--gemm_sms", type=int, default=256, help="Number of persistent programs")
    parser.add_argument("--total_sms", type=int, default=304, help="Total number of SMs")
    parser.add_argument("--virtual_ranks", type=int, default=1, help="Ranks played by this one GPU")
    return vars(parser.parse_args(argv))


def main(algorithm, argv=None):
    torch.manual_seed(123)
    random.seed(123)
    matmul, defaults, k_split, atol = ALGORITHMS[algorithm]
    args = parse_args(defaults, argv)

    ranks = args["virtual_ranks"]
    # one process per rank when a launcher's environment says so, else this process plays `ranks` ranks
    if args["heap_size"] is None:
        args["heap_size"] = 1 << 33  # the reference scripts' default (benchmark.py:67)
        if ranks == 1 and iris.launched_as_ranks():
            # peers map this heap through IPC, which takes less than 2 GiB per mapping here; only a size the
            # user asked for is an error
            args["heap_size"] = iris.IPC_MAX_HEAP_BYTES
            print(f"[Iris] heap_size defaults to {args['heap_size']} bytes with one process per rank "
                  "(IPC mappings stay under 2 GiB)")
    shmem = iris.iris(args["heap_size"], virtual_ranks=ranks) if ranks > 1 else iris.iris(args["heap_size"])
    rank = shmem.get_rank()
    world_size = shmem.get_num_ranks()
    cu_count = shmem.get_cu_count()
    multi_process = shmem.comm is not None
    played = [rank] if multi_process else list(range(world_size))
    if multi_process:
        matmul.scope = ops.SCOPE_SYSTEM  # peers are other processes (the reference's scope="sys")
    if multi_process and iris._hip.count_devices() < world_size:
        # Ranks that share a GPU: programs wait for programs (09 for the peers' tiles, 07 / 08 for the other
        # parts of a tile whose K range the launcher has shared out), so every rank's whole grid must fit the
        # device at once.
        fit = max(8, (cu_count // world_size) // 8 * 8)
        if args["gemm_sms"] > fit:
            shmem.log(f"gemm_sms {args['gemm_sms']} -> {fit}: {world_size} ranks share the {cu_count} CUs of one GPU")
            args["gemm_sms"] = fit

    datatype = DATATYPES[args["datatype"]]
    if datatype not in (torch.float16, torch.bfloat16, torch.float32):
        print(f"Datatype {args['datatype']} is not supported by the HIP kernels (fp16, bf16 and fp32 are).")
        sys.exit(1)

    assert args["n"] % world_size == 0, f"N ({args['n']}) must be divisible by world size ({world_size})."
    assert args["k"] % world_size == 0, f"K ({args['k']}) must be divisible by world size ({world_size})."

    A = shmem.randn(args["m"], args["k"], device="cuda", dtype=datatype)
    B = shmem.randn(args["n"], args["k"], device="cuda", dtype=datatype).T
    C = shmem.zeros((args["m"], args["n"]), device="cuda", dtype=A.dtype)

    args["M"], args["N"], args["K"] = args["m"], args["n"], args["k"]

    json_writer = JSONWriter(args["output_file"])
    json_writer.add_field("world_size", world_size)

    # one (local_A, local_B) pair per rank this GPU plays
    if k_split:
        ks = args["k"] // world_size
        args["k"] = ks
        shards = {r: (A[:, r * ks:(r + 1) * ks], B[r * ks:(r + 1) * ks, :]) for r in played}
    else:
        ns = args["n"] // world_size
        args["n"] = ns
        shards = {r: (A, B[:, r * ns:(r + 1) * ns].clone()) for r in played}

    for key, value in args.items():
        json_writer.add_field(key, value)

    global_C = shmem.zeros((args["M"], args["N"]), device="cuda", dtype=A.dtype)
    local_C = shmem.zeros((args["m"], args["n"]), device="cuda", dtype=A.dtype)

    total_tiles = ops.cdiv(args["m"], args["BLK_M"]) * ops.cdiv(args["n"], args["BLK_N"])

    if k_split and args["gemm_sms"] >= args["total_sms"]:
        print(f"Invalid number of stream-K SMs. {args['gemm_sms']} >= {args['total_sms']}")
        sys.exit(1)

    tile_completed = shmem.zeros((total_tiles,), device="cuda", dtype=torch.int32)
    locks = shmem.zeros((args["gemm_sms"],), device="cuda", dtype=torch.int32)
    P = shmem.zeros((args["gemm_sms"], args["BLK_M"] * args["BLK_N"]), device="cuda", dtype=torch.float32)
    bias = None

    gemm_stream = torch.cuda.Stream()
    json_writer.add_field("gemm_sms", args["gemm_sms"])

    timing = {
        "start_event": torch.cuda.Event(enable_timing=True),
        "end_event": torch.cuda.Event(enable_timing=True),
        "ms": 0,
        "experiments": 0,
    }
    timestamps = Timestamps(num_tiles=total_tiles)

    def launch(r, phase=None):
        if phase is not None:
            matmul.phase = phase
        local_A, local_B = shards[r]
        # the matmul of rank r sees rank r's buffers and flags
        return matmul.apply(
            local_A, local_B, shmem.on_rank(local_C, r), shmem.on_rank(global_C, r), bias, P, locks,
            shmem.on_rank(tile_completed, r), r, world_size, args["gemm_sms"], args["BLK_M"], args["BLK_N"],
            args["BLK_K"], args["gsize_m"], args["two_tiles"], args["num_stages"], args["num_warps"],
            args["waves_per_eu"], args["mfmaInstrSize"], args["kpack"], shmem.get_heap_bases(), cu_count,
            args["trace_tiles"], timestamps.mm_begin_timestamp, timestamps.mm_end_timestamp,
        )

    def preamble():
        shmem.barrier()
        for r in played:
            iris.memset_tensor(shmem.on_rank(tile_completed, r), 0)
        shmem.barrier()

    def run_experiment():
        shmem.barrier()
        if args["trace_tiles"]:
            timestamps.reset()
            shmem.barrier()
        torch.cuda.nvtx.range_push("GEMM + Communication")
        with torch.cuda.stream(gemm_stream):
            timing["start_event"].record()
            if algorithm == "one_shot_all_reduce" and world_size > 1 and not multi_process:
                for r in played:
                    launch(r, ops.PHASE_PRODUCE)
                for r in played:
                    launch(r, ops.PHASE_CONSUME)
            else:
                # (one rank per process: 09 is the reference's single program, ops.PHASE_FUSED)
                for r in played:
                    launch(r, ops.PHASE_FUSED if algorithm == "one_shot_all_reduce" else None)
            timing["end_event"].record()
            timing["experiments"] += 1
        torch.cuda.nvtx.range_pop()
        shmem.barrier()
        timing["ms"] += timing["start_event"].elapsed_time(timing["end_event"])

    matmul.set_debug(args["debug"])
    shmem.barrier()
    run_experiment()  # warm-up, and the one run that --validate checks
    gemm_registers, gemm_spills = matmul.streamk_registers, matmul.streamk_spills
    matmul.set_debug(False)
    shmem.barrier()
    preamble()
    shmem.barrier()
    timing["ms"] = 0
    timing["experiments"] = 0

    json_writer.add_field("gemm_registers", gemm_registers)
    json_writer.add_field("gemm_spills", gemm_spills)

    if args["validate"]:
        shmem.log("Validating...")
        success = validate_gemm(A, B, global_C, shmem, atol=atol)
        shmem.log(f"Final C validation {'passed' if success else 'failed'}.")
        shmem.barrier()
        json_writer.add_field("success", success)
        shmem.log("Validation completed")

    if args["benchmark"]:
        shmem.log("Benchmarking...")

        def zeroing_preamble():
            preamble()
            if algorithm == "atomics_all_reduce":
                for r in played:
                    shmem.on_rank(global_C, r).zero_()
                shmem.barrier()

        triton_ms = iris.do_bench(run_experiment, shmem.barrier, zeroing_preamble)
        triton_tflops = 2 * args["M"] * args["N"] * args["K"] * 1e-12 / (triton_ms * 1e-3)
        what = "all_scatter" if algorithm == "all_scatter" else "all_reduce"
        shmem.log_stats(f"tile matmul + {what} (grid={total_tiles}): {triton_ms:.3f} ms  {triton_tflops:.3f} tflops")
        json_writer.add_field("triton_tflops", triton_tflops)
        json_writer.add_field("triton_ms", triton_ms)
        json_writer.add_field("gemm_ms", timing["ms"] / timing["experiments"])
        json_writer.add_field("gemm_experiments", timing["experiments"])
        shmem.barrier()

    if rank == 0:
        json_writer.flush()
        json_writer.display()

    if args["trace_tiles"] and rank == 0:
        gpu_freq = shmem.wall_clock_rate(rank) * 1e-3
        stem = "gemm_tiles_all_scatter_trace" if algorithm == "all_scatter" else "gemm_all_reduce_tiles_trace"
        timestamps.to_json(f"{stem}_rank{rank}.json", gpu_freq)

    shmem.barrier()
    return json_writer.data
