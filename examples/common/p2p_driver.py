"""Shared driver of the point-to-point microbenchmarks.

One ``main(kind)`` stands in for the reference's six scripts
(examples/00_load/load_bench.py, 01_store/store_bench.py,
02_all_load/all_load_bench.py, 03_all_store/all_store_bench.py,
04_atomic_add/atomic_add_bench.py, 05_atomic_xchg/atomic_xchg_bench.py):
the same command-line flags, timing protocol (``do_bench`` of the kernel,
minus ``do_bench`` of a local store kernel where the reference subtracts one),
validation, tables and JSON records.  The kernels are HIP kernels over
``include/iris_device.hpp`` (``iris_p2p_bench_launch``).

``--virtual_ranks P`` (new) lets the one GPU play P ranks, each launch in its
turn; the figures are then bandwidths of the local HBM through the symmetric
heap's address translation, not of a link.
"""

import argparse
import json
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

import iris_amd as iris  # noqa: E402
from iris_amd import ops  # noqa: E402

DATATYPES = {"int8": torch.int8, "fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32,
             "int32": torch.int32}

# kind: (pairwise?, default datatype, choices, flag of --num_experiments, its default, default warm-ups,
#        default heap size, table label)
KINDS = {
    "load": (True, "fp16", ("int8", "fp16", "bf16", "fp32"), "-n", 10, 1, 1 << 33,
             "Unidirectional LOAD bandwidth GiB/s [Remote read]"),
    "store": (True, "fp16", ("int8", "fp16", "bf16", "fp32"), "-n", 10, 1, 1 << 33,
              "Unidirectional STORE bandwidth GiB/s [Remote write]"),
    "atomic_add": (True, "fp16", ("fp16", "fp32", "bf16", "int32"), "-x", 16, 4, 1 << 33,
                   "Unidirectional ATOMIC_ADD bandwidth GiB/s [Remote atomic]"),
    "atomic_xchg": (True, "int32", ("fp16", "fp32", "bf16", "int32"), "-x", 16, 4, 1 << 33,
                    "Unidirectional ATOMIC_XCHG bandwidth GiB/s [Remote atomic]"),
    "all_load": (False, "fp16", ("fp16", "fp32", "int8", "bf16"), "-x", 20, 2, 1 << 36,
                 "Total Bandwidth (GiB/s) vs Buffer Size"),
    "all_store": (False, "fp16", ("fp16", "fp32", "int8", "bf16"), "-x", 20, 2, 1 << 36,
                  "Total Bandwidth (GiB/s) vs Buffer Size"),
}


def parse_args(kind, argv=None):
    pairwise, dt, choices, nflag, nexp, nwarm, heap, _ = KINDS[kind]
    parser = argparse.ArgumentParser(description="Parse Message Passing configuration.",
                                     formatter_class=argparse.ArgumentDefaultsHelpFormatter)
    parser.add_argument("-t", "--datatype", type=str, default=dt, choices=list(choices), help="Datatype of computation")
    if pairwise:
        parser.add_argument("-z", "--buffer_size", type=int, default=1 << 32, help="Buffer Size")
    else:
        parser.add_argument("-m", "--buffer_size_min", type=int, default=1 << 20, help="Minimum buffer size")
        parser.add_argument("-M", "--buffer_size_max", type=int, default=1 << 32, help="Maximum buffer size")
        parser.add_argument("-a", "--active_ranks", type=int, default=8, help="Number of active ranks")
    parser.add_argument("-b", "--block_size", type=int, default=512, help="Block Size")
    parser.add_argument("-v", "--verbose", action="store_true", help="Enable verbose output")
    parser.add_argument("-d", "--validate", action="store_true", help="Enable validation output")
    parser.add_argument("-p", "--heap_size", type=int, default=heap, help="Iris heap size")
    parser.add_argument("-o", "--output_file", type=str, default="", help="Output file")
    parser.add_argument(nflag, "--num_experiments", type=int, default=nexp, help="Number of experiments")
    parser.add_argument("-w", "--num_warmup", type=int, default=nwarm, help="Number of warmup iterations")
    parser.add_argument("--virtual_ranks", type=int, default=1, help="Ranks played by this one GPU")
    return vars(parser.parse_args(argv))


def _expected_index(n, dtype):
    """Element i holds i, converted the way the kernels convert it (wrapping for int8)."""
    return torch.arange(n, device="cuda").to(dtype)


def _check(shmem, got, want, verbose):
    """torch.allclose(atol=1) with the first mismatch logged, as the reference's scripts do."""
    got, want = got.double(), want.double()
    if torch.allclose(got, want, atol=1):
        if verbose:
            shmem.log("Validation successful.")
        return True
    shmem.log(f"Max absolute difference: {(got - want).abs().max().item()}")
    idx = int(torch.nonzero(~torch.isclose(got, want, atol=1))[0])
    shmem.log(f"Mismatch at index ({idx},): C={got[idx]}, expected={want[idx]}")
    if verbose:
        shmem.log("Validation failed.")
    return False


def bench_pair(kind, shmem, src, dst, buffer, result, args):
    """One (source rank, destination rank) cell: launches run as rank ``src``
    and address rank ``dst``.  Returns (GiB/s, validation ok)."""
    hb, nr = shmem.get_heap_bases(), shmem.get_num_ranks()
    n, bs = buffer.numel(), args["block_size"]
    buf_s, res_s = shmem.on_rank(buffer, src), shmem.on_rank(result, src)
    if args["verbose"]:
        shmem.log(f"Measuring bandwidth between the ranks {src} and {dst}...")

    def run():
        ops.p2p_bench(kind, buf_s, res_s, hb, src, dst, nr, block_size=bs)

    def run_local_store():
        ops.p2p_bench("local_store", None, res_s, None, src, src, nr, block_size=bs)

    def reset():
        if kind in ("store", "atomic_add", "atomic_xchg"):
            shmem.on_rank(buffer, dst).zero_()

    ms = iris.do_bench(run, shmem.barrier, reset, n_repeat=args["num_experiments"], n_warmup=args["num_warmup"])
    if kind == "load":  # the reference subtracts the local store of the result (load_bench.py:149-153)
        ms -= iris.do_bench(run_local_store, shmem.barrier, n_repeat=args["num_experiments"],
                            n_warmup=args["num_warmup"])
    total_bytes = n * buffer.element_size()
    # (as in the reference, a buffer too small to time against the baseline gives a meaningless figure)
    gibps = total_bytes / (ms * 1e-3) / 2**30 if ms != 0 else float("inf")
    if args["verbose"]:
        shmem.log(f"Copied {total_bytes / 2**30:.2f} GiB in {ms * 1e-3:.4f} seconds")
        shmem.log(f"Bandwidth between {src} and {dst} is {gibps:.4f} GiB/s")

    ok = True
    if args["validate"]:
        if args["verbose"]:
            shmem.log("Validating output...")
        reset()
        run()
        shmem.barrier()
        if kind == "load":      # the source buffer holds its own index on every rank
            ok = _check(shmem, res_s, _expected_index(n, buffer.dtype), args["verbose"])
        elif kind == "store":
            ok = _check(shmem, shmem.on_rank(buffer, dst), _expected_index(n, buffer.dtype), args["verbose"])
        elif kind == "atomic_add":
            ok = _check(shmem, shmem.on_rank(buffer, dst), torch.ones_like(buffer), args["verbose"])
        else:  # atomic_xchg: the old values come back, ones stay behind
            ok = _check(shmem, res_s, torch.zeros_like(buffer), args["verbose"]) and \
                _check(shmem, shmem.on_rank(buffer, dst), torch.ones_like(buffer), args["verbose"])
    return gibps, ok


def bench_all(kind, shmem, rank, buffer, result, args):
    """One (buffer size, rank) cell of the all-to-one benchmarks."""
    hb, nr = shmem.get_heap_bases(), shmem.get_num_ranks()
    n, bs = buffer.numel(), args["block_size"]
    buf_r, res_r = shmem.on_rank(buffer, rank), shmem.on_rank(result, rank)
    active = rank < args["active_ranks"]

    def run():
        if active:
            ops.p2p_bench(kind, buf_r, res_r, hb, rank, -1, nr, block_size=bs)

    def run_local_store():
        ops.p2p_bench("local_store", None, res_r, None, rank, rank, nr, block_size=bs)

    ms = iris.do_bench(run, shmem.barrier, n_repeat=args["num_experiments"], n_warmup=args["num_warmup"])
    if kind == "all_load":  # minus the local store of the sums (all_load_bench.py:171-186)
        store_ms = iris.do_bench(run_local_store, shmem.barrier, n_repeat=args["num_experiments"],
                                 n_warmup=args["num_warmup"])
        if args["verbose"]:
            shmem.log(f"Total time: {ms:.4f} ms, Store overhead: {store_ms:.4f} ms, Net all_get time: {ms - store_ms:.4f} ms")
        ms -= store_ms
    total_bytes = n * buffer.element_size() * (nr - 1)
    gibps = (total_bytes / (ms * 1e-3) / 2**30 if ms != 0 else float("inf")) if active else 0.0
    if args["verbose"]:
        shmem.log(f"Total bandwidth for rank {rank} is {gibps:.4f} GiB/s")

    ok = True
    if args["validate"] and active:
        run()
        shmem.barrier()
        if kind == "all_load":
            # every rank's buffer holds index / num_ranks, so that the sum over ranks is the index again
            want = sum(shmem.on_rank(buffer, r).float() for r in range(nr)).to(buffer.dtype)
            ok = _check(shmem, res_r, want, args["verbose"])
        else:
            for r in range(nr):
                if r != rank:
                    ok = ok and _check(shmem, shmem.on_rank(buffer, r), _expected_index(n, buffer.dtype),
                                       args["verbose"])
    return gibps, ok


def print_pair_matrix(matrix, label, output_file):
    """Table and JSON records of load_bench.py:198-232."""
    nr = matrix.shape[0]
    print(f"\n{label}")
    print(" SRC\\DST ".ljust(10) + "".join(f"GPU {d:02d}".rjust(10) for d in range(nr)))
    for s in range(nr):
        print(f"GPU {s:02d}  ->".ljust(10) + "".join(f"{matrix[s, d]:10.2f}" for d in range(nr)))
    if output_file:
        if not output_file.endswith(".json"):
            raise ValueError(f"Unsupported output file extension: {output_file}")
        records = [{"source_gpu": f"GPU_{s:02d}", "destination_gpu": f"GPU_{d:02d}", "source_rank": s,
                    "destination_rank": d, "bandwidth_gbps": float(matrix[s, d])}
                   for s in range(nr) for d in range(nr)]
        with open(output_file, "w") as f:
            json.dump(records, f, indent=2)


def print_size_table(data, sizes, label, output_file):
    """Table and JSON records of all_load_bench.py:231-299."""
    nr = len(data)
    headers = ["Size (MiB)", "log2(bytes)"] + [f"GPU {i:02d}" for i in range(nr)]
    rows = [[f"{sz / 1024 / 1024:.1f}", f"{int(np.log2(sz))}"] + [f"{data[r][i]:.2f}" for r in range(nr)]
            for i, sz in enumerate(sizes)]
    widths = [max(len(h), *(len(row[c]) for row in rows)) for c, h in enumerate(headers)]
    line = " | ".join(f"{h:>{w}}" for h, w in zip(headers, widths))
    print(f"\n{label}\n{line}\n" + "-" * len(line))
    for row in rows:
        print(" | ".join(f"{v:>{w}}" for v, w in zip(row, widths)))
    if output_file:
        if not output_file.endswith(".json"):
            raise ValueError(f"Unsupported output file extension: {output_file}")
        records = [{"buffer_size_bytes": sz, "buffer_size_mib": sz / 1024 / 1024, "log2_bytes": int(np.log2(sz)),
                    "gpu_rank": r, "gpu_id": f"GPU_{r:02d}", "bandwidth_gbps": float(data[r][i])}
                   for i, sz in enumerate(sizes) for r in range(nr)]
        with open(output_file, "w") as f:
            json.dump(records, f, indent=2)


def main(kind, argv=None):
    torch.manual_seed(123)
    args = parse_args(kind, argv)
    pairwise, *_, label = KINDS[kind]
    shmem = iris.iris(args["heap_size"], virtual_ranks=args["virtual_ranks"])
    nr = shmem.get_num_ranks()
    dtype = DATATYPES[args["datatype"]]
    es = torch.tensor([], dtype=dtype).element_size()
    ok = True

    if pairwise:
        n = args["buffer_size"] // es
        buffer = shmem.zeros(n, device="cuda", dtype=dtype)
        result = shmem.zeros_like(buffer)
        if kind == "load":
            for r in range(nr):
                shmem.on_rank(buffer, r).copy_(_expected_index(n, dtype))
        matrix = np.zeros((nr, nr), dtype=np.float32)
        for s in range(nr):
            for d in range(nr):
                matrix[s, d], good = bench_pair(kind, shmem, s, d, buffer, result, args)
                ok = ok and good
                shmem.barrier()
        if shmem.get_rank() == 0:
            print_pair_matrix(matrix, label, args["output_file"])
        return matrix, ok

    sizes = []
    size = args["buffer_size_min"]
    while size <= args["buffer_size_max"]:
        sizes.append(size)
        size *= 2
    full = shmem.zeros(args["buffer_size_max"] // es, device="cuda", dtype=dtype)
    full_result = shmem.zeros_like(full)
    data = [[0.0] * len(sizes) for _ in range(nr)]
    for i, size in enumerate(sizes):
        n = size // es
        buffer, result = full[:n], full_result[:n]
        if kind == "all_load":
            for r in range(nr):
                shmem.on_rank(buffer, r).copy_((torch.arange(n, device="cuda", dtype=torch.float32) / nr).to(dtype))
        for r in range(nr):
            if kind == "all_store":
                for q in range(nr):
                    shmem.on_rank(buffer, q).zero_()
            data[r][i], good = bench_all(kind, shmem, r, buffer, result, args)
            ok = ok and good
        shmem.barrier()
    if shmem.get_rank() == 0:
        print_size_table(data, sizes, label, args["output_file"])
    return data, ok
