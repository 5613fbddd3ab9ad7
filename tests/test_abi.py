"""The C-ABI: the libraries load and export every symbol ``include/iris_amd.h``
(the product) and ``include/iris_amd_testing.h`` (test and bench kernels)
declare, and the ctypes structs have the layout the C compiler gives them.
No compute call is made."""

import ctypes
import os
import re
import subprocess
import sys

import pytest

from iris_amd import _native

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
HEADER = os.path.join(ROOT, "include", "iris_amd.h")
TESTING_HEADER = os.path.join(ROOT, "include", "iris_amd_testing.h")


def declared_functions(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(iris_[a-z0-9_]+|finegrained_hip[A-Za-z]+)\s*\(", text)))


def test_header_and_bindings_name_the_same_functions():
    names = declared_functions()
    lib_names = [n for n in names if n.startswith("iris_")]
    assert sorted(lib_names) == sorted(_native.SIGNATURES)
    assert sorted(n for n in names if n.startswith("finegrained_")) == sorted(_native.ALLOCATOR_SYMBOLS)
    assert declared_functions(TESTING_HEADER) == sorted(_native.TESTING_SIGNATURES)


def test_the_product_library_exports_no_test_or_probe_kernel():
    lib = ctypes.CDLL(_native.LIB_PATH)
    for name in _native.TESTING_SIGNATURES:
        assert not hasattr(lib, name), f"{name} belongs to libiris_amd_testing.so"


def test_libraries_load_and_export_every_declared_symbol():
    lib = _native.lib()
    for name in _native.SIGNATURES:
        assert getattr(lib, name) is not None
    assert lib.iris_amd_abi_version() == 5
    testing = _native.testing_lib()
    for name in _native.TESTING_SIGNATURES:
        assert getattr(testing, name) is not None
    alloc = ctypes.CDLL(_native.ALLOCATOR_LIB_PATH)
    for name in _native.ALLOCATOR_SYMBOLS:
        assert getattr(alloc, name) is not None


def test_struct_layout_matches_the_c_compiler(tmp_path):
    def probe(struct, cname):
        lines = [f'printf("%zu\\n", sizeof({cname}));']
        for fname, _ in struct._fields_:
            lines.append(f'printf("{fname} %zu\\n", offsetof({cname}, {fname}));')
        return "\n".join(lines)

    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "iris_amd.h"\nint main(void){\n'
        + probe(_native.GemmArgs, "iris_gemm_args") + 'printf("--\\n");' + probe(_native.ReduceArgs, "iris_reduce_args")
        + "return 0;}\n"
    )
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o",
                    str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    first, second = out.split("--\n")
    for struct, block in ((_native.GemmArgs, first), (_native.ReduceArgs, second)):
        rows = block.strip().splitlines()
        assert int(rows[0]) == ctypes.sizeof(struct)
        for row in rows[1:]:
            name, off = row.split()
            assert getattr(struct, name).offset == int(off), name


def test_error_strings_and_missing_library_is_loud(monkeypatch):
    assert b"invalid" in _native.lib().iris_hip_error_string(1).lower()
    with pytest.raises(RuntimeError, match="HIP error code 1"):
        _native.hip_try(1)
    _native.hip_try(0)
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", "/nonexistent/libiris_amd.so")
    with pytest.raises(RuntimeError, match="no other implementation"):
        _native.lib()


def test_launchers_reject_bad_arguments_without_a_device():
    lib = _native.lib()
    assert lib.iris_gemm_launch(None, None) == _native.HIP_ERROR_INVALID_VALUE
    g = _native.GemmArgs()  # all zero: no block sizes, no grid
    assert lib.iris_gemm_launch(ctypes.byref(g), None) == _native.HIP_ERROR_INVALID_VALUE
    g.block_m = g.block_n = g.group_size_m = g.num_sms = g.num_xcds = g.world_size = 1
    g.ab_dtype = 7  # no such operand type
    assert lib.iris_gemm_launch(ctypes.byref(g), None) == _native.HIP_ERROR_INVALID_VALUE
    g.ab_dtype, g.epilogue, g.c_global_dtype = _native.DTYPE_F32, _native.EPI_ALL_SCATTER, _native.DTYPE_BF16
    g.c_global = 1024  # (never dereferenced: fp32 operands need an fp32 output, which the launcher checks first)
    assert lib.iris_gemm_launch(ctypes.byref(g), None) == _native.HIP_ERROR_INVALID_VALUE
    g.c_global, g.epilogue = None, 0
    g.ab_dtype = _native.DTYPE_BF16
    g.num_sms, g.num_xcds = 12, 8  # the XCD remap needs an even split
    assert lib.iris_gemm_launch(ctypes.byref(g), None) == _native.HIP_ERROR_INVALID_VALUE
    r = _native.ReduceArgs()
    assert lib.iris_one_shot_reduce_launch(ctypes.byref(r), None) == _native.HIP_ERROR_INVALID_VALUE
    assert lib.iris_signal_tiles_launch(None, None, 4, 0, 0, 0, 0, None) == _native.HIP_ERROR_INVALID_VALUE
    assert lib.iris_memset_i32_launch(None, 0, -1, None) == _native.HIP_ERROR_INVALID_VALUE
    assert lib.iris_memset_i32_launch(None, 0, 0, None) == 0  # empty fill is a no-op


def test_host_build_of_the_kernel_tile_map_is_bit_exact():
    """The kernels' tile_map function, compiled for the host, against the
    oracle over whole tile grids (the same source is compiled for the
    device; the GPU tests check that build)."""
    from iris_amd import ops
    from oracle import iris_oracle as O

    for M, N, BM, BN, G in [(8192, 8192, 256, 256, 4), (8192, 8192, 256, 256, 6), (4096, 4096, 256, 256, 6),
                            (2048, 1376, 256, 64, 4), (1, 1376, 256, 256, 8), (1000, 999, 64, 64, 5),
                            (8192, 4608, 256, 64, 4), (768, 512, 256, 128, 6), (16384, 16384, 64, 64, 7),
                            (8192, 200, 32, 200, 3), (40, 40, 8, 8, 1), (256, 100000, 256, 16, 2)]:
        total = O.cdiv(M, BM) * O.cdiv(N, BN)
        want = O.tile_map_all(M, N, BM, BN, G)
        got = [ops.tile_map_host(t, M, N, BM, BN, G) for t in range(total)]
        assert got == [tuple(r) for r in want.tolist()]


def test_host_build_of_the_tile_map_beyond_the_multiply_high_bound():
    """Tile grids too large for the multiply-high constants (tile id times
    divisor no longer fits 32 bits) make the kernels divide instead: sampled
    tile ids of such grids, and of grids just inside the bound, against the
    oracle."""
    import random

    from iris_amd import ops
    from oracle import iris_oracle as O

    rng = random.Random(7)
    for M, N, BM, BN, G in [(40000, 40000, 1, 1, 8), (46000, 46000, 1, 1, 3), (3000, 90000, 1, 1, 7),
                            (46340, 46340, 1, 1, 1), (1 << 20, 2000, 512, 1, 5)]:
        total = O.cdiv(M, BM) * O.cdiv(N, BN)
        assert total < (1 << 31)
        ids = [0, 1, total - 1, total - 2] + [rng.randrange(total) for _ in range(400)]
        for t in ids:
            assert ops.tile_map_host(t, M, N, BM, BN, G) == O.tile_map(t, M, N, BM, BN, G), (t, M, N, G)


def test_host_build_of_the_stream_k_schedule_partitions_the_k_steps():
    """The kernels' stream-K run arithmetic, compiled for the host: the runs
    cut the launch's K-steps without gap or overlap, differ by at most one
    step, every tile has exactly one owner, and the owner's count of parts is
    the number of consecutive programs that hold the rest of its tile."""
    from iris_amd import ops

    for tiles, nk, programs in [(176, 64, 256), (24, 8, 5), (24, 8, 4), (5, 64, 8), (2, 128, 16), (20, 22, 24),
                                (1024, 16, 256), (300, 16, 256), (1, 40, 7), (7, 3, 21)]:
        sched = [ops.stream_k_schedule_host(tiles, nk, programs, pid) for pid in range(programs)]
        lengths = [sum(ke - kb for _, kb, ke, _ in items) for items in sched]
        assert sum(lengths) == tiles * nk and max(lengths) - min(lengths) <= 1
        assert lengths == sorted(lengths, reverse=True)  # the longer runs come first
        covered = {}
        g = 0  # global step the next item must start at
        for pid, items in enumerate(sched):
            for n, (tile, kb, ke, parts) in enumerate(items):
                assert 0 <= kb < ke <= nk and tile * nk + kb == g
                assert kb == 0 or n == 0  # only a run's first item starts inside a tile
                g = tile * nk + ke
                for k in range(kb, ke):
                    assert (tile, k) not in covered
                    covered[(tile, k)] = pid
                assert (parts == 0) == (kb != 0)
        assert g == tiles * nk and len(covered) == tiles * nk
        for pid, items in enumerate(sched):
            for tile, kb, ke, parts in items:
                if kb == 0:  # the owner: the rest of the tile is with the programs right after it
                    holders = sorted({covered[(tile, k)] for k in range(nk)})
                    assert holders == list(range(pid, pid + parts))
    with pytest.raises(ValueError):
        ops.stream_k_schedule_host(4, 4, 32, 0)  # runs would be empty
