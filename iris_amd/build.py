"""Build the shared libraries of the package with hipcc for gfx950.

    python -m iris_amd.build            # build what is out of date
    python -m iris_amd.build --force    # rebuild everything

``libiris_amd.so`` (HIP runtime helpers + kernel launchers) is written next to
this file, ``libfinegrained_allocator.so`` to ``csrc/finegrained_alloc/`` --
the place the reference's package looks for it (iris/__init__.py:29-38; built
there by setup.py:22-84 / csrc/finegrained_alloc/build.sh).
``libiris_amd_testing.so`` (``csrc/testing/``: measurement probes and unit-test
kernels that only the tests and bench.py call) is a library of its own, so
that the product library exports nothing but the product's entry points.
"""

from __future__ import annotations

import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = CSRC / "build"
LIB = PKG / "libiris_amd.so"
ALLOC_LIB = CSRC / "finegrained_alloc" / "libfinegrained_allocator.so"
TESTING_LIB = PKG / "libiris_amd_testing.so"

ARCH = "gfx950"
# packed-fp32 instructions are kept out of all device code
COMMON = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP libraries of iris_amd cannot be built")
    return exe


def kernel_sources():
    return sorted(p for p in CSRC.glob("*.hip"))


def testing_sources():
    return sorted(p for p in (CSRC / "testing").glob("*.hip"))


def _headers():
    inc = PKG.parent / "include"
    return list(CSRC.glob("*.hpp")) + [inc / "iris_amd.h", inc / "iris_amd_testing.h", inc / "iris_device.hpp"]


def _stale(target: Path, deps) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(map(str, cmd)) + "\n" + proc.stdout + proc.stderr)
    return proc


def build(force: bool = False, jobs: int | None = None, verbose: bool = True) -> None:
    cc = hipcc()
    OBJ.mkdir(parents=True, exist_ok=True)
    hdrs = _headers()
    jobs = jobs or min(8, os.cpu_count() or 1)

    todo = []
    objs, testing_objs = [], []
    for sources, into in ((kernel_sources(), objs), (testing_sources(), testing_objs)):
        for src in sources:
            obj = OBJ / (src.stem + ".o")
            into.append(obj)
            if force or _stale(obj, [src] + hdrs):
                todo.append((src, obj))

    def compile_one(item):
        src, obj = item
        _run([cc, *COMMON, "-c", str(src), "-o", str(obj)])
        return src.name

    if todo:
        with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
            for name in pool.map(compile_one, todo):
                if verbose:
                    print(f"[iris_amd.build] compiled {name}", flush=True)
    if force or todo or _stale(LIB, objs):
        _run([cc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)])
        if verbose:
            print(f"[iris_amd.build] linked {LIB.name}", flush=True)
    if force or todo or _stale(TESTING_LIB, testing_objs):
        _run([cc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(TESTING_LIB), *map(str, testing_objs)])
        if verbose:
            print(f"[iris_amd.build] linked {TESTING_LIB.name}", flush=True)

    alloc_src = CSRC / "finegrained_alloc" / "finegrained_allocator.hip"
    if force or _stale(ALLOC_LIB, [alloc_src]):
        _run([cc, *COMMON, "-Wall", "-Wextra", "-Werror", "-shared", "-o", str(ALLOC_LIB), str(alloc_src)])
        if verbose:
            print(f"[iris_amd.build] linked {ALLOC_LIB.name}", flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true")
    ap.add_argument("-j", "--jobs", type=int, default=None)
    args = ap.parse_args(argv)
    build(force=args.force, jobs=args.jobs)
    return 0


if __name__ == "__main__":
    sys.exit(main())
