#!/usr/bin/env python3
"""Point-to-point microbenchmark "atomic_add"; CLI of the reference's examples/04_atomic_add/atomic_add_bench.py."""

import os
import sys

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

from examples.common.p2p_driver import main  # noqa: E402

if __name__ == "__main__":
    _, ok = main("atomic_add")
    sys.exit(0 if ok else 1)
