#!/usr/bin/env python3
"""Point-to-point microbenchmark "all_store"; CLI of the reference's examples/03_all_store/all_store_bench.py."""

import os
import sys

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

from examples.common.p2p_driver import main  # noqa: E402

if __name__ == "__main__":
    _, ok = main("all_store")
    sys.exit(0 if ok else 1)
