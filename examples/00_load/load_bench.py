#!/usr/bin/env python3
"""Point-to-point microbenchmark "load"; CLI of the reference's examples/00_load/load_bench.py."""

import os
import sys

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

from examples.common.p2p_driver import main  # noqa: E402

if __name__ == "__main__":
    _, ok = main("load")
    sys.exit(0 if ok else 1)
