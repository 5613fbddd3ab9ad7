#!/usr/bin/env python3
"""GEMM + atomics_all_reduce driver; CLI of the reference's examples/08_gemm_atomics_all_reduce/benchmark.py."""

import os
import sys

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

from examples.common.gemm_driver import main  # noqa: E402

if __name__ == "__main__":
    main("atomics_all_reduce")
