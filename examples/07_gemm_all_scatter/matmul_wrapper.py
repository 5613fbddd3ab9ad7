"""``matmul`` of the all_scatter example: same ``matmul.apply(...)`` signature as
the reference's examples/07_gemm_all_scatter/matmul_wrapper.py, HIP kernel underneath."""

import os
import sys

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

from iris_amd.matmul import matmul_all_scatter as matmul  # noqa: E402

__all__ = ["matmul"]
