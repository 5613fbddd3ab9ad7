"""``matmul`` of the one_shot_all_reduce example: same ``matmul.apply(...)`` signature as
the reference's examples/09_gemm_one_shot_all_reduce/matmul_wrapper.py, HIP kernel underneath."""

import os
import sys

sys.path.insert(0, os.path.abspath(os.path.join(os.path.dirname(__file__), "..", "..")))

from iris_amd.matmul import matmul_one_shot_all_reduce as matmul  # noqa: E402

__all__ = ["matmul"]
