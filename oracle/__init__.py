"""CPU oracle for the fused GEMM + tile-publishing hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; it is the checker used by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``.
"""

from .iris_oracle import *  # noqa: F401,F403
