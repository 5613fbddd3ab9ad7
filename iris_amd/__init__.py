"""iris_amd -- the Iris host API over an MI355X-native fused GEMM + tile-publishing path.

``import iris_amd as iris`` gives the names the reference package exports for
this path (iris/__init__.py:9-26): ``iris.iris(heap_size)``, ``Iris``,
``do_bench`` and ``memset_tensor``.  The device-side primitives of the
reference are Triton functions; here they live inside the HIP kernels
(``csrc/``), reached through ``iris_amd.ops`` and the examples' ``matmul``
wrappers.

Set ``IRIS_AMD_PLUGGABLE_ALLOCATOR=1`` before the first import to make *every*
torch device allocation fine-grained through the allocator plug-in, as the
reference does (iris/__init__.py:29-45); by default only the symmetric heap
is.
"""

import os as _os

# One process per rank: peers map each other's heaps through hipIpcOpenMemHandle, and on hosts whose driver
# only supports dmabuf IPC that needs HSA_ENABLE_IPC_MODE_LEGACY=0 in the environment before the HIP runtime
# initialises (else hipIpcGetMemHandle fails with "invalid argument").  A value the user set is kept.
_os.environ.setdefault("HSA_ENABLE_IPC_MODE_LEGACY", "0")

from . import _native  # noqa: E402
from ._bootstrap import launched_as_ranks  # noqa: E402
from .iris import IPC_MAX_HEAP_BYTES, Iris, iris  # noqa: E402
from .util import do_bench, memset_tensor  # noqa: E402

__all__ = ["Iris", "iris", "do_bench", "memset_tensor", "use_finegrained_allocator", "launched_as_ranks",
           "IPC_MAX_HEAP_BYTES"]


def use_finegrained_allocator():
    """Route all of torch's device allocations through the fine-grained
    plug-in.  Must run before the first device allocation of the process."""
    import torch

    path = _native.ALLOCATOR_LIB_PATH
    if not _os.path.exists(path):
        raise RuntimeError(
            f"Fine-grained allocator library not found at {path}. Build it with `python -m iris_amd.build`."
        )
    allocator = torch.cuda.memory.CUDAPluggableAllocator(path, "finegrained_hipMalloc", "finegrained_hipFree")
    torch.cuda.memory.change_current_allocator(allocator)
    return allocator


if _os.environ.get("IRIS_AMD_PLUGGABLE_ALLOCATOR") == "1":
    use_finegrained_allocator()
