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

from . import _native
from .iris import Iris, iris
from .util import do_bench, memset_tensor

__all__ = ["Iris", "iris", "do_bench", "memset_tensor", "use_finegrained_allocator"]


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
