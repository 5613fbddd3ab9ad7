"""Host side of the symmetric heap: the ``iris.iris(heap_size)`` context.

Drop-in for the reference's ``Iris`` class (iris/iris.py:31-314, factory
:524-534): same constructor, tensor factories, accessors, defaults and error
behaviour.  What differs is underneath:

* the heap is one fine-grained HBM allocation made through the C-ABI shim
  (``hipExtMallocWithFlags(hipDeviceMallocFinegrained)``) and handed to torch
  zero-copy; the rest of the process keeps torch's own caching allocator.
  ``IRIS_AMD_PLUGGABLE_ALLOCATOR=1`` instead routes *every* torch allocation
  through the plug-in, as the reference does (iris/__init__.py:40-45);
* ranks come in two kinds.  Several processes (one rank each, started by
  ``torchrun``, by an MPI launcher when mpi4py is there, or with
  ``IRIS_AMD_RENDEZVOUS``; see ``_bootstrap.py``) exchange the IPC handles and
  base addresses of their heaps through a host-side store and map each
  other's heaps, as the reference does over MPI (iris/iris.py:53-77).  Or one
  process plays every rank: ``virtual_ranks=P`` carves one allocation into P
  equal sub-heaps, so that ``heap_bases``/pointer translation, flags and
  partial buffers behave exactly as with P processes.  Either way an
  allocation advances every rank's heap alike, which is the symmetric-heap
  property.
"""

from __future__ import annotations

import math
import os

import numpy as np
import torch

from . import _bootstrap, _hip

STATS = True
LOGGING = True
DEBUG = False

_TORCH_TYPESTR = "|i1"


class _DeviceBytes:
    """Zero-copy window on raw device memory for ``torch.as_tensor``, and the
    owner of that memory: torch keeps a reference to this object for as long as
    any tensor views the storage, and the allocation is released when the last
    of them is gone (the reference's pool is a torch tensor with the same
    lifetime, iris/iris.py:48)."""

    def __init__(self, ptr: int, nbytes: int, owns: bool = False):
        self._ptr = ptr if owns else None
        self.__cuda_array_interface__ = {
            "shape": (nbytes,),
            "typestr": _TORCH_TYPESTR,
            "data": (ptr, False),
            "strides": None,
            "version": 3,
        }

    def __del__(self):
        ptr, self._ptr = self._ptr, None
        if ptr is None:
            return
        try:
            _hip.device_synchronize()  # no kernel may still be using the heap
            _hip.hip_free(ptr)
        except Exception:  # interpreter shutdown: the driver reclaims the memory
            pass


def _finegrained_pool(nbytes: int, device: str) -> torch.Tensor:
    """int8[nbytes] on fine-grained device memory."""
    if os.environ.get("IRIS_AMD_PLUGGABLE_ALLOCATOR") == "1":
        # every torch allocation is fine-grained in this mode (see __init__)
        return torch.empty(nbytes, device=device, dtype=torch.int8)
    ptr = _hip.malloc_fine_grained(nbytes)
    return torch.as_tensor(_DeviceBytes(ptr.value, nbytes, owns=True), device=device)


# hipIpcOpenMemHandle has been seen not to return for larger allocations
_IPC_MAX_BYTES = (2 << 30) - 1
# the largest heap a launcher should default to with one process per rank: 2 GiB less one allocation unit
IPC_MAX_HEAP_BYTES = (2 << 30) - (1 << 20)


class Iris:
    def __init__(self, heap_size=1 << 30, *, virtual_ranks=None, cur_rank=0, _pool_factory=None, _comm=None):
        self._peer_pools = None
        if virtual_ranks is None and "IRIS_AMD_VIRTUAL_RANKS" not in os.environ and _pool_factory is None:
            comm = _comm if _comm is not None else _bootstrap.init_comm()
            if comm is not None and comm.size > 1:
                self._init_multi_process(heap_size, comm)
                return
        if virtual_ranks is None:
            virtual_ranks = int(os.environ.get("IRIS_AMD_VIRTUAL_RANKS", "1"))
        if virtual_ranks < 1 or not (0 <= cur_rank < virtual_ranks):
            raise ValueError(f"invalid rank layout: cur_rank={cur_rank}, virtual_ranks={virtual_ranks}")
        self.comm = None
        self.num_ranks = virtual_ranks
        self.cur_rank = cur_rank
        self.heap_size = heap_size
        self.heap_offset = 0
        self.alignment = 1024

        if _pool_factory is None:
            num_gpus = _hip.count_devices()
            self.gpu_id = cur_rank % num_gpus
            _hip.set_device(self.gpu_id)
            self.device = f"cuda:{self.gpu_id}"
            self._pool_all = _finegrained_pool(heap_size * virtual_ranks, self.device)
        else:
            # test seam: the pool comes from the caller (host memory on a
            # machine without a GPU); nothing in the package passes it
            self.gpu_id = 0
            self._pool_all = _pool_factory(heap_size * virtual_ranks)
            self.device = str(self._pool_all.device)
        base = self._pool_all.data_ptr()
        self._bases = [base + r * heap_size for r in range(virtual_ranks)]
        self.memory_pool = self._pool_all[cur_rank * heap_size:(cur_rank + 1) * heap_size]
        for r, b in enumerate(self._bases):
            self.log_debug(f"GPU {r}: Heap base {hex(b)}")
        self.heap_bases = torch.from_numpy(np.array(self._bases, dtype=np.uint64)).to(
            device=self.device, dtype=torch.uint64
        )

    def _init_multi_process(self, heap_size, comm):
        """One rank per process: iris/iris.py:32-79 with the store (or MPI) of
        ``_bootstrap`` in the place of the MPI helpers."""
        if heap_size > _IPC_MAX_BYTES and os.environ.get("IRIS_AMD_ALLOW_LARGE_IPC") != "1":
            raise ValueError(
                f"heap_size {heap_size}: a heap that peers map through IPC must stay under 2 GiB here "
                "(set IRIS_AMD_ALLOW_LARGE_IPC=1 to try a larger one)"
            )
        self.comm = comm
        self.num_ranks, self.cur_rank = comm.size, comm.rank
        self.heap_size, self.heap_offset, self.alignment = heap_size, 0, 1024
        self.gpu_id = self.cur_rank % _hip.count_devices()
        _hip.set_device(self.gpu_id)
        self.device = f"cuda:{self.gpu_id}"
        # peers keep this memory mapped: like the reference's pool it is never handed back
        ptr = _hip.malloc_fine_grained(heap_size)
        self._pool_all = torch.as_tensor(_DeviceBytes(ptr.value, heap_size), device=self.device)
        self.memory_pool = self._pool_all
        handle = _hip.get_ipc_handle(ptr, self.cur_rank)
        comm.barrier()
        all_handles = comm.allgather(handle)
        all_bases = comm.allgather(np.array([ptr.value], dtype=np.uint64))
        comm.barrier()
        assert int(all_bases[self.cur_rank][0]) == ptr.value
        self._bases, self._peer_pools = [], []
        for rank in range(self.num_ranks):
            if rank == self.cur_rank:
                self._bases.append(ptr.value)
                self._peer_pools.append(self._pool_all)
            else:
                mapped = _hip.open_ipc_handle(np.ascontiguousarray(all_handles[rank]), self.cur_rank)
                self._bases.append(int(mapped))
                self._peer_pools.append(torch.as_tensor(_DeviceBytes(int(mapped), heap_size), device=self.device))
        for r, b in enumerate(self._bases):
            self.log_debug(f"GPU {r}: Heap base {hex(b)}")
        comm.barrier()
        self.heap_bases = torch.from_numpy(np.array(self._bases, dtype=np.uint64)).to(
            device=self.device, dtype=torch.uint64
        )
        comm.barrier()

    # ------------------------------------------------------------------ logging
    def _say(self, message):
        print(f"[Iris] [{self.cur_rank}/{self.num_ranks}] {message}")

    def log(self, message):
        if LOGGING:
            self._say(message)

    def log_debug(self, message):
        if DEBUG:
            self._say(message)

    def log_stats(self, message):
        if STATS:
            self._say(message)

    def broadcast(self, source_rank, value):
        # Callers pass (value, rank): the reference forwards the pair
        # positionally to a (value, root) helper, iris/iris.py:93-94.  With
        # one process holding every rank the root's value is the caller's.
        if self.comm is not None:
            return self.comm.broadcast_scalar(source_rank, value)
        return source_rank

    # --------------------------------------------------------------- allocation
    def allocate(self, num_elements, dtype):
        """Bump allocation, 1 KiB granularity, never freed (iris/iris.py:96-110)."""
        self.log_debug(f"allocate: num_elements = {num_elements}, dtype = {dtype}")
        element_size = torch.tensor([], dtype=dtype).element_size()
        size_in_bytes = num_elements * element_size
        aligned_size = math.ceil(size_in_bytes / self.alignment) * self.alignment
        if self.heap_offset + aligned_size > self.heap_size:
            raise MemoryError("Heap out of memory")
        start = self.heap_offset
        self.heap_offset += aligned_size
        return self.memory_pool[start:start + size_in_bytes].view(dtype).reshape((num_elements,))

    def deallocate(self, pointer):
        pass

    def parse_size(self, size):
        if len(size) == 1 and isinstance(size[0], (tuple, list)):
            size = size[0]
        return size, math.prod(size)

    def _take(self, size, dtype, out=None):
        """(flat tensor, shape): a fresh allocation, or the validated ``out``."""
        size, num_elements = self.parse_size(size)
        if out is not None:
            self.__throw_if_invalid_output_tensor(out, num_elements, dtype)
            return out, size
        return self.allocate(num_elements=num_elements, dtype=dtype), size

    # ----------------------------------------------------------------- factories
    def zeros(self, *size, dtype=torch.int, device=None, requires_grad=False, **kwargs):
        self.log_debug(f"zeros: size = {size}, dtype = {dtype}, device = {device}, requires_grad = {requires_grad}")
        tensor, size = self._take(size, dtype)
        tensor.zero_()
        if requires_grad:
            tensor.requires_grad_()
        return tensor.reshape(size)

    def zeros_like(self, tensor):
        new_tensor = self.allocate(tensor.numel(), tensor.dtype)
        new_tensor.zero_()
        return new_tensor

    def ones(self, *size, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
        self.log_debug(f"ones: size = {size}, dtype = {dtype}, device = {device}, requires_grad = {requires_grad}")
        if dtype is None:
            dtype = torch.get_default_dtype()
        tensor, size = self._take(size, dtype, out)
        tensor.fill_(1)
        if requires_grad:
            tensor.requires_grad_()
        return tensor.reshape(size)

    def full(self, size, fill_value, dtype=torch.int):
        self.log_debug(f"full: size = {size}, fill_value = {fill_value}, dtype = {dtype}")
        tensor, size = self._take(size, dtype)
        tensor.fill_(fill_value)
        return tensor.reshape(size)

    def empty(self, size, dtype=torch.float):
        self.log_debug(f"empty: size = {size}, dtype = {dtype}")
        tensor, size = self._take(size, dtype)
        return tensor.reshape(size)

    def uniform(self, size, low=0.0, high=1.0, dtype=torch.float):
        self.log_debug(f"uniform: size = {size}, low = {low}, high = {high}, dtype = {dtype}")
        tensor, size = self._take(size, dtype)
        tensor.uniform_(low, high)
        return tensor.reshape(size)

    def randn(self, *size, generator=None, dtype=torch.float, layout=torch.strided, device=None,
              requires_grad=False, pin_memory=False):
        self.log_debug(
            f"randn: size = {size}, dtype = {dtype}, device = {device}, requires_grad = {requires_grad}, "
            f"pin_memory = {pin_memory}"
        )
        tensor, size = self._take(size, dtype)
        # drawn with torch on `device` (host when None), then copied into the heap
        tensor.copy_(torch.randn(tensor.numel(), generator=generator, dtype=dtype, device=device, layout=layout))
        if requires_grad:
            tensor.requires_grad_()
        return tensor.reshape(size)

    def randint(self, size, low, high, dtype=torch.int):
        self.log_debug(f"randint: size = {size}, low = {low}, high = {high}, dtype = {dtype}")
        tensor, size = self._take(size, dtype)
        tensor[:] = torch.randint(low, high, (tensor.numel(),), device=self.device, dtype=dtype)
        return tensor.reshape(size)

    def linspace(self, start, end, steps, dtype=torch.float):
        self.log_debug(f"linspace: start = {start}, end = {end}, steps = {steps}, dtype = {dtype}")
        tensor = self.allocate(num_elements=int(steps), dtype=dtype)
        torch.linspace(start, end, int(steps), out=tensor, dtype=dtype, device=self.device)
        return tensor

    def arange(self, start=0, end=None, step=1, out=None, dtype=None, layout=torch.strided, device=None,
               requires_grad=False):
        """Values of [start, end) with common difference ``step``, on the heap."""
        self.log_debug(f"arange: start = {start}, end = {end}, step = {step}, dtype = {dtype}")
        if end is None:
            start, end = 0, start
        num_elements = math.ceil((end - start) / step)
        if dtype is None:
            is_float = any(isinstance(x, float) for x in (start, end, step))
            dtype = torch.get_default_dtype() if is_float else torch.int64
        tensor, _ = self._take((num_elements,), dtype, out)
        tensor[:] = torch.arange(start, end, step, dtype=dtype, device=self.device)
        if requires_grad:
            tensor.requires_grad_()
        return tensor

    # ----------------------------------------------------------------- accessors
    def get_heap_bases(self):
        return self.heap_bases

    def barrier(self):
        # all queued device work done, then meet the other processes, if any
        # (iris/iris.py:272-276)
        if self._pool_all.is_cuda:
            torch.cuda.synchronize()
        if self.comm is not None:
            self.comm.barrier()

    def get_device(self):
        return self.memory_pool.device

    def get_cu_count(self):
        return _hip.get_cu_count(self.gpu_id)

    def get_rank(self):
        return self.cur_rank

    def get_num_ranks(self):
        return self.num_ranks

    def wall_clock_rate(self, rank):
        return _hip.get_wall_clock_rate(self.gpu_id)

    # ------------------------------------------------------------ virtual ranks
    def on_rank(self, tensor: torch.Tensor, rank: int) -> torch.Tensor:
        """The tensor at the same heap offset on (virtual) rank ``rank``.

        What a peer's IPC-mapped heap gives a process of the reference: the
        address ``translate(ptr, cur_rank, rank)`` (iris/iris.py:317-339) as
        a tensor of the same shape, dtype and strides.
        """
        if not (0 <= rank < self.num_ranks):
            raise ValueError(f"rank {rank} out of range [0, {self.num_ranks})")
        if not self.__on_symmetric_heap(tensor):
            raise RuntimeError("The tensor is not on the symmetric heap")
        off = tensor.data_ptr() - self._bases[self.cur_rank]
        es = tensor.element_size()
        if self._peer_pools is not None:  # one process per rank: the peer's heap as mapped here
            window = self._peer_pools[rank][off:]
        else:
            window = self._pool_all[rank * self.heap_size + off:(rank + 1) * self.heap_size]
        typed = window[:(window.numel() // es) * es].view(tensor.dtype)
        return typed.as_strided(tensor.size(), tensor.stride())

    # ------------------------------------------------------------------- checks
    def __throw_if_invalid_output_tensor(self, tensor: torch.Tensor, num_elements: int, dtype: torch.dtype):
        if not self.__tensor_on_device(tensor):
            raise RuntimeError(
                f"The output tensor is not on the same device as the Iris instance. The Iris instance is on device "
                f"{self.device} but the output tensor is on device {tensor.device}"
            )
        if not self.__on_symmetric_heap(tensor):
            raise RuntimeError(
                f"The output tensor is not on the symmetric heap. The Iris instance is on heap base "
                f"{self._bases[self.cur_rank]} but the output tensor is on heap base {tensor.data_ptr()}"
            )
        if tensor.numel() != num_elements:
            raise RuntimeError(f"The output tensor has {tensor.numel()} elements, but {num_elements} are required")
        if tensor.dtype != dtype:
            raise RuntimeError(f"The output tensor has dtype {tensor.dtype}, but {dtype} is required")

    def __tensor_on_device(self, tensor: torch.Tensor):
        return tensor.device == torch.device(self.device)

    def __on_symmetric_heap(self, tensor: torch.Tensor):
        base = self._bases[self.cur_rank]
        return base <= tensor.data_ptr() < base + self.heap_size


def iris(heap_size=1 << 30, **kwargs):
    """Create the Iris context with a heap of ``heap_size`` bytes (per rank)."""
    return Iris(heap_size, **kwargs)
