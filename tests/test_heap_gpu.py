"""The Iris context on the GPU: fine-grained heap through the C-ABI shim,
factories, heap bases, device facts."""

import ctypes

import pytest
import torch

import iris_amd
from iris_amd import _hip, _native

pytestmark = pytest.mark.gpu


def test_device_facts():
    assert _hip.count_devices() >= 1
    dev = _hip.get_device_id()
    assert _hip.get_arch_name(dev).startswith("gfx950")
    assert _hip.get_cu_count(dev) == 256
    assert _hip.get_wall_clock_rate(dev) == 100000  # kHz: the 100 MHz constant clock


def test_heap_is_device_memory_torch_can_use(shmem):
    assert shmem.get_device().type == "cuda"
    hb = shmem.get_heap_bases()
    assert hb.is_cuda and hb.dtype == torch.uint64 and hb.numel() == 8
    bases = hb.cpu().view(torch.int64).tolist()
    assert bases[0] == shmem.memory_pool.data_ptr() and all(b - a == shmem.heap_size for a, b in zip(bases, bases[1:]))
    z = shmem.zeros((128, 64), dtype=torch.bfloat16)
    assert z.is_cuda and float(z.float().abs().sum()) == 0.0
    o = shmem.ones(1000, dtype=torch.float32)
    assert float(o.sum()) == 1000.0
    r = shmem.randn(64, 32, device="cuda", dtype=torch.float16)
    assert r.shape == (64, 32) and float(r.float().std()) > 0.5
    a = shmem.arange(0, 10, 2)
    assert a.cpu().tolist() == [0, 2, 4, 6, 8]
    x = shmem.full((4,), 3, dtype=torch.int32)
    y = shmem.on_rank(x, 5)
    y.fill_(11)
    torch.cuda.synchronize()
    assert x.cpu().tolist() == [3] * 4 and y.cpu().tolist() == [11] * 4
    assert float((x.float() @ x.float()).item()) == 36.0  # ordinary torch kernels run on heap tensors
    assert shmem.get_cu_count() == 256 and shmem.wall_clock_rate(0) == 100000
    shmem.barrier()
    with pytest.raises(MemoryError):
        shmem.zeros((shmem.heap_size + 1,), dtype=torch.int8)
    with pytest.raises(RuntimeError, match="not on the symmetric heap"):
        shmem.ones(4, out=torch.zeros(4, device="cuda"), dtype=torch.float32)


def test_shim_malloc_free_and_ipc_handle():
    lib = _native.lib()
    p = _hip.malloc_fine_grained(1 << 20)
    assert p.value
    h = _hip.get_ipc_handle(p)
    assert h.shape == (64,) and h.any()
    _hip.hip_free(p)
    q = _hip.hip_malloc(4096)
    _hip.hip_free(q)
    assert lib.iris_hip_device_synchronize() == 0


def test_allocator_plugin_entry_points():
    """The two symbols torch's pluggable allocator binds, called directly."""
    alloc = ctypes.CDLL(_native.ALLOCATOR_LIB_PATH)
    alloc.finegrained_hipMalloc.restype = ctypes.c_void_p
    alloc.finegrained_hipMalloc.argtypes = [ctypes.c_ssize_t, ctypes.c_int, ctypes.c_void_p]
    alloc.finegrained_hipFree.restype = None
    alloc.finegrained_hipFree.argtypes = [ctypes.c_void_p, ctypes.c_ssize_t, ctypes.c_int, ctypes.c_void_p]
    p = alloc.finegrained_hipMalloc(1 << 16, 0, None)
    assert p
    alloc.finegrained_hipFree(p, 1 << 16, 0, None)
