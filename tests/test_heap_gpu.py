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


def test_heap_is_released_with_its_last_tensor():
    """The context's allocation lives as long as any tensor that views it and
    goes back to the device after that (the reference's pool is a torch tensor
    with the same lifetime, iris/iris.py:48)."""
    import gc

    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    size = 1 << 30
    ctx = iris_amd.iris(size)
    t = ctx.ones((1024,), dtype=torch.float32)
    free1, _ = torch.cuda.mem_get_info()
    assert free0 - free1 >= size * 0.9
    del ctx
    gc.collect()
    assert float(t.sum()) == 1024.0  # a tensor of the heap keeps it alive
    assert torch.cuda.mem_get_info()[0] <= free1 + (64 << 20)
    del t
    gc.collect()
    assert torch.cuda.mem_get_info()[0] >= free0 - (64 << 20)  # returned


_PLUGIN_CHILD = r"""
import os, sys
sys.path.insert(0, {root!r})
import torch
import iris_amd                      # IRIS_AMD_PLUGGABLE_ALLOCATOR=1: binds the plug-in before any allocation
from iris_amd import ops
from oracle import iris_oracle as O

assert torch.cuda.memory.get_allocator_backend() == "pluggable", torch.cuda.memory.get_allocator_backend()
ws = 2
shmem = iris_amd.iris(64 << 20, virtual_ranks=ws)   # the pool itself is a torch allocation in this mode
g = torch.Generator().manual_seed(123)
M, N, K, BM, BN, G = 256, 192, 128, 128, 64, 4
A = (torch.randn(M, K, generator=g) * 0.05).to(torch.bfloat16)
B = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).T
a = shmem.zeros((M, K), dtype=torch.bfloat16); a.copy_(A)
bt = shmem.zeros((N, K), dtype=torch.bfloat16); bt.copy_(B.T)
b = bt.T
c = shmem.zeros((M, N), dtype=torch.float32)
out = shmem.zeros((M, N), dtype=torch.bfloat16)
total = ops.cdiv(M, BM) * ops.cdiv(N, BN)
flags = shmem.zeros((total,), dtype=torch.int32)
hb = shmem.get_heap_bases()
ks = K // ws
for r in range(ws):
    for t in (c, out, flags):
        shmem.on_rank(t, r).zero_()
for r in range(ws):
    ops.gemm_launch(a[:, r * ks:(r + 1) * ks], b[r * ks:(r + 1) * ks, :], shmem.on_rank(c, r), shmem.on_rank(out, r),
                    shmem.on_rank(flags, r), hb, r, ws, 16, BM, BN, 64, G, ops.EPI_ONE_SHOT, phase=ops.PHASE_PRODUCE)
ops.one_shot_reduce(c, out, flags, hb, 0, ws, BM, BN, G)
torch.cuda.synchronize()
partials = torch.stack([shmem.on_rank(c, r).cpu() for r in range(ws)])
assert torch.equal(out.cpu(), O.one_shot_reduce(partials, torch.bfloat16))
want = O.one_shot_all_reduce(O.k_shards(A, B, ws), torch.float32, torch.bfloat16)
assert torch.allclose(out.float().cpu(), want.float(), rtol=1e-2, atol=1e-2)
assert flags.cpu().tolist() == [0] * total
print("PLUGIN-OK")
"""


def test_torch_binds_the_allocator_plugin_in_a_fresh_process(tmp_path):
    """IRIS_AMD_PLUGGABLE_ALLOCATOR=1: torch's CUDAPluggableAllocator loads
    libfinegrained_allocator.so and routes every device allocation through its
    two symbols, as iris/__init__.py:40-45 does; a small K-split GEMM + reduce
    then runs on a heap that is an ordinary torch tensor.  The allocator can
    only be swapped before a process's first allocation, hence the child."""
    import os
    import subprocess
    import sys

    root = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
    script = tmp_path / "plugin_child.py"
    script.write_text(_PLUGIN_CHILD.format(root=root))
    env = dict(os.environ, IRIS_AMD_PLUGGABLE_ALLOCATOR="1", LOG_FINEGRAINED_ALLOCATOR="1")
    proc = subprocess.run([sys.executable, "-u", str(script)], capture_output=True, text=True, timeout=300, env=env,
                          cwd=str(tmp_path))
    assert proc.returncode == 0 and "PLUGIN-OK" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-3000:]
    # the plug-in's own log: torch really allocated (the 128 MiB pool among others) through its symbols
    assert f"size={2 * (64 << 20)} bytes" in proc.stdout and "[finegrained_allocator] Allocation" in proc.stdout
