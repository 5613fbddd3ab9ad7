"""Python launchers of the HIP kernels, over the C-ABI of ``libiris_amd.so``.

These check operand shapes against what the kernels and their grids assume
*before* anything is launched, fill the C argument structs and launch on
torch's current stream.  They never synchronise and never allocate.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _native
from ._native import (
    DTYPE_BF16,
    DTYPE_F16,
    DTYPE_F32,
    EPI_ALL_SCATTER,
    EPI_ATOMIC_ADD,
    EPI_ONE_SHOT,
    PHASE_CONSUME,
    PHASE_FUSED,
    PHASE_PRODUCE,
    PHASE_TWO_KERNELS,
    SCOPE_AGENT,
    SCOPE_SYSTEM,
    VARIANT_FEW_ROWS,
    VARIANT_PERSISTENT,
    SPLIT_STREAM_K,
    HANDOVER_AUTO,
    HANDOVER_OWNER,
    HANDOVER_SLICED,
    HANDOVER_PAIR,
    FLAG_SEM_WRITE_THROUGH,
    FLAG_SEM_RELEASE_ACQUIRE,
    TOUCH_AUTO,
    TOUCH_ON,
    TOUCH_OFF,
)

__all__ = [
    "gemm_launch",
    "gemm_kernel_info",
    "gemm_split_k",
    "gemm_plan_name",
    "stream_k_schedule_host",
    "gemm_variant_name",
    "one_shot_reduce",
    "signal_tiles",
    "tile_schedule",
    "tile_map_host",
    "cdiv",
    "default_num_xcds",
    "EPI_ALL_SCATTER",
    "EPI_ATOMIC_ADD",
    "EPI_ONE_SHOT",
    "PHASE_PRODUCE",
    "PHASE_CONSUME",
    "PHASE_FUSED",
    "PHASE_TWO_KERNELS",
    "SCOPE_AGENT",
    "SCOPE_SYSTEM",
    "FLAG_SEM_WRITE_THROUGH",
    "FLAG_SEM_RELEASE_ACQUIRE",
    "TOUCH_AUTO",
    "TOUCH_ON",
    "TOUCH_OFF",
]

_DTYPES = {torch.float32: DTYPE_F32, torch.float16: DTYPE_F16, torch.bfloat16: DTYPE_BF16}

# limits of iris_gemm_launch_noalloc (include/iris_amd.h)
NOALLOC_MAX_PROGRAMS, NOALLOC_MAX_TILE_ELEMS = 256, 16384

# element types of iris_p2p_bench_launch beside the floating-point ones (include/iris_amd.h)
_RMA_DTYPES = dict(_DTYPES)
_RMA_DTYPES.update({torch.int8: 3, torch.int16: 4, torch.int32: 5, torch.int64: 6})


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def default_num_xcds(cu_count: int, num_sms: int) -> int:
    """XCDs to spread the persistent programs over.

    The reference hard-codes "8 iff 304 CUs" (matmul_wrapper.py:63-65, the
    MI300X).  An MI355X has 8 XCDs of 32 CUs; workgroups are dealt to XCDs
    round-robin, so the same remap keeps neighbouring tiles on one XCD's L2.
    The remap only changes which CU computes a tile, never a result or flag.
    """
    if cu_count in (304, 256) and num_sms % 8 == 0:
        return 8
    return 1


def _dtype_code(t: torch.Tensor, what: str) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"{what}: unsupported dtype {t.dtype}") from None


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _require_cuda(what: str, t: torch.Tensor, device: torch.device):
    if not t.is_cuda or t.device != device:
        raise RuntimeError(f"{what} must be on {device}, got {t.device}")


def _extent_ok(t: torch.Tensor, rows: int, cols: int) -> bool:
    return t.dim() == 2 and t.shape[0] >= rows and t.shape[1] >= cols


def _check_flags(tile_completed, total_tiles, device):
    if tile_completed is None:
        return
    _require_cuda("tile_completed", tile_completed, device)
    if tile_completed.dtype != torch.int32 or not tile_completed.is_contiguous():
        raise TypeError("tile_completed must be a contiguous int32 tensor")
    if tile_completed.numel() < total_tiles:
        raise ValueError(f"tile_completed has {tile_completed.numel()} flags, {total_tiles} tiles need one each")


def _check_heap_bases(heap_bases, world_size, device):
    if heap_bases is None:
        if world_size > 1:
            raise ValueError("heap_bases is required when world_size > 1")
        return
    _require_cuda("heap_bases", heap_bases, device)
    if heap_bases.dtype not in (torch.uint64, torch.int64) or heap_bases.numel() < world_size:
        raise TypeError("heap_bases must hold one 64-bit base address per rank")


def _fill_gemm_args(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N, BLK_K,
                    gsize_m, epilogue, phase, notify, num_xcds, scope, variant, mm_begin_timestamp,
                    mm_end_timestamp, status, spin_timeout_ticks, partials=None, locks=None, split_k=0):
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0], "incompatible dimensions"
    device = a.device
    M, K = a.shape
    _, N = b.shape
    _require_cuda("a", a, device)
    _require_cuda("b", b, device)
    if a.dtype != b.dtype:
        raise TypeError(f"a and b must share a dtype, got {a.dtype} and {b.dtype}")
    if a.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"operands must be fp16, bf16 or fp32, got {a.dtype}")
    if BLK_M <= 0 or BLK_N <= 0 or gsize_m <= 0 or num_sms <= 0:
        raise ValueError("block sizes, gsize_m and the grid must be positive")
    total_tiles = cdiv(M, BLK_M) * cdiv(N, BLK_N)

    if epilogue == EPI_ALL_SCATTER:
        # rank r's columns land at offset r*N of c_global[M, N*world_size]
        if c_global is None or not _extent_ok(c_global, M, N * world_size):
            raise ValueError(f"c_global must be at least [{M}, {N * world_size}] for the all-scatter epilogue")
    elif epilogue == EPI_ATOMIC_ADD:
        if c_global is None or not _extent_ok(c_global, M, N):
            raise ValueError(f"c_global must be at least [{M}, {N}]")
    elif epilogue == EPI_ONE_SHOT:
        if c is None or not _extent_ok(c, M, N):
            raise ValueError(f"c must be at least [{M}, {N}]")
        if c_global is None or not _extent_ok(c_global, M, N):
            raise ValueError(f"c_global must be at least [{M}, {N}]")
    else:
        raise ValueError(f"unknown epilogue {epilogue}")
    for name, t in (("c", c), ("c_global", c_global)):
        if t is not None:
            _require_cuda(name, t, device)
    _check_flags(tile_completed, total_tiles, device)
    _check_heap_bases(heap_bases, world_size, device)
    for name, t in (("mm_begin_timestamp", mm_begin_timestamp), ("mm_end_timestamp", mm_end_timestamp)):
        if t is not None:
            _require_cuda(name, t, device)
            if t.dtype != torch.int64 or t.numel() < total_tiles or not t.is_contiguous():
                raise TypeError(f"{name} must be a contiguous int64 tensor with one entry per tile")
    if status is not None:
        _require_cuda("status", status, device)
        if status.dtype not in (torch.int32, torch.uint32) or status.numel() < 1:
            raise TypeError("status must be a 32-bit device word")

    args = _native.GemmArgs()
    args.a, args.b = _ptr(a), _ptr(b)
    args.c, args.c_global = _ptr(c), _ptr(c_global)
    args.tile_completed = _ptr(tile_completed)
    args.heap_bases = _ptr(heap_bases)
    args.mm_begin_timestamp = _ptr(mm_begin_timestamp)
    args.mm_end_timestamp = _ptr(mm_end_timestamp)
    args.status = _ptr(status)
    args.M, args.N, args.K = M, N, K
    args.stride_am, args.stride_ak = a.stride(0), a.stride(1)
    args.stride_bk, args.stride_bn = b.stride(0), b.stride(1)
    if c is not None:
        args.stride_cm, args.stride_cn = c.stride(0), c.stride(1)
        args.c_dtype = _dtype_code(c, "c")
    if c_global is not None:
        args.stride_cm_global, args.stride_cn_global = c_global.stride(0), c_global.stride(1)
        args.c_global_dtype = _dtype_code(c_global, "c_global")
    args.block_m, args.block_n, args.block_k = BLK_M, BLK_N, BLK_K
    args.group_size_m = gsize_m
    args.num_sms = num_sms
    args.num_xcds = num_xcds
    args.cur_rank, args.world_size = rank, world_size
    args.ab_dtype = _dtype_code(a, "a")
    args.epilogue = epilogue
    args.phase = phase
    args.notify = 1 if notify else 0
    args.scope = scope
    args.variant = variant
    args.spin_timeout_ticks = spin_timeout_ticks
    # workspace: the wrappers' P [num_sms, BLK_M*BLK_N] fp32 and locks [num_sms] int32.  Split-K needs both;
    # the few-rows kernel only counts arrivals in locks.
    if partials is not None and locks is None:
        raise ValueError("partials need locks")
    if locks is not None:
        _require_cuda("locks", locks, device)
        if locks.dtype != torch.int32 or not locks.is_contiguous():
            raise TypeError("locks must be a contiguous int32 tensor")
        if locks.numel() < num_sms:
            raise ValueError("locks need one slot per program")
        args.locks = _ptr(locks)
    if partials is not None:
        _require_cuda("partials", partials, device)
        if partials.dtype != torch.float32 or partials.dim() != 2 or not partials.is_contiguous():
            raise TypeError("partials must be a contiguous fp32 matrix [num_sms, BLK_M * BLK_N]")
        if partials.shape[0] < num_sms:
            raise ValueError("partials need one slot per program")
        args.partials = _ptr(partials)
        args.partials_slot_elems = partials.shape[1]
    if partials is None and (split_k > 1 or split_k == SPLIT_STREAM_K):
        raise ValueError("a forced split of K needs the partials and locks workspace")
    args.split_k = split_k
    return args


def gemm_launch(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N, BLK_K,
                gsize_m, epilogue, *, phase=PHASE_FUSED, notify=True, num_xcds=1, scope=SCOPE_AGENT, variant=0,
                mm_begin_timestamp=None, mm_end_timestamp=None, status=None, spin_timeout_ticks=0, partials=None,
                locks=None, split_k=0, noalloc=False, split_handover=HANDOVER_AUTO,
                flag_sem=FLAG_SEM_WRITE_THROUGH, touch_ahead=TOUCH_AUTO):
    """Launch the persistent shard GEMM ``a @ b`` with a tile-publishing epilogue.

    ``touch_ahead``: ``TOUCH_AUTO`` lets the launcher decide whether the
    256 x 256 tile runs the build that touches the operand lines of K-steps to
    come (it does where a round of tiles streams more bytes than the last-level
    cache holds), ``TOUCH_ON`` / ``TOUCH_OFF`` force the choice; same bits.

    ``flag_sem``: ``FLAG_SEM_WRITE_THROUGH`` (write-through stores, then a
    relaxed flag add: validated with concurrent producers and consumers on one
    device) or ``FLAG_SEM_RELEASE_ACQUIRE`` (the reference's
    ``sem="release"`` on the flag add, gemm_one_shot_all_reduce.py:207-218).

    ``partials`` / ``locks`` are the wrappers' ``P`` and ``locks`` buffers
    (matmul_wrapper.py:29-31): with them, a launch with far fewer tiles than
    programs splits each tile's K range over several programs (``split_k`` 0:
    the launcher decides, 1: never, n: exactly n); ``split_k=SPLIT_STREAM_K``
    cuts the launch's K-steps into equal runs that cross tile boundaries
    (stream-K, on request only).  ``split_handover``: how the
    parts of a split tile meet: ``HANDOVER_OWNER`` (the first part adds the
    others' partials and stores the tile), ``HANDOVER_SLICED`` (every part sums
    and stores its share of the rows) or ``HANDOVER_AUTO``; bit-identical results.

    ``noalloc=True`` goes through ``iris_gemm_launch_noalloc``: no workspace
    is passed, the library's own device array takes its place.

    The kernel launch of the reference wrappers (matmul_wrapper.py:109-150).
    """
    if noalloc:
        if partials is not None or locks is not None:
            raise ValueError("the no-allocation launch takes no workspace")
        if num_sms > NOALLOC_MAX_PROGRAMS:
            raise ValueError(f"the no-allocation launch takes at most {NOALLOC_MAX_PROGRAMS} programs")
        forced = split_k > 1 or split_k == SPLIT_STREAM_K
        if forced and BLK_M * BLK_N > NOALLOC_MAX_TILE_ELEMS:
            raise ValueError(f"a forced split of K needs tiles of at most {NOALLOC_MAX_TILE_ELEMS} elements here")
        args = _fill_gemm_args(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M,
                               BLK_N, BLK_K, gsize_m, epilogue, phase, notify, num_xcds, scope, variant,
                               mm_begin_timestamp, mm_end_timestamp, status, spin_timeout_ticks, None, None, 0)
        args.split_k = split_k
        launch = _native.lib().iris_gemm_launch_noalloc
    else:
        args = _fill_gemm_args(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M,
                               BLK_N, BLK_K, gsize_m, epilogue, phase, notify, num_xcds, scope, variant,
                               mm_begin_timestamp, mm_end_timestamp, status, spin_timeout_ticks, partials, locks,
                               split_k)
        launch = _native.lib().iris_gemm_launch
    args.split_handover = split_handover
    args.flag_sem = flag_sem
    args.touch_ahead = touch_ahead
    stream = torch.cuda.current_stream(a.device).cuda_stream
    with torch.cuda.device(a.device):
        err = launch(ctypes.byref(args), stream)
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError(
            "iris_gemm_launch rejected the arguments (shape, strides, dtypes, grid or rank layout it does not take)"
        )
    _native.hip_try(err)


def gemm_split_k(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N, BLK_K,
                 gsize_m, epilogue, *, phase=PHASE_FUSED, notify=True, num_xcds=1, variant=0, partials=None,
                 locks=None, split_k=0):
    """The split-K factor a launch with these arguments would use (1: unsplit)."""
    args = _fill_gemm_args(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N,
                           BLK_K, gsize_m, epilogue, phase, notify, num_xcds, SCOPE_AGENT, variant, None, None, None,
                           0, partials, locks, split_k)
    sk = ctypes.c_int()
    with torch.cuda.device(a.device):
        err = _native.lib().iris_gemm_split_k(ctypes.byref(args), ctypes.byref(sk))
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_gemm_split_k rejected the arguments")
    _native.hip_try(err)
    return sk.value


def gemm_plan_name(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N, BLK_K,
                   gsize_m, epilogue, *, phase=PHASE_FUSED, notify=True, num_xcds=1, variant=0, partials=None,
                   locks=None, split_k=0, touch_ahead=TOUCH_AUTO):
    """Name of the kernel a launch with these arguments would run."""
    args = _fill_gemm_args(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N,
                           BLK_K, gsize_m, epilogue, phase, notify, num_xcds, SCOPE_AGENT, variant, None, None, None,
                           0, partials, locks, split_k)
    args.touch_ahead = touch_ahead
    buf = ctypes.create_string_buffer(128)
    with torch.cuda.device(a.device):
        err = _native.lib().iris_gemm_plan_name(ctypes.byref(args), buf, 128)
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_gemm_plan_name rejected the arguments")
    _native.hip_try(err)
    return buf.value.decode()


def gemm_kernel_info(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N, BLK_K,
                     gsize_m, epilogue, *, phase=PHASE_FUSED, notify=True, num_xcds=1, variant=0):
    """(registers, spill bytes per lane) of the kernel a launch would use."""
    args = _fill_gemm_args(a, b, c, c_global, tile_completed, heap_bases, rank, world_size, num_sms, BLK_M, BLK_N,
                           BLK_K, gsize_m, epilogue, phase, notify, num_xcds, SCOPE_AGENT, variant, None, None, None,
                           0)
    regs, spills = ctypes.c_int(), ctypes.c_int()
    with torch.cuda.device(a.device):
        _native.hip_try(_native.lib().iris_gemm_kernel_info(ctypes.byref(args), ctypes.byref(regs),
                                                            ctypes.byref(spills)))
    return regs.value, spills.value


def gemm_variant_name(dtype: torch.dtype, out_is_f32: bool, atomic: bool, variant: int) -> Optional[str]:
    buf = ctypes.create_string_buffer(128)
    err = _native.lib().iris_gemm_variant_name(_DTYPES[dtype], int(out_is_f32), int(atomic), variant, buf, 128)
    return None if err else buf.value.decode()


def stream_k_schedule_host(total_tiles: int, k_steps: int, num_programs: int, pid: int):
    """Items ``(tile, k_begin, k_end, parts)`` of program ``pid`` under the
    kernels' stream-K schedule (host build of the same source)."""
    cap = total_tiles + 2
    items = (ctypes.c_int32 * (4 * cap))()
    n = ctypes.c_int32()
    err = _native.lib().iris_stream_k_schedule_host(total_tiles, k_steps, num_programs, pid, items, cap,
                                                    ctypes.byref(n))
    if err:
        raise ValueError("iris_stream_k_schedule_host rejected the arguments")
    return [tuple(items[4 * i:4 * i + 4]) for i in range(n.value)]


def one_shot_reduce(c, c_global, tile_completed, heap_bases, rank, world_size, BLK_M, BLK_N, gsize_m, *,
                    num_sms=0, num_xcds=1, scope=SCOPE_AGENT, wait_flags=True, variant=0, status=None,
                    spin_timeout_ticks=0, flag_sem=FLAG_SEM_WRITE_THROUGH):
    """Sum the ``world_size`` partial buffers that sit at ``c``'s heap offset on
    every rank into ``c_global``, tile by tile, behind the tiles' flags.

    The consumer half of gemm_one_shot_all_reduce.py:220-271.
    ``flag_sem=FLAG_SEM_RELEASE_ACQUIRE`` adds the reference's acquire after
    every flag wait (:220-234); by default the loads are coherent at the
    flags' scope by themselves.
    """
    if c.dim() != 2 or c_global.dim() != 2:
        raise ValueError("c and c_global must be matrices")
    M, N = c.shape
    device = c.device
    _require_cuda("c", c, device)
    _require_cuda("c_global", c_global, device)
    if not _extent_ok(c_global, M, N):
        raise ValueError(f"c_global must be at least [{M}, {N}]")
    if BLK_M <= 0 or BLK_N <= 0 or gsize_m <= 0 or num_sms < 0:
        raise ValueError("block sizes and gsize_m must be positive")
    total_tiles = cdiv(M, BLK_M) * cdiv(N, BLK_N)
    if wait_flags and world_size > 1 and tile_completed is None:
        raise ValueError("tile_completed is required to wait on flags")
    _check_flags(tile_completed, total_tiles, device)
    _check_heap_bases(heap_bases, world_size, device)
    args = _native.ReduceArgs()
    args.c, args.c_global = _ptr(c), _ptr(c_global)
    args.tile_completed = _ptr(tile_completed)
    args.heap_bases = _ptr(heap_bases)
    args.status = _ptr(status)
    args.M, args.N = M, N
    args.stride_cm, args.stride_cn = c.stride(0), c.stride(1)
    args.stride_cm_global, args.stride_cn_global = c_global.stride(0), c_global.stride(1)
    args.block_m, args.block_n, args.group_size_m = BLK_M, BLK_N, gsize_m
    args.num_sms, args.num_xcds = num_sms, num_xcds
    args.cur_rank, args.world_size = rank, world_size
    args.c_dtype, args.c_global_dtype = _dtype_code(c, "c"), _dtype_code(c_global, "c_global")
    args.scope = scope
    args.wait_flags = 1 if wait_flags else 0
    args.variant = variant
    args.spin_timeout_ticks = spin_timeout_ticks
    args.flag_sem = flag_sem
    stream = torch.cuda.current_stream(device).cuda_stream
    with torch.cuda.device(device):
        err = _native.lib().iris_one_shot_reduce_launch(ctypes.byref(args), stream)
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_one_shot_reduce_launch rejected the arguments")
    _native.hip_try(err)


def tile_schedule(M, N, BLK_M, BLK_N, gsize_m, num_sms, num_xcds, device="cuda"):
    """int32[total_tiles, 4] = (pid_m, pid_n, program, position) per tile id,
    computed on the device by the functions the kernels use."""
    total = cdiv(M, BLK_M) * cdiv(N, BLK_N)
    out = torch.full((total, 4), -1, dtype=torch.int32, device=device)
    stream = torch.cuda.current_stream(out.device).cuda_stream
    with torch.cuda.device(out.device):
        err = _native.lib().iris_tile_schedule_launch(out.data_ptr(), M, N, BLK_M, BLK_N, gsize_m, num_sms,
                                                      num_xcds, stream)
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_tile_schedule_launch rejected the arguments")
    _native.hip_try(err)
    return out


def tile_map_host(tile_id, M, N, BLK_M, BLK_N, gsize_m):
    """(pid_m, pid_n) from the host build of the kernels' tile map."""
    pm, pn = ctypes.c_int32(), ctypes.c_int32()
    _native.lib().iris_tile_map_host(tile_id, M, N, BLK_M, BLK_N, gsize_m, ctypes.byref(pm), ctypes.byref(pn))
    return pm.value, pn.value


# iris_p2p_bench_launch (include/iris_amd.h)
P2P_OPS = {"load": 0, "local_store": 1, "store": 2, "all_load": 3, "all_store": 4, "atomic_add": 5,
           "atomic_xchg": 6}


def p2p_bench(op, buffer, result, heap_bases, rank, peer, num_ranks, *, block_size=512):
    """One launch of a point-to-point microbenchmark kernel as rank ``rank``:
    ``op`` is a key of ``P2P_OPS`` (examples/00_load .. 05_atomic_xchg of the
    reference); thread i owns element i of ``buffer`` / ``result``."""
    ref = buffer if buffer is not None else result
    if ref is None:
        raise ValueError("a buffer is needed")
    if ref.dtype not in _RMA_DTYPES or ref.dtype in (torch.int16, torch.int64):
        raise ValueError(f"unsupported element type {ref.dtype}")
    if buffer is not None and result is not None and (buffer.dtype != result.dtype or buffer.numel() != result.numel()):
        raise ValueError("buffer and result must have the same element type and length")
    if op != "local_store":
        _check_heap_bases(heap_bases, num_ranks, ref.device)
    stream = torch.cuda.current_stream(ref.device).cuda_stream
    err = _native.lib().iris_p2p_bench_launch(
        P2P_OPS[op], _RMA_DTYPES[ref.dtype], _ptr(buffer), _ptr(result), ref.numel(), rank, peer, num_ranks,
        _ptr(heap_bases), block_size, ctypes.c_void_p(stream))
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_p2p_bench_launch rejected the arguments")
    _native.hip_try(err)


def signal_tiles(tile_completed, heap_bases, total_tiles, rank, world_size, *, include_self=False,
                 scope=SCOPE_AGENT):
    """+1 (release) on the flag of every tile on the other ranks (on every rank
    with ``include_self``); gemm_one_shot_all_reduce.py:207-218 on its own."""
    device = tile_completed.device
    _check_flags(tile_completed, total_tiles, device)
    _check_heap_bases(heap_bases, world_size, device)
    stream = torch.cuda.current_stream(device).cuda_stream
    with torch.cuda.device(device):
        err = _native.lib().iris_signal_tiles_launch(tile_completed.data_ptr(), _ptr(heap_bases), total_tiles, rank,
                                                     world_size, 1 if include_self else 0, scope, stream)
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_signal_tiles_launch rejected the arguments")
    _native.hip_try(err)
