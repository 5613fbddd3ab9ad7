"""ctypes view of ``libiris_amd.so`` (the C-ABI declared in ``include/iris_amd.h``).

The library is built in-tree by ``python -m iris_amd.build``.  Nothing here
falls back to another implementation: if the library is missing, loading
raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libiris_amd.so")
ALLOCATOR_LIB_PATH = os.path.join(_PKG_DIR, "csrc", "finegrained_alloc", "libfinegrained_allocator.so")
# kernels that only the tests and bench.py call (include/iris_amd_testing.h)
TESTING_LIB_PATH = os.path.join(_PKG_DIR, "libiris_amd_testing.so")

# element types (IRIS_DTYPE_*)
DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
# epilogues (IRIS_EPI_*)
EPI_ALL_SCATTER, EPI_ATOMIC_ADD, EPI_ONE_SHOT = 0, 1, 2
# ONE_SHOT phases (IRIS_PHASE_*)
PHASE_PRODUCE, PHASE_CONSUME, PHASE_FUSED, PHASE_TWO_KERNELS = 1, 2, 3, 7
# flag scopes (IRIS_SCOPE_*)
SCOPE_AGENT, SCOPE_SYSTEM = 0, 1
# special values of GemmArgs.variant (include/iris_amd.h)
VARIANT_FEW_ROWS, VARIANT_PERSISTENT = 1000, 1001
SPLIT_STREAM_K = -1  # GemmArgs.split_k: stream-K
HANDOVER_AUTO, HANDOVER_OWNER, HANDOVER_SLICED, HANDOVER_PAIR = 0, 1, 2, 3  # GemmArgs.split_handover
# how a tile's flag orders its data (IRIS_FLAG_SEM_*)
FLAG_SEM_WRITE_THROUGH, FLAG_SEM_RELEASE_ACQUIRE = 0, 1
TOUCH_AUTO, TOUCH_ON, TOUCH_OFF = 0, 1, 2
# status word (IRIS_STATUS_*)
STATUS_OK, STATUS_SPIN_TIMEOUT = 0, 1

HIP_ERROR_INVALID_VALUE = 1


class GemmArgs(ctypes.Structure):
    """``iris_gemm_args``."""

    _fields_ = [
        ("a", ctypes.c_void_p),
        ("b", ctypes.c_void_p),
        ("c", ctypes.c_void_p),
        ("c_global", ctypes.c_void_p),
        ("tile_completed", ctypes.c_void_p),
        ("heap_bases", ctypes.c_void_p),
        ("mm_begin_timestamp", ctypes.c_void_p),
        ("mm_end_timestamp", ctypes.c_void_p),
        ("status", ctypes.c_void_p),
        ("M", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("stride_am", ctypes.c_int64),
        ("stride_ak", ctypes.c_int64),
        ("stride_bk", ctypes.c_int64),
        ("stride_bn", ctypes.c_int64),
        ("stride_cm", ctypes.c_int64),
        ("stride_cn", ctypes.c_int64),
        ("stride_cm_global", ctypes.c_int64),
        ("stride_cn_global", ctypes.c_int64),
        ("block_m", ctypes.c_int32),
        ("block_n", ctypes.c_int32),
        ("block_k", ctypes.c_int32),
        ("group_size_m", ctypes.c_int32),
        ("num_sms", ctypes.c_int32),
        ("num_xcds", ctypes.c_int32),
        ("cur_rank", ctypes.c_int32),
        ("world_size", ctypes.c_int32),
        ("ab_dtype", ctypes.c_int32),
        ("c_dtype", ctypes.c_int32),
        ("c_global_dtype", ctypes.c_int32),
        ("epilogue", ctypes.c_int32),
        ("phase", ctypes.c_int32),
        ("notify", ctypes.c_int32),
        ("scope", ctypes.c_int32),
        ("variant", ctypes.c_int32),
        ("spin_timeout_ticks", ctypes.c_uint64),
        ("partials", ctypes.c_void_p),
        ("locks", ctypes.c_void_p),
        ("partials_slot_elems", ctypes.c_int64),
        ("split_k", ctypes.c_int32),
        ("split_handover", ctypes.c_int32),
        ("flag_sem", ctypes.c_int32),
        ("touch_ahead", ctypes.c_int32),
    ]


class ReduceArgs(ctypes.Structure):
    """``iris_reduce_args``."""

    _fields_ = [
        ("c", ctypes.c_void_p),
        ("c_global", ctypes.c_void_p),
        ("tile_completed", ctypes.c_void_p),
        ("heap_bases", ctypes.c_void_p),
        ("status", ctypes.c_void_p),
        ("M", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("stride_cm", ctypes.c_int64),
        ("stride_cn", ctypes.c_int64),
        ("stride_cm_global", ctypes.c_int64),
        ("stride_cn_global", ctypes.c_int64),
        ("block_m", ctypes.c_int32),
        ("block_n", ctypes.c_int32),
        ("group_size_m", ctypes.c_int32),
        ("num_sms", ctypes.c_int32),
        ("num_xcds", ctypes.c_int32),
        ("cur_rank", ctypes.c_int32),
        ("world_size", ctypes.c_int32),
        ("c_dtype", ctypes.c_int32),
        ("c_global_dtype", ctypes.c_int32),
        ("scope", ctypes.c_int32),
        ("wait_flags", ctypes.c_int32),
        ("variant", ctypes.c_int32),
        ("spin_timeout_ticks", ctypes.c_uint64),
        ("flag_sem", ctypes.c_int32),
    ]


# every symbol include/iris_amd.h declares for libiris_amd.so:
# name -> (restype, argtypes)
_P = ctypes.c_void_p
_I = ctypes.c_int
SIGNATURES = {
    "iris_hip_error_string": (ctypes.c_char_p, [_I]),
    "iris_hip_device_count": (_I, [ctypes.POINTER(_I)]),
    "iris_hip_set_device": (_I, [_I]),
    "iris_hip_get_device": (_I, [ctypes.POINTER(_I)]),
    "iris_hip_cu_count": (_I, [_I, ctypes.POINTER(_I)]),
    "iris_hip_wall_clock_rate": (_I, [_I, ctypes.POINTER(_I)]),
    "iris_hip_malloc_finegrained": (_I, [ctypes.POINTER(_P), ctypes.c_size_t]),
    "iris_hip_malloc": (_I, [ctypes.POINTER(_P), ctypes.c_size_t]),
    "iris_hip_free": (_I, [_P]),
    "iris_hip_ipc_get_handle": (_I, [_P, _P]),
    "iris_hip_ipc_open_handle": (_I, [ctypes.POINTER(_P), _P]),
    "iris_hip_device_synchronize": (_I, []),
    "iris_hip_arch_name": (_I, [_I, ctypes.c_char_p, ctypes.c_size_t]),
    "iris_gemm_launch": (_I, [ctypes.POINTER(GemmArgs), _P]),
    "iris_gemm_launch_noalloc": (_I, [ctypes.POINTER(GemmArgs), _P]),
    "iris_gemm_kernel_info": (_I, [ctypes.POINTER(GemmArgs), ctypes.POINTER(_I), ctypes.POINTER(_I)]),
    "iris_gemm_split_k": (_I, [ctypes.POINTER(GemmArgs), ctypes.POINTER(_I)]),
    "iris_gemm_variant_name": (_I, [_I, _I, _I, _I, ctypes.c_char_p, ctypes.c_size_t]),
    "iris_gemm_plan_name": (_I, [ctypes.POINTER(GemmArgs), ctypes.c_char_p, ctypes.c_size_t]),
    "iris_one_shot_reduce_launch": (_I, [ctypes.POINTER(ReduceArgs), _P]),
    "iris_signal_tiles_launch": (_I, [_P, _P, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
                                      ctypes.c_int32, _P]),
    "iris_memset_i32_launch": (_I, [_P, ctypes.c_int32, ctypes.c_int64, _P]),
    "iris_tile_schedule_launch": (_I, [_P] + [ctypes.c_int32] * 7 + [_P]),
    "iris_tile_map_host": (None, [ctypes.c_int32] * 6 + [ctypes.POINTER(ctypes.c_int32)] * 2),
    "iris_stream_k_schedule_host": (_I, [ctypes.c_int32] * 4 + [ctypes.POINTER(ctypes.c_int32), ctypes.c_int32,
                                         ctypes.POINTER(ctypes.c_int32)]),
    "iris_p2p_bench_launch": (_I, [ctypes.c_int32] * 2 + [_P, _P, ctypes.c_int64] + [ctypes.c_int32] * 3
                              + [_P, ctypes.c_int32, _P]),
    "iris_amd_abi_version": (_I, []),
}
ALLOCATOR_SYMBOLS = ("finegrained_hipMalloc", "finegrained_hipFree")
# every symbol include/iris_amd_testing.h declares for libiris_amd_testing.so
TESTING_SIGNATURES = {
    "iris_mfma_probe_launch": (_I, [_P, _P, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, _P]),
    "iris_store_probe_launch": (_I, [_P, _P, _P, ctypes.c_uint64] + [ctypes.c_int32] * 5 + [_P]),
    "iris_rma_selftest_launch": (_I, [ctypes.c_int32] * 4 + [_P, _P, _P] + [ctypes.c_int32] * 3 + [_P]),
}

_lib = None
_testing_lib = None
_lock = threading.Lock()


def lib() -> ctypes.CDLL:
    """Load ``libiris_amd.so`` once and type its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"iris_amd native library not found at {LIB_PATH}. Build it with `python -m iris_amd.build`; "
                    "there is no other implementation to fall back to."
                )
            handle = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = handle
    return _lib


def testing_lib() -> ctypes.CDLL:
    """Load ``libiris_amd_testing.so`` (tests and bench.py only) once and type its entry points."""
    global _testing_lib
    if _testing_lib is not None:
        return _testing_lib
    with _lock:
        if _testing_lib is None:
            if not os.path.exists(TESTING_LIB_PATH):
                raise RuntimeError(f"{TESTING_LIB_PATH} not found. Build it with `python -m iris_amd.build`.")
            handle = ctypes.CDLL(TESTING_LIB_PATH)
            for name, (restype, argtypes) in TESTING_SIGNATURES.items():
                fn = getattr(handle, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _testing_lib = handle
    return _testing_lib


def hip_try(err: int) -> None:
    """Raise ``RuntimeError`` on a HIP error, worded as iris/_hip.py:12-16."""
    if err != 0:
        msg = lib().iris_hip_error_string(int(err))
        text = msg.decode("utf-8") if msg else "unknown error"
        raise RuntimeError(f"HIP error code {err}: {text}")
