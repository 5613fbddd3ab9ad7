"""HIP runtime helpers of the host API, over the C-ABI shim.

Same function names and results as the reference's ctypes module
(iris/_hip.py), but every call goes through ``libiris_amd.so`` instead of
binding ``libamdhip64.so`` by hand.
"""

from __future__ import annotations

import ctypes

import numpy as np

from ._native import hip_try, lib

__all__ = [
    "hip_try",
    "open_ipc_handle",
    "get_ipc_handle",
    "count_devices",
    "set_device",
    "get_device_id",
    "get_cu_count",
    "get_wall_clock_rate",
    "get_arch_name",
    "malloc_fine_grained",
    "hip_malloc",
    "hip_free",
    "device_synchronize",
]


def open_ipc_handle(ipc_handle_data, rank=None):
    """iris/_hip.py:23-53 -- map a peer's allocation; returns the pointer."""
    if isinstance(ipc_handle_data, np.ndarray):
        if ipc_handle_data.dtype != np.uint8 or ipc_handle_data.size != 64:
            raise ValueError("ipc_handle_data must be a 64-element uint8 numpy array")
        raw = ipc_handle_data.tobytes()
    else:
        raise TypeError("ipc_handle_data must be a numpy.ndarray of dtype uint8 with 64 elements")
    buf = ctypes.create_string_buffer(raw, 64)
    ptr = ctypes.c_void_p()
    hip_try(lib().iris_hip_ipc_open_handle(ctypes.byref(ptr), ctypes.cast(buf, ctypes.c_void_p)))
    return ptr.value


def get_ipc_handle(ptr, rank=None):
    """iris/_hip.py:56-59 -- 64-byte IPC handle of a device allocation, as a
    uint8[64] numpy array."""
    buf = ctypes.create_string_buffer(64)
    p = ptr if isinstance(ptr, ctypes.c_void_p) else ctypes.c_void_p(int(ptr))
    hip_try(lib().iris_hip_ipc_get_handle(ctypes.cast(buf, ctypes.c_void_p), p))
    return np.frombuffer(buf.raw, dtype=np.uint8).copy()


def count_devices():
    n = ctypes.c_int()
    hip_try(lib().iris_hip_device_count(ctypes.byref(n)))
    return n.value


def set_device(gpu_id):
    hip_try(lib().iris_hip_set_device(int(gpu_id)))


def get_device_id():
    d = ctypes.c_int()
    hip_try(lib().iris_hip_get_device(ctypes.byref(d)))
    return d.value


def get_cu_count(device_id=None):
    if device_id is None:
        device_id = get_device_id()
    n = ctypes.c_int()
    hip_try(lib().iris_hip_cu_count(int(device_id), ctypes.byref(n)))
    return n.value


def get_wall_clock_rate(device_id):
    """kHz of the constant-rate wall clock (s_memrealtime)."""
    n = ctypes.c_int()
    hip_try(lib().iris_hip_wall_clock_rate(int(device_id), ctypes.byref(n)))
    return n.value


def get_arch_name(device_id=None):
    if device_id is None:
        device_id = get_device_id()
    buf = ctypes.create_string_buffer(256)
    hip_try(lib().iris_hip_arch_name(int(device_id), buf, 256))
    return buf.value.decode("utf-8")


def malloc_fine_grained(size):
    ptr = ctypes.c_void_p()
    hip_try(lib().iris_hip_malloc_finegrained(ctypes.byref(ptr), int(size)))
    return ptr


def hip_malloc(size):
    ptr = ctypes.c_void_p()
    hip_try(lib().iris_hip_malloc(ctypes.byref(ptr), int(size)))
    return ptr


def hip_free(ptr):
    p = ptr if isinstance(ptr, ctypes.c_void_p) else ctypes.c_void_p(int(ptr))
    hip_try(lib().iris_hip_free(p))


def device_synchronize():
    hip_try(lib().iris_hip_device_synchronize())
