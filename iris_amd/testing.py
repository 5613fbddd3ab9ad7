"""Python launchers of the kernels in ``libiris_amd_testing.so``
(``include/iris_amd_testing.h``): measurement probes for the matrix cores and
the store path, and the unit-test kernels over the device-side remote-access
header.  Only the tests and ``bench.py`` use this module; the product's
launchers are in ``iris_amd.ops``.
"""

from __future__ import annotations

import ctypes

import torch

from . import _native
from ._native import SCOPE_AGENT, SCOPE_SYSTEM
from .ops import _DTYPES, _RMA_DTYPES, _check_heap_bases, _ptr

# iris_rma_selftest_launch (include/iris_amd_testing.h)
RMA_OPS = {"load": 0, "store": 1, "get": 2, "put": 3, "atomic_add": 4, "atomic_sub": 5, "atomic_cas": 6,
           "atomic_xchg": 7}
RMA_SEMS = {"relaxed": 0, "acquire": 1, "release": 2, "acq_rel": 3}
RMA_SCOPES = {"cta": 2, "gpu": SCOPE_AGENT, "sys": SCOPE_SYSTEM}


def mfma_probe(operands, sink, iters, num_groups):
    """Launch the register-only MFMA loop (a measurement aid): returns the FLOP
    count of the launch.  ``operands``: >= 64 KiB of fp16/bf16 on the device,
    ``sink``: >= num_groups * 512 floats."""
    if operands.dtype not in _DTYPES or operands.dtype == torch.float32:
        raise ValueError("operands must be fp16 or bf16")
    if operands.numel() * operands.element_size() < 65536 or sink.numel() < num_groups * 512:
        raise ValueError("operands: at least 64 KiB; sink: at least num_groups * 512 floats")
    if sink.dtype != torch.float32 or not operands.is_contiguous():
        raise ValueError("sink must be fp32 and operands contiguous")
    stream = torch.cuda.current_stream(operands.device).cuda_stream
    _native.hip_try(_native.testing_lib().iris_mfma_probe_launch(_ptr(operands), _ptr(sink), _DTYPES[operands.dtype], iters,
                                                         num_groups, ctypes.c_void_p(stream)))
    return num_groups * 8 * iters * 16 * 16384


def store_probe(operands, sink, out, tiles, chunk, num_groups, *, write_through=True, lockstep=True):
    """Launch the store probe (a measurement aid): ``tiles`` tiles per group of
    8 waves, each 16 K-steps of register-only MFMAs and 128 KiB of stores to
    ``out``, ``chunk`` one-KiB stores a wave back to back every ``chunk``
    K-steps (16, 4, 1, or 0 for none).  Returns the bytes stored per launch."""
    if operands.dtype != torch.bfloat16 or operands.numel() * 2 < 65536 or not operands.is_contiguous():
        raise ValueError("operands: at least 64 KiB of contiguous bf16")
    if sink.dtype != torch.float32 or sink.numel() < num_groups * 512:
        raise ValueError("sink: at least num_groups * 512 floats")
    out_bytes = out.numel() * out.element_size()
    if not out.is_contiguous() or out_bytes < num_groups * 131072:
        raise ValueError("out: contiguous, at least 128 KiB per group")
    stream = torch.cuda.current_stream(operands.device).cuda_stream
    err = _native.testing_lib().iris_store_probe_launch(_ptr(operands), _ptr(sink), _ptr(out), out_bytes, tiles, chunk,
                                                1 if write_through else 0, 1 if lockstep else 0, num_groups,
                                                ctypes.c_void_p(stream))
    if err == _native.HIP_ERROR_INVALID_VALUE:
        raise ValueError("iris_store_probe_launch rejected the arguments")
    _native.hip_try(err)
    return 0 if chunk == 0 else tiles * num_groups * 131072


def rma_selftest(op, data, results, heap_bases, rank, num_ranks, block_size, *, sem="acq_rel", scope="sys"):
    """Run one of the unit-test kernels over the device-side remote-access
    functions (include/iris_device.hpp) as rank ``rank``: ``op`` is a key of
    ``RMA_OPS``, ``sem`` / ``scope`` the reference's strings
    (tests/unittests/test_atomic_add.py:44-60)."""
    if results.dtype not in _RMA_DTYPES:
        raise ValueError(f"unsupported element type {results.dtype}")
    if data is not None and data.dtype != results.dtype:
        raise ValueError("data and results must have the same element type")
    if not 1 <= block_size <= 64 or results.numel() < block_size or (data is not None and data.numel() < block_size):
        raise ValueError("block_size must be 1..64 and fit the buffers")
    _check_heap_bases(heap_bases, num_ranks, results.device)
    stream = torch.cuda.current_stream(results.device).cuda_stream
    _native.hip_try(_native.testing_lib().iris_rma_selftest_launch(
        RMA_OPS[op], _RMA_DTYPES[results.dtype], RMA_SEMS[sem], RMA_SCOPES[scope], _ptr(data), _ptr(results),
        _ptr(heap_bases), rank, num_ranks, block_size, ctypes.c_void_p(stream)))
