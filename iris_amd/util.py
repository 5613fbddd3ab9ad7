"""Bench protocol and the int32 fill of the reference's ``iris/util.py``."""

from __future__ import annotations

import math
import statistics

import torch

from . import _native

__all__ = ["do_bench", "memset_tensor"]

_CACHE_BYTES = 256 * 1024 * 1024


def _flush_buffer():
    # 256 MiB of int32, zeroed between repetitions so that no run starts with
    # its operands in L2 / infinity cache (iris/util.py:11-19)
    return torch.empty(_CACHE_BYTES // 4, dtype=torch.int, device="cuda")


def _quantile(a, q):
    """Linear-interpolation quantiles of ``a`` at the points ``q``
    (iris/util.py:28-41); equals ``numpy.quantile(a, q, method="linear")``."""
    ordered = sorted(a)
    last = len(ordered) - 1
    out = []
    for point in q:
        if not (0 <= point <= 1):
            raise ValueError("Quantiles must be in the range [0, 1]")
        pos = point * last
        lo, hi = math.floor(pos), math.ceil(pos)
        frac = pos - lo
        out.append((1 - frac) * ordered[lo] + frac * ordered[hi])
    return out


def _summarize_statistics(times, quantiles, return_mode):
    if quantiles is not None:
        ret = _quantile(times, quantiles)
        return ret[0] if len(ret) == 1 else ret
    pick = {
        "all": lambda t: t,
        "min": min,
        "max": max,
        "mean": statistics.mean,
        "median": statistics.median,
    }.get(return_mode)
    return pick(times) if pick else None


def do_bench(fn, barrier_fn=lambda: None, preamble_fn=lambda: None, n_warmup=25, n_repeat=100, quantiles=None,
             return_mode="mean"):
    """Time ``fn`` in milliseconds with device events (iris/util.py:62-104).

    One untimed call, ``n_warmup`` warm-ups, then ``n_repeat`` timed calls;
    before each call: barrier, ``preamble_fn``, cache flush, barrier.
    """
    barrier_fn()
    preamble_fn()
    fn()
    barrier_fn()

    cache = _flush_buffer()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]

    def prepare():
        barrier_fn()
        preamble_fn()
        cache.zero_()
        barrier_fn()

    for _ in range(n_warmup):
        prepare()
        fn()
    for i in range(n_repeat):
        prepare()
        starts[i].record()
        fn()
        ends[i].record()
    barrier_fn()

    times = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return _summarize_statistics(times, quantiles, return_mode)


def memset_tensor(tensor, value):
    """Fill a contiguous int32 tensor on the current stream (iris/util.py:117-128)."""
    assert tensor.is_contiguous(), "Tensor must be contiguous"
    assert tensor.dtype == torch.int32, "Only torch.int32 tensors are supported"
    if not tensor.is_cuda:
        raise RuntimeError("memset_tensor needs a device tensor")
    stream = torch.cuda.current_stream(tensor.device).cuda_stream
    with torch.cuda.device(tensor.device):
        _native.hip_try(_native.lib().iris_memset_i32_launch(tensor.data_ptr(), int(value), tensor.numel(), stream))
