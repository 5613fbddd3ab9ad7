"""The examples' ``matmul`` launch wrappers.

``matmul.apply(a, b, c, c_global, bias, P, locks, tile_completed, rank,
world_size, grid, BLK_M, BLK_N, BLK_K, gsize_m, two_tiles, num_stages,
num_warps, waves_per_eu, mfmaInstrSize, kpack, heap_bases_ptr, cu_count,
COLLECT_TIMESTAMPS, mm_begin_timestamp, mm_end_timestamp)`` keeps the
positional signature of the reference's three (identical) wrappers
(examples/0{7,8,9}_*/matmul_wrapper.py:161-219) and launches the HIP kernel in
place of the Triton one (:109-150).

Arguments that only steer the Triton compiler (``num_stages``, ``num_warps``,
``waves_per_eu``, ``mfmaInstrSize``, ``kpack``) and ``two_tiles`` are accepted
and ignored; ``BLK_K`` does not change any result.  ``P`` and ``locks``, which
the reference allocates and never reads, serve as workspace when they have
the reference's shapes (split-K partials; arrival counters of the few-rows
kernel) and are ignored otherwise.  ``bias`` is never applied (the reference
forces ``BIAS=False``, matmul_wrapper.py:104).
"""

from __future__ import annotations

import torch

from . import ops

__all__ = ["make_matmul", "matmul_all_scatter", "matmul_atomics_all_reduce", "matmul_one_shot_all_reduce"]


def _workspace_ok(P, locks, programs, BLK_M, BLK_N):
    """Whether the caller's P / locks buffers (benchmark.py:136-142) can serve
    as the split-K workspace: fp32 [programs, BLK_M*BLK_N] and int32 [programs]."""
    return (isinstance(P, torch.Tensor) and isinstance(locks, torch.Tensor) and P.is_cuda and locks.is_cuda
            and P.dtype == torch.float32 and locks.dtype == torch.int32 and P.dim() == 2 and P.is_contiguous()
            and locks.is_contiguous() and P.shape[0] >= programs and locks.numel() >= programs
            and P.shape[1] >= BLK_M * BLK_N)


def _streamk_report(M, N, K, BLK_M, BLK_N, BLK_K, programs):
    """The split the reference prints in debug mode (matmul_wrapper.py:67-102);
    its kernels never use it."""
    blocks_m, blocks_n = ops.cdiv(M, BLK_M), ops.cdiv(N, BLK_N)
    total_tiles = blocks_m * blocks_n
    iters_per_tile = ops.cdiv(K, BLK_K)
    sk_tiles = total_tiles % programs if programs > 0 else 0
    blocking = total_tiles - sk_tiles
    sk_iters = sk_tiles * iters_per_tile
    full = sk_iters // programs if programs > 0 else 0
    partial = sk_iters % programs if programs > 0 else 0
    print(f"M,N,K={M},{N},{K} ; BLK_M,N,K={BLK_M},{BLK_N},{BLK_K}")
    print(f"total_blocks_M={blocks_m} x total_blocks_N={blocks_n} = total_tiles={total_tiles}")
    print(f"total_tiles_streamk={sk_tiles} + total_blocking_tiles={blocking} = total_tiles={total_tiles}")
    print(f"total_programs_streamk={programs}")
    print(f"total_blocking_tiles={blocking}")
    print(f"total_full_tiles_streamk={full}")
    print(f"iters_per_tile={iters_per_tile}")
    print(f"total_iters_streamk={sk_iters}")
    print("total_remainder_iters_streamk=", partial)


def make_matmul(epilogue: int, name: str):
    class matmul(torch.autograd.Function):
        _debug = True
        streamk_registers = 0
        streamk_spills = 0
        # knobs that have no counterpart in the positional signature
        notify = True            # all-scatter: publish a ready flag per tile
        phase = ops.PHASE_FUSED  # one-shot: produce, consume or both
        scope = ops.SCOPE_AGENT
        variant = 0
        status = None            # optional int32 device word for flag-wait timeouts
        spin_timeout_ticks = 0
        split_k = 0  # 0: the launcher decides, 1: never split K, n: exactly n parts

        @staticmethod
        def set_debug(debug: bool):
            matmul._debug = debug
            matmul.streamk_registers = 0
            matmul.streamk_spills = 0

        @staticmethod
        def _call(a, b, c, c_global, bias, P, locks, tile_completed, rank, world_size, total_programs_streamk,
                  BLK_M, BLK_N, BLK_K, gsize_m, two_tiles, num_stages, num_warps, waves_per_eu, mfmaInstrSize,
                  kpack, heap_bases_ptr=None, cu_count=304, COLLECT_TIMESTAMPS=False, mm_begin_timestamp=None,
                  mm_end_timestamp=None):
            assert a.shape[1] == b.shape[0], "incompatible dimensions"
            M, K = a.shape
            _, N = b.shape
            if matmul._debug:
                _streamk_report(M, N, K, BLK_M, BLK_N, BLK_K, total_programs_streamk)
            launch = dict(
                a=a, b=b, c=c, c_global=c_global, tile_completed=tile_completed, heap_bases=heap_bases_ptr,
                rank=rank, world_size=world_size, num_sms=total_programs_streamk, BLK_M=BLK_M, BLK_N=BLK_N,
                BLK_K=BLK_K, gsize_m=gsize_m, epilogue=epilogue, phase=matmul.phase, notify=matmul.notify,
                num_xcds=ops.default_num_xcds(cu_count, total_programs_streamk), variant=matmul.variant,
            )
            ops.gemm_launch(
                **launch,
                partials=P if _workspace_ok(P, locks, total_programs_streamk, BLK_M, BLK_N) else None,
                locks=locks if _workspace_ok(P, locks, total_programs_streamk, BLK_M, BLK_N) else None,
                split_k=matmul.split_k,
                scope=matmul.scope,
                mm_begin_timestamp=mm_begin_timestamp if COLLECT_TIMESTAMPS else None,
                mm_end_timestamp=mm_end_timestamp if COLLECT_TIMESTAMPS else None,
                status=matmul.status,
                spin_timeout_ticks=matmul.spin_timeout_ticks,
            )
            if matmul._debug:
                regs, spills = ops.gemm_kernel_info(**launch)
                matmul.streamk_registers, matmul.streamk_spills = regs, spills
                print(f"{regs} registers used, {spills} spills")
            return c

        @staticmethod
        def forward(ctx, a, b, c, c_global, bias, P, locks, tile_completed, rank, world_size, grid, BLK_M=128,
                    BLK_N=128, BLK_K=32, gsize_m=1, two_tiles=True, num_stages=3, num_warps=4, waves_per_eu=2,
                    mfmaInstrSize=16, kpack=1, heap_bases_ptr=None, cu_count=304, COLLECT_TIMESTAMPS=False,
                    mm_begin_timestamp=None, mm_end_timestamp=None):
            matmul._call(a, b, c, c_global, bias, P, locks, tile_completed, rank, world_size, grid, BLK_M, BLK_N,
                         BLK_K, gsize_m, two_tiles, num_stages, num_warps, waves_per_eu, mfmaInstrSize, kpack,
                         heap_bases_ptr, cu_count, COLLECT_TIMESTAMPS, mm_begin_timestamp, mm_end_timestamp)
            return c

    matmul.__name__ = "matmul"
    matmul.__qualname__ = f"matmul[{name}]"
    return matmul


matmul_all_scatter = make_matmul(ops.EPI_ALL_SCATTER, "all_scatter")
matmul_atomics_all_reduce = make_matmul(ops.EPI_ATOMIC_ADD, "atomics_all_reduce")
matmul_one_shot_all_reduce = make_matmul(ops.EPI_ONE_SHOT, "one_shot_all_reduce")
