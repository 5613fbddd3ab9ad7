// One-shot reduce: the consumer half of
// examples/09_gemm_one_shot_all_reduce/gemm_one_shot_all_reduce.py:220-271 as a
// kernel of its own.  For every tile: wait until the tile's flag shows that
// all other ranks have published their partial (CAS ws-1 -> 0, acquire), sum
// the tile over ranks 0..ws-1 in fp32 and store it to c_global.
//
// The kernel is HBM-bound: per output element it reads ws partials and writes
// one result.  Each lane moves 8 consecutive columns per step (two 16-byte
// loads per rank for fp32 partials), lanes run along a row so that a wave
// covers whole contiguous row segments, and several steps are kept in flight.
#pragma once

#include "common.hpp"

namespace iris_amd {

struct ReduceKArgs {
  const char* c;  // this rank's partial buffer
  char* cg;
  int32_t* flags;
  const uint64_t* heap_bases;
  uint32_t* status;
  uint64_t timeout;
  int64_t scm, scn, sgm, sgn;
  int M, N, BM, BN, G;
  int num_pid_m, num_pid_n, total_tiles;
  int num_xcds, cur_rank, ws;
  int c_dt, cg_dt;
  int sys, wait_flags;
};

template <int DT, bool NT>
__device__ inline void load8(const IRIS_GLOBAL char* p, float (&v)[8]) {
  if constexpr (DT == IRIS_DTYPE_F32) {
    const IRIS_GLOBAL f32x4* q = reinterpret_cast<const IRIS_GLOBAL f32x4*>(p);
    const f32x4 x0 = NT ? __builtin_nontemporal_load(q) : q[0];
    const f32x4 x1 = NT ? __builtin_nontemporal_load(q + 1) : q[1];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[e] = x0[e];
      v[4 + e] = x1[e];
    }
  } else {
    const IRIS_GLOBAL u32x4* q = reinterpret_cast<const IRIS_GLOBAL u32x4*>(p);
    const u32x4 x = NT ? __builtin_nontemporal_load(q) : q[0];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = from16<DT>((unsigned short)(x[e / 2] >> (16 * (e & 1))));
  }
}

template <int DT, bool NT>
__device__ inline void store8(IRIS_GLOBAL char* p, const float (&v)[8]) {
  if constexpr (DT == IRIS_DTYPE_F32) {
    IRIS_GLOBAL f32x4* q = reinterpret_cast<IRIS_GLOBAL f32x4*>(p);
    const f32x4 y0 = {v[0], v[1], v[2], v[3]}, y1 = {v[4], v[5], v[6], v[7]};
    if (NT) {
      __builtin_nontemporal_store(y0, q);
      __builtin_nontemporal_store(y1, q + 1);
    } else {
      q[0] = y0;
      q[1] = y1;
    }
  } else {
    const u32x4 y = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3]), pack2<DT>(v[4], v[5]), pack2<DT>(v[6], v[7])};
    if (NT)
      __builtin_nontemporal_store(y, reinterpret_cast<IRIS_GLOBAL u32x4*>(p));
    else
      *reinterpret_cast<IRIS_GLOBAL u32x4*>(p) = y;
  }
}

// Block-wide wait for one tile's flag.  One lane polls; the outcome is
// broadcast through LDS and every wave then acquires.
__device__ inline bool block_wait_tile(const ReduceKArgs& p, int tile_id, IRIS_LDS int* slot) {
  if (!p.wait_flags || p.ws <= 1) return true;
  if (threadIdx.x == 0)
    *slot = wait_tile_flag((IRIS_GLOBAL int32_t*)(p.flags + tile_id), p.ws, p.sys != 0, p.timeout, p.status) ? 1 : 0;
  __syncthreads();
  const int ok = *slot;
  if (p.sys)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
  else
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  __syncthreads();  // the slot may be rewritten for the next tile
  return ok != 0;
}

// Vector kernel: unit-stride columns, 16-byte aligned rows, tile widths that
// are multiples of 8.  WS > 0 fixes the rank count at compile time.
template <int IN_DT, int OUT_DT, int WS, int UNROLL, bool NT>
__global__ __launch_bounds__(256) void reduce_tiles_vec_kernel(const ReduceKArgs p) {
  __shared__ int slot;
  const int ws = WS > 0 ? WS : p.ws;
  constexpr int IES = (IN_DT == IRIS_DTYPE_F32) ? 4 : 2;
  constexpr int OES = (OUT_DT == IRIS_DTYPE_F32) ? 4 : 2;
  const int tid = threadIdx.x;
  const uint64_t cur_base = p.heap_bases ? p.heap_bases[p.cur_rank] : 0;

  for (int tile_id = xcd_remap(blockIdx.x, gridDim.x, p.num_xcds); tile_id < p.total_tiles; tile_id += gridDim.x) {
    const TileCoord tc = tile_map(tile_id, p.num_pid_m, p.num_pid_n, p.G);
    const int m0 = tc.pid_m * p.BM, n0 = tc.pid_n * p.BN;
    const int rows = min(p.M, m0 + p.BM) - m0, cols = min(p.N, n0 + p.BN) - n0;
    if (!block_wait_tile(p, tile_id, (IRIS_LDS int*)&slot)) continue;
    const int c8 = cols / 8;
    const int units = rows * c8;
    IRIS_GLOBAL char* out0 = (IRIS_GLOBAL char*)p.cg + ((int64_t)m0 * p.sgm + n0) * OES;
    const int64_t in0 = ((int64_t)m0 * p.scm + n0) * IES;

    for (int u0 = tid; u0 < units; u0 += 256 * UNROLL) {
      float acc[UNROLL][8];
      int64_t ioff[UNROLL], ooff[UNROLL];
      bool live[UNROLL];
#pragma unroll
      for (int s = 0; s < UNROLL; ++s) {
        const int u = u0 + s * 256;
        live[s] = u < units;
        const int uu = live[s] ? u : 0;
        const int r = uu / c8, c = (uu - r * c8) * 8;
        ioff[s] = in0 + ((int64_t)r * p.scm + c) * IES;
        ooff[s] = ((int64_t)r * p.sgm + c) * OES;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[s][e] = 0.f;
      }
      // fixed rank order 0..ws-1 (gemm_one_shot_all_reduce.py:267-269)
      if constexpr (WS > 0) {
        float v[WS][UNROLL][8];
#pragma unroll
        for (int rk = 0; rk < WS; ++rk) {
          const IRIS_GLOBAL char* base = (rk == p.cur_rank || !p.heap_bases)
                                             ? (const IRIS_GLOBAL char*)p.c
                                             : translate(p.c, cur_base, p.heap_bases[rk]);
#pragma unroll
          for (int s = 0; s < UNROLL; ++s) load8<IN_DT, NT>(base + ioff[s], v[rk][s]);
        }
#pragma unroll
        for (int rk = 0; rk < WS; ++rk)
#pragma unroll
          for (int s = 0; s < UNROLL; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[s][e] += v[rk][s][e];
      } else {
        for (int rk = 0; rk < ws; ++rk) {
          const IRIS_GLOBAL char* base = (rk == p.cur_rank || !p.heap_bases)
                                             ? (const IRIS_GLOBAL char*)p.c
                                             : translate(p.c, cur_base, p.heap_bases[rk]);
          float v[UNROLL][8];
#pragma unroll
          for (int s = 0; s < UNROLL; ++s) load8<IN_DT, NT>(base + ioff[s], v[s]);
#pragma unroll
          for (int s = 0; s < UNROLL; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[s][e] += v[s][e];
        }
      }
#pragma unroll
      for (int s = 0; s < UNROLL; ++s)
        if (live[s]) store8<OUT_DT, NT>(out0 + ooff[s], acc[s]);
    }
  }
}

// Element-wise kernel: any strides, alignment, tile shape and element types.
__global__ __launch_bounds__(256) void reduce_tiles_generic_kernel(const ReduceKArgs p) {
  __shared__ int slot;
  const int tid = threadIdx.x;
  const uint64_t cur_base = p.heap_bases ? p.heap_bases[p.cur_rank] : 0;
  const int ies = dtype_size(p.c_dt), oes = dtype_size(p.cg_dt);
  for (int tile_id = xcd_remap(blockIdx.x, gridDim.x, p.num_xcds); tile_id < p.total_tiles; tile_id += gridDim.x) {
    const TileCoord tc = tile_map(tile_id, p.num_pid_m, p.num_pid_n, p.G);
    const int m0 = tc.pid_m * p.BM, n0 = tc.pid_n * p.BN;
    const int rows = min(p.M, m0 + p.BM) - m0, cols = min(p.N, n0 + p.BN) - n0;
    if (!block_wait_tile(p, tile_id, (IRIS_LDS int*)&slot)) continue;
    for (int idx = tid; idx < rows * cols; idx += 256) {
      const int r = idx / cols, cidx = idx - r * cols;
      const int64_t ioff = ((int64_t)(m0 + r) * p.scm + (int64_t)(n0 + cidx) * p.scn) * ies;
      float acc = 0.f;
      for (int rk = 0; rk < p.ws; ++rk) {
        const IRIS_GLOBAL char* src = ((rk == p.cur_rank || !p.heap_bases) ? (const IRIS_GLOBAL char*)p.c
                                                                            : translate(p.c, cur_base, p.heap_bases[rk])) +
                                      ioff;
        if (p.c_dt == IRIS_DTYPE_F32)
          acc += *reinterpret_cast<const IRIS_GLOBAL float*>(src);
        else if (p.c_dt == IRIS_DTYPE_BF16)
          acc += bf16_bits_to_f32(*reinterpret_cast<const IRIS_GLOBAL unsigned short*>(src));
        else
          acc += f16_bits_to_f32(*reinterpret_cast<const IRIS_GLOBAL unsigned short*>(src));
      }
      IRIS_GLOBAL char* d = (IRIS_GLOBAL char*)p.cg + ((int64_t)(m0 + r) * p.sgm + (int64_t)(n0 + cidx) * p.sgn) * oes;
      if (p.cg_dt == IRIS_DTYPE_F32)
        *reinterpret_cast<IRIS_GLOBAL float*>(d) = acc;
      else if (p.cg_dt == IRIS_DTYPE_BF16)
        *reinterpret_cast<IRIS_GLOBAL unsigned short*>(d) = f32_to_bf16_bits(acc);
      else
        *reinterpret_cast<IRIS_GLOBAL unsigned short*>(d) = f32_to_f16_bits(acc);
    }
  }
}

// +1 (release) on tile_completed[tile] of the other ranks (or of every rank);
// gemm_one_shot_all_reduce.py:207-218 on its own.
__global__ __launch_bounds__(256) void signal_tiles_kernel(int32_t* flags, const uint64_t* heap_bases, int total_tiles,
                                                           int cur_rank, int ws, int include_self, int sys) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= total_tiles) return;
  const uint64_t cur_base = heap_bases ? heap_bases[cur_rank] : 0;
  for (int r = 0; r < ws; ++r) {
    if (r == cur_rank && !include_self) continue;
    IRIS_GLOBAL int32_t* f = (r == cur_rank || !heap_bases) ? (IRIS_GLOBAL int32_t*)(flags + t)
                                                            : translate(flags + t, cur_base, heap_bases[r]);
    flag_add_release(f, 1, sys != 0);
  }
}

// The tile schedule as the kernels compute it, one row per tile id:
// (pid_m, pid_n, owning program, position in that program's tile list).
// Program p of a grid of num_sms visits xcd_remap(p), +num_sms, ...
__global__ __launch_bounds__(256) void tile_schedule_kernel(int32_t* out, int num_pid_m, int num_pid_n, int G,
                                                            int num_sms, int num_xcds) {
  const int prog = blockIdx.x * 256 + threadIdx.x;
  if (prog >= num_sms) return;
  const int total = num_pid_m * num_pid_n;
  int pos = 0;
  for (int t = xcd_remap(prog, num_sms, num_xcds); t < total; t += num_sms, ++pos) {
    const TileCoord tc = tile_map(t, num_pid_m, num_pid_n, G);
    out[4 * t + 0] = tc.pid_m;
    out[4 * t + 1] = tc.pid_n;
    out[4 * t + 2] = prog;
    out[4 * t + 3] = pos;
  }
}

// int32 fill; iris/util.py:107-114.
__global__ __launch_bounds__(256) void memset_i32_kernel(int32_t* ptr, int32_t value, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 1024 + threadIdx.x;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t k = i + j * 256;
    if (k < n) ptr[k] = value;
  }
}

}  // namespace iris_amd
