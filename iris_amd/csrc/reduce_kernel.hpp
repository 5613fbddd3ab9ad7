// One-shot reduce: the consumer half of
// examples/09_gemm_one_shot_all_reduce/gemm_one_shot_all_reduce.py:220-271 as a
// kernel of its own.  For every tile: wait until the tile's flag shows that
// all other ranks have published their partial (CAS ws-1 -> 0, acquire), sum
// the tile over ranks 0..ws-1 in fp32 and store it to c_global.
//
// The kernel is HBM-bound: per output element it reads ws partials and writes
// one result.  Each lane moves one 16-byte strip per rank and step, lanes run
// along a row so that a wave covers contiguous row segments, and the strips
// of several rows are kept in flight.
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
  // row-band kernel: an item is `band_rows` rows x `band_vecs` 16-byte strips
  int band_rows, band_vecs, band_chunks, band_items;
  // tile kernel: fetch the ranks' heap bases with vector loads (see there)
  int pace;
  // row-band kernel: the group that finishes last takes the consumed flags
  // back to 0 (else the launcher enqueues reset_consumed_flags_kernel)
  int reset_in_kernel;
  // an acquire fence at the flags' scope after every flag wait, as the reference's sem="acquire" (the loads are
  // coherent at that scope by themselves and need none)
  int acquire;
};

// The row-band kernel counts its finished groups in the upper half of the
// first tile's flag (a producer's +1 only ever touches the lower half), so a
// flag's value is its lower half.
constexpr int FLAG_COUNT_SHIFT = 16, FLAG_VALUE_MASK = 0xFFFF;

// Block-wide wait for one tile's flag.  One lane polls; the outcome is
// broadcast through LDS and every wave then acquires.
template <bool FENCE = true>
__device__ inline bool block_wait_tile(const ReduceKArgs& p, int tile_id, IRIS_LDS int* slot) {
  if (!p.wait_flags || p.ws <= 1) return true;
  if (threadIdx.x == 0)
    *slot = wait_tile_flag((IRIS_GLOBAL int32_t*)(p.flags + tile_id), p.ws, p.sys != 0, p.timeout, p.status) ? 1 : 0;
  __syncthreads();
  const int ok = *slot;
  if (FENCE || p.acquire) {
    if (p.sys)
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
    else
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  __syncthreads();  // the slot may be rewritten for the next tile
  return ok != 0;
}

// Vector kernel: unit-stride columns, 16-byte aligned rows, tile widths that
// are multiples of the vector width.  WS > 0 fixes the rank count at compile
// time.  A lane owns one 16-byte strip per rank; UNROLL rows of the tile are
// in flight per lane, i.e. WS * UNROLL independent loads.
template <int IN_DT, int OUT_DT, int WS, int UNROLL, int LAUX>
__global__ __launch_bounds__(256) void reduce_tiles_vec_kernel(const ReduceKArgs p) {
  // Loads that carry sc1 are coherent at the flags' scope by themselves: they
  // never hit a stale line, so the wait needs no cache-invalidating fence.
  constexpr bool FENCE = (LAUX & AUX_SC1) == 0;
  __shared__ int slot;
  const int ws = WS > 0 ? WS : p.ws;
  constexpr int IES = Vec<IN_DT>::ES, VE = Vec<IN_DT>::N;
  constexpr int OES = Vec<OUT_DT>::ES;
  const int tid = threadIdx.x;
  const uint64_t cur_base = p.heap_bases ? uniform_u64(p.heap_bases[p.cur_rank]) : 0;

  for (int tile_id = xcd_remap(blockIdx.x, gridDim.x, p.num_xcds); tile_id < p.total_tiles; tile_id += gridDim.x) {
    const TileCoord tc = tile_map(tile_id, p.num_pid_m, p.num_pid_n, p.G);
    const int m0 = tc.pid_m * p.BM, n0 = tc.pid_n * p.BN;
    const int rows = min(p.M, m0 + p.BM) - m0, cols = min(p.N, n0 + p.BN) - n0;
    if (!block_wait_tile<FENCE>(p, tile_id, (IRIS_LDS int*)&slot)) continue;
    const int cv = cols / VE;  // 16-byte strips per tile row
    // Lanes run along a tile row; the block covers `rpp` rows per pass and
    // UNROLL passes are in flight.
    const int tpr = min(cv, 256), rpp = 256 / tpr;
    const int r0 = tid / tpr, cl = tid - r0 * tpr;
    const uint32_t in_bytes = ((uint32_t)(rows - 1) * (uint32_t)p.scm + cols) * IES;
    const uint32_t out_bytes = ((uint32_t)(rows - 1) * (uint32_t)p.sgm + cols) * OES;
    const int64_t in0 = ((int64_t)m0 * p.scm + n0) * IES;
    const __amdgpu_buffer_rsrc_t out_rs =
        tile_rsrc((const IRIS_GLOBAL char*)p.cg + ((int64_t)m0 * p.sgm + n0) * OES, out_bytes);
    // With many tiles per program the bases come through vector loads on
    // purpose: the wait for the outstanding loads that such a load forces
    // between the ranks' batches paces the tile walk, and measured 9% faster
    // than scalar loads of them.  A program with a single small tile has
    // nothing to pace and eight round trips to lose: its bases come through
    // scalar loads and all ranks' strips are in flight together.
    auto rank_rsrc = [&](int rk) __attribute__((always_inline)) {
      const IRIS_GLOBAL char* b = (const IRIS_GLOBAL char*)p.c;
      if (rk != p.cur_rank && p.heap_bases)
        b = translate(p.c, cur_base,
                      p.pace ? uniform_u64(p.heap_bases[rk]) : uniform_u64(heap_base_at(p.heap_bases, rk)));
      return tile_rsrc(b + in0, in_bytes);
    };

    for (int cc = 0; cc < cv; cc += tpr) {
      const int c = cc + cl;
      const bool col_live = r0 < rpp && c < cv;
      for (int rb = 0; rb < rows; rb += rpp * UNROLL) {
        float acc[UNROLL][VE];
        uint32_t ioff[UNROLL], ooff[UNROLL];
#pragma unroll
        for (int s = 0; s < UNROLL; ++s) {
          const uint32_t row = rb + r0 + s * rpp;
          ioff[s] = col_live ? (row * (uint32_t)p.scm + c * VE) * IES : DEAD_OFFSET;
          ooff[s] = col_live ? (row * (uint32_t)p.sgm + c * VE) * OES : DEAD_OFFSET;
#pragma unroll
          for (int e = 0; e < VE; ++e) acc[s][e] = 0.f;
        }
        // fixed rank order 0..ws-1 (gemm_one_shot_all_reduce.py:267-269)
        if constexpr (WS > 0) {
          float v[WS][UNROLL][VE];
#pragma unroll
          for (int rk = 0; rk < WS; ++rk) {
            const __amdgpu_buffer_rsrc_t rs = rank_rsrc(rk);
#pragma unroll
            for (int s = 0; s < UNROLL; ++s) load_vec<IN_DT, LAUX>(rs, ioff[s], v[rk][s]);
          }
#pragma unroll
          for (int rk = 0; rk < WS; ++rk)
#pragma unroll
            for (int s = 0; s < UNROLL; ++s)
#pragma unroll
              for (int e = 0; e < VE; ++e) acc[s][e] += v[rk][s][e];
        } else {
          for (int rk = 0; rk < ws; ++rk) {
            const __amdgpu_buffer_rsrc_t rs = rank_rsrc(rk);
            float v[UNROLL][VE];
#pragma unroll
            for (int s = 0; s < UNROLL; ++s) load_vec<IN_DT, LAUX>(rs, ioff[s], v[s]);
#pragma unroll
            for (int s = 0; s < UNROLL; ++s)
#pragma unroll
              for (int e = 0; e < VE; ++e) acc[s][e] += v[s][e];
          }
        }
#pragma unroll
        for (int s = 0; s < UNROLL; ++s) store_vec<OUT_DT, VE, AUX_NT>(out_rs, ooff[s], acc[s]);
      }
    }
  }
}

// Row-band kernel, for matrices whose rows are long.  The tile kernel above
// reads a tile as 1 KiB row segments 32 KiB apart; here a group of 256 threads
// takes `band_rows` whole rows (or an 8192-column chunk of one row) at a time,
// 32 KiB of contiguous memory per partial, and streams the partials one after
// another, the next one in flight while the current one is added.  Adjacent
// groups read adjacent rows.  On [8192, 8192] fp32 x 8 this is what the HBM
// likes best: about 8% more bandwidth than the tile walk.
//
// Flags: the band crosses every tile of its tile row, so the group waits for
// all of them (one lane per tile) without consuming them; a tile that does
// not arrive within the timeout only masks its own columns.  The flags that
// reached ws-1 are reset to 0 by the group that finishes last (the groups
// count themselves on the upper half of the first flag), or, for grids too
// large for that count, by reset_consumed_flags_kernel, which the launcher
// then enqueues behind this kernel.  The sum is in rank order 0..ws-1.
template <int IN_DT, int OUT_DT, int LAUX, int WS>
__global__ __launch_bounds__(256) void reduce_rows_kernel(const ReduceKArgs p) {
  constexpr int IES = Vec<IN_DT>::ES, VE = Vec<IN_DT>::N, OES = Vec<OUT_DT>::ES;
  constexpr int K = 32 / VE;  // strips per lane: 8192 elements per item
  // the result is written through, like the reference's store (cache_modifier=".wt")
  // (measured on 8 x fp32 [8192,8192]: sc1 353 us, nt sc1 364, nt 362, plain write-back stores 379)
  constexpr int SAUX = (LAUX & AUX_SC0) ? (AUX_SC0 | AUX_SC1) : AUX_SC1;
  __shared__ int ready[256];
  const int tid = threadIdx.x;
  const uint64_t cur_base = p.heap_bases ? uniform_u64(heap_base_at(p.heap_bases, p.cur_rank)) : 0;
  const bool wait = p.wait_flags && p.ws > 1;
  // the partial buffer of every rank, looked up once
  const IRIS_GLOBAL char* rank_c[WS > 0 ? WS : 1];
  if constexpr (WS > 0) {
#pragma unroll
    for (int rk = 0; rk < WS; ++rk)
      rank_c[rk] = (rk == p.cur_rank || !p.heap_bases)
                       ? (const IRIS_GLOBAL char*)p.c
                       : translate(p.c, cur_base, uniform_u64(heap_base_at(p.heap_bases, rk)));
  }

  // strip k of this lane: row `rr` of the band, strip `cv` of the row chunk
  uint32_t ibase[K], obase[K];
  int colv[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int j = k * 256 + tid;
    const int rr = j / p.band_vecs, cv = j - rr * p.band_vecs;
    const bool live = rr < p.band_rows;
    colv[k] = live ? cv * VE : 0x40000000;  // a dead strip's column is past every row
    ibase[k] = ((uint32_t)rr * (uint32_t)p.scm + cv * VE) * IES;
    obase[k] = ((uint32_t)rr * (uint32_t)p.sgm + cv * VE) * OES;
  }

  for (int item = blockIdx.x; item < p.band_items; item += gridDim.x) {
    const int rg = item / p.band_chunks, ch = item - rg * p.band_chunks;
    const int row0 = rg * p.band_rows, col0 = ch * p.band_vecs * VE;
    const int rows = min(p.band_rows, p.M - row0), cols = min(p.band_vecs * VE, p.N - col0);
    const int tn0 = col0 / p.BN;
    bool all = true;
    if (wait) {
      const int ntn = (col0 + cols - 1) / p.BN - tn0 + 1;
      int ok = 1;
      if (tid < ntn) {
        const int t = tile_id_of(row0 / p.BM, tn0 + tid, p.num_pid_m, p.num_pid_n, p.G);
        ok = wait_tile_ready((IRIS_GLOBAL int32_t*)(p.flags + t), p.ws - 1, p.sys != 0, p.timeout, p.status,
                             FLAG_VALUE_MASK)
                 ? 1
                 : 0;
        ready[tid] = ok;
      }
      all = __syncthreads_and(ok) != 0;
      if (p.acquire) {
        if (p.sys)
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "");
        else
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      }
    }
    uint32_t ioff[K], ooff[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      bool live = colv[k] < cols;
      if (!all && live) live = ready[(col0 + colv[k]) / p.BN - tn0] != 0;
      ioff[k] = live ? ibase[k] : DEAD_OFFSET;
      ooff[k] = live ? obase[k] : DEAD_OFFSET;
    }
    const uint32_t in_bytes = ((uint32_t)(rows - 1) * (uint32_t)p.scm + cols) * IES;
    const uint32_t out_bytes = ((uint32_t)(rows - 1) * (uint32_t)p.sgm + cols) * OES;
    const int64_t in0 = ((int64_t)row0 * p.scm + col0) * IES;
    auto rank_rsrc = [&](int rk) __attribute__((always_inline)) {
      const IRIS_GLOBAL char* b;
      if constexpr (WS > 0)
        b = rank_c[rk];
      else
        b = (rk == p.cur_rank || !p.heap_bases)
                ? (const IRIS_GLOBAL char*)p.c
                : translate(p.c, cur_base, uniform_u64(heap_base_at(p.heap_bases, rk)));
      return tile_rsrc(b + in0, in_bytes);
    };
    float acc[K][VE], v[2][K][VE];
    {
      const __amdgpu_buffer_rsrc_t rs = rank_rsrc(0);
#pragma unroll
      for (int k = 0; k < K; ++k) load_vec<IN_DT, LAUX>(rs, ioff[k], v[0][k]);
    }
    if constexpr (WS > 0) {
      // rank count known: the whole pipeline is straight-line code
#pragma unroll
      for (int rk = 0; rk < WS; ++rk) {
        if (rk + 1 < WS) {
          const __amdgpu_buffer_rsrc_t rs = rank_rsrc(rk + 1);
#pragma unroll
          for (int k = 0; k < K; ++k) load_vec<IN_DT, LAUX>(rs, ioff[k], v[(rk + 1) & 1][k]);
        }
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < VE; ++e) acc[k][e] = (rk == 0 ? 0.f : acc[k][e]) + v[rk & 1][k][e];
      }
    } else {
      // ranks two at a time, so that the double buffer is indexed statically
      for (int rk = 0; rk < p.ws; rk += 2) {
        if (rk + 1 < p.ws) {
          const __amdgpu_buffer_rsrc_t rs = rank_rsrc(rk + 1);
#pragma unroll
          for (int k = 0; k < K; ++k) load_vec<IN_DT, LAUX>(rs, ioff[k], v[1][k]);
        }
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
          for (int e = 0; e < VE; ++e) acc[k][e] = (rk == 0 ? 0.f : acc[k][e]) + v[0][k][e];
        if (rk + 1 < p.ws) {
          if (rk + 2 < p.ws) {
            const __amdgpu_buffer_rsrc_t rs = rank_rsrc(rk + 2);
#pragma unroll
            for (int k = 0; k < K; ++k) load_vec<IN_DT, LAUX>(rs, ioff[k], v[0][k]);
          }
#pragma unroll
          for (int k = 0; k < K; ++k)
#pragma unroll
            for (int e = 0; e < VE; ++e) acc[k][e] += v[1][k][e];
        }
      }
    }
    const __amdgpu_buffer_rsrc_t out_rs =
        tile_rsrc((const IRIS_GLOBAL char*)p.cg + ((int64_t)row0 * p.sgm + col0) * OES, out_bytes);
#pragma unroll
    for (int k = 0; k < K; ++k) store_vec<OUT_DT, VE, SAUX>(out_rs, ooff[k], acc[k]);
    if (wait) __syncthreads();  // `ready` is rewritten for the next item
  }
  if (wait && p.reset_in_kernel) {
    // This group is past all its waits.  Groups count themselves on the upper
    // half of flags[0]; the one that counts last knows that nobody polls any
    // more and takes every flag that reached ws-1 back to 0, which is what the
    // consumer's CAS(ws-1 -> 0) leaves (gemm_one_shot_all_reduce.py:228-234).
    // The count comes off with one atomic per flag, so a +1 of the next round
    // that lands meanwhile is kept.
    if (tid == 0) {
      // (at the flags' scope, like the producers' increments of the same word)
      const int before = p.sys ? __hip_atomic_fetch_add((IRIS_GLOBAL int32_t*)p.flags, 1 << FLAG_COUNT_SHIFT,
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)
                               : __hip_atomic_fetch_add((IRIS_GLOBAL int32_t*)p.flags, 1 << FLAG_COUNT_SHIFT,
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ready[0] = (before >> FLAG_COUNT_SHIFT) == (int)gridDim.x - 1 ? 1 : 0;
    }
    __syncthreads();
    if (ready[0]) {
      const int consumed = p.ws - 1;
      for (int t = tid; t < p.total_tiles; t += 256) {
        IRIS_GLOBAL int32_t* f = (IRIS_GLOBAL int32_t*)(p.flags + t);
        const int v = p.sys ? __hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)
                            : __hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int take = (v & FLAG_VALUE_MASK) >= consumed ? consumed : 0;
        if (t == 0) take += (int)gridDim.x << FLAG_COUNT_SHIFT;  // the groups' count, too
        if (take) flag_add_relaxed(f, -take, p.sys != 0);
      }
    }
  }
}

// Flags that the row-band kernel has consumed (value ws-1) back to 0, as the
// consumer's CAS(ws-1 -> 0) leaves them (gemm_one_shot_all_reduce.py:228-234):
// the stand-in, as a kernel behind the reduce, for the reset by the group
// that finishes last, when the grid is too large for that group count.  The
// count is taken off with one atomic: a +1 of the next round that lands on
// the flag meanwhile is kept.
__global__ __launch_bounds__(256) void reset_consumed_flags_kernel(int32_t* flags, int consumed, int total) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= total) return;
  IRIS_GLOBAL int32_t* f = (IRIS_GLOBAL int32_t*)(flags + t);
  if (__hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= consumed)
    __hip_atomic_fetch_add(f, -consumed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
                                                            int num_sms, int num_xcds, TileDivs divs) {
  const int prog = blockIdx.x * 256 + threadIdx.x;
  if (prog >= num_sms) return;
  const int total = num_pid_m * num_pid_n;
  int pos = 0;
  for (int t = xcd_remap(prog, num_sms, num_xcds); t < total; t += num_sms, ++pos) {
    const TileCoord tc = tile_map_fast(t, num_pid_m, num_pid_n, G, divs);  // as the GEMM kernels decode a tile
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
