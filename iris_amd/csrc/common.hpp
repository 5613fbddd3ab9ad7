// Shared device/host helpers for the gfx950 kernels of the fused GEMM +
// tile-publishing path.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/iris_amd.h"

namespace iris_amd {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

#define IRIS_LDS __attribute__((address_space(3)))
// Device memory.  Pointers rebuilt from integers would otherwise be "flat",
// and flat accesses tie the LDS counter to the vector-memory counter.
#define IRIS_GLOBAL __attribute__((address_space(1)))

// s_waitcnt immediates for gfx9-family encodings: vmcnt[3:0] in bits 3:0,
// vmcnt[5:4] in bits 15:14, expcnt in 6:4, lgkmcnt in 11:8.  These leave
// expcnt and lgkmcnt unconstrained.
#define IRIS_WAIT_VMCNT(n) \
  __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (0x7 << 4) | (0xF << 8) | ((((n) >> 4) & 0x3) << 14))
#define IRIS_WAIT_LGKMCNT0() __builtin_amdgcn_s_waitcnt(0xC07F)

struct TileCoord {
  int pid_m;
  int pid_n;
};

// tile_id -> (pid_m, pid_n) with the GROUP_SIZE_M swizzle; the arithmetic of
// examples/09_gemm_one_shot_all_reduce/gemm_one_shot_all_reduce.py:155-160.
__host__ __device__ inline TileCoord tile_map(int tile_id, int num_pid_m, int num_pid_n, int G) {
  const int num_pid_in_group = G * num_pid_n;
  const int group_id = tile_id / num_pid_in_group;
  const int first_pid_m = group_id * G;
  const int rem = num_pid_m - first_pid_m;
  const int group_size_m = rem < G ? rem : G;
  const int in_group = tile_id % num_pid_in_group;
  TileCoord t;
  t.pid_m = first_pid_m + (in_group % group_size_m);
  t.pid_n = in_group / group_size_m;
  return t;
}

// Division of a launch's small integers (tile and item indices) by a divisor
// that is fixed for the launch, as a multiply-high: with m = ceil(2^32 / d),
// floor(n m / 2^32) = floor(n / d) for every n with n d < 2^32 (the error term
// n (m d - 2^32) / (d 2^32) stays below 1 / d).  The launcher fills `m` when
// every dividend of the launch obeys that bound and leaves 0 otherwise; the
// kernels then fall back to the hardware-less division sequence.  A tile
// switch of the persistent kernels decodes two tiles with five divisions each,
// in every wave: ~200 scalar instructions apiece as division sequences, a
// dozen this way.
struct FastDiv {
  uint32_t d, m;
};
__host__ __device__ inline FastDiv make_fast_div(uint32_t d, uint64_t max_dividend) {
  FastDiv f{d ? d : 1u, 0u};
  if (f.d > 1 && max_dividend * f.d < ((uint64_t)1 << 32)) f.m = (uint32_t)((((uint64_t)1 << 32) + f.d - 1) / f.d);
  return f;
}
__host__ __device__ inline uint32_t fast_div(uint32_t n, const FastDiv& f) {
  if (f.d == 1) return n;
  if (f.m) return (uint32_t)(((uint64_t)n * f.m) >> 32);
  return n / f.d;
}

// The divisors of a launch's tile decode.
struct TileDivs {
  FastDiv in_group;  // G * num_pid_n: tiles per group of G tile rows
  FastDiv group;     // G: rows of a full group
  FastDiv tail;      // num_pid_m % G: rows of the last, short group (1 when there is none)
};
__host__ __device__ inline TileDivs make_tile_divs(int num_pid_m, int num_pid_n, int G) {
  const uint64_t total = (uint64_t)num_pid_m * num_pid_n + 1;
  TileDivs t;
  t.in_group = make_fast_div((uint32_t)(G * num_pid_n), total);
  t.group = make_fast_div((uint32_t)G, total);
  t.tail = make_fast_div((uint32_t)(num_pid_m % G ? num_pid_m % G : 1), total);
  return t;
}
// tile_map with the launch's precomputed divisors: the same arithmetic.
__host__ __device__ inline TileCoord tile_map_fast(int tile_id, int num_pid_m, int num_pid_n, int G,
                                                   const TileDivs& dv) {
  const int group_id = (int)fast_div((uint32_t)tile_id, dv.in_group);
  const int first_pid_m = group_id * G;
  const int rem = num_pid_m - first_pid_m;
  const int in_group = tile_id - group_id * (G * num_pid_n);
  TileCoord t;
  if (rem < G) {  // the last group, num_pid_m % G rows
    t.pid_n = (int)fast_div((uint32_t)in_group, dv.tail);
    t.pid_m = first_pid_m + in_group - t.pid_n * rem;
  } else {
    t.pid_n = (int)fast_div((uint32_t)in_group, dv.group);
    t.pid_m = first_pid_m + in_group - t.pid_n * G;
  }
  return t;
}

// (pid_m, pid_n) -> tile_id: the inverse of tile_map.
__host__ __device__ inline int tile_id_of(int pid_m, int pid_n, int num_pid_m, int num_pid_n, int G) {
  const int group_id = pid_m / G;
  const int first_pid_m = group_id * G;
  const int rem = num_pid_m - first_pid_m;
  const int group_size_m = rem < G ? rem : G;
  return group_id * G * num_pid_n + pid_n * group_size_m + (pid_m - first_pid_m);
}

// program-id remap that keeps consecutive tiles on one XCD;
// gemm_one_shot_all_reduce.py:135-136.
__host__ __device__ inline int xcd_remap(int pid, int num_sms, int num_xcds) {
  if (num_xcds != 1) pid = (pid % num_xcds) * (num_sms / num_xcds) + (pid / num_xcds);
  return pid;
}

// Entry r of the table of heap bases through a scalar load.  The table does
// not change while a kernel runs, and a scalar load, unlike a vector load of
// the same word, does not make the wave wait for its outstanding vector
// loads and stores before the value can be used.
__device__ inline uint64_t heap_base_at(const uint64_t* heap_bases, int r) {
  return ((const __attribute__((address_space(4))) uint64_t*)heap_bases)[r];
}

// A 64-bit value every lane of the wave agrees on, as scalar registers.
__device__ inline uint64_t uniform_u64(uint64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// Pointer rebasing between symmetric heaps; iris/iris.py:317-339.
template <typename P>
__device__ inline IRIS_GLOBAL P* translate(P* ptr, uint64_t cur_base, uint64_t target_base) {
  const uint64_t off = reinterpret_cast<uint64_t>(ptr) - cur_base;
  return (IRIS_GLOBAL P*)(target_base + off);
}

// ---- element conversions ---------------------------------------------------

__device__ inline unsigned short f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(unsigned short, (__bf16)f);  // round-to-nearest-even
}
__device__ inline float bf16_bits_to_f32(unsigned short h) {
  return __builtin_bit_cast(float, ((unsigned int)h) << 16);
}
__device__ inline unsigned short f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;  // v_cvt_f16_f32, round-to-nearest-even
  return __builtin_bit_cast(unsigned short, h);
}
__device__ inline float f16_bits_to_f32(unsigned short h) {
  return (float)__builtin_bit_cast(_Float16, h);
}

// to16<DT>(f): fp32 -> 16-bit pattern of element type DT (IRIS_DTYPE_*),
// round-to-nearest-even (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32 on gfx950)
template <int DT>
__device__ inline unsigned int pack2(float lo, float hi) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  if constexpr (DT == IRIS_DTYPE_BF16)
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2));
  else
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, f16x2));
}
template <int DT>
__device__ inline unsigned short to16(float f) {
  return (unsigned short)(pack2<DT>(f, 0.f) & 0xFFFFu);
}
template <int DT>
__device__ inline float from16(unsigned short h) {
  if constexpr (DT == IRIS_DTYPE_BF16)
    return bf16_bits_to_f32(h);
  else
    return f16_bits_to_f32(h);
}

// ---- 16-byte strips through buffer descriptors ------------------------------

// VE<DT>: elements in one 16-byte load of type DT.  A lane always moves 16
// bytes per rank, so that one wave-wide load covers 1 KiB of contiguous
// memory; wider per-lane strips (two loads a lane) measured ~20% slower.
template <int DT>
struct Vec {
  static constexpr int ES = (DT == IRIS_DTYPE_F32) ? 4 : 2;
  static constexpr int N = 16 / ES;
};

// Loads and stores go through buffer descriptors that span exactly one tile:
// the hardware bounds check returns zeros for (and drops stores of) strips
// below a ragged tile's last row, so the inner loop has no branches, and a
// lane that owns no strip parks its offset at DEAD_OFFSET.
constexpr uint32_t DEAD_OFFSET = 0x80000000u;
// cache-policy bits of the buffer instructions
constexpr int AUX_SC0 = 1, AUX_NT = 2, AUX_SC1 = 16;

__device__ inline __amdgpu_buffer_rsrc_t tile_rsrc(const IRIS_GLOBAL char* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)bytes, 0x00020000);
}

template <int DT, int AUX>
__device__ inline void load_vec(__amdgpu_buffer_rsrc_t rs, uint32_t off, float (&v)[Vec<DT>::N]) {
  const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)off, 0, AUX);
  if constexpr (DT == IRIS_DTYPE_F32) {
    // cast the whole vector: a bit_cast of one element reads element 0
    const f32x4 f = __builtin_bit_cast(f32x4, x);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = f[e];
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = from16<DT>((unsigned short)(x[e / 2] >> (16 * (e & 1))));
  }
}

// store NE fp32 values as elements of type DT
template <int DT, int NE, int AUX>
__device__ inline void store_vec(__amdgpu_buffer_rsrc_t rs, uint32_t off, const float (&v)[NE]) {
  constexpr int aux = AUX;
  if constexpr (DT == IRIS_DTYPE_F32) {
#pragma unroll
    for (int h = 0; h < NE / 4; ++h) {
      const f32x4 f = {v[4 * h], v[4 * h + 1], v[4 * h + 2], v[4 * h + 3]};
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, f), rs, (int)(off + 16 * h), 0, aux);
    }
  } else if constexpr (NE == 4) {
    const u32x2 y = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3])};
    __builtin_amdgcn_raw_buffer_store_b64(y, rs, (int)off, 0, aux);
  } else {
    const u32x4 y = {pack2<DT>(v[0], v[1]), pack2<DT>(v[2], v[3]), pack2<DT>(v[4], v[5]), pack2<DT>(v[6], v[7])};
    __builtin_amdgcn_raw_buffer_store_b128(y, rs, (int)off, 0, aux);
  }
}

// Bare workgroup barrier.  __syncthreads() (and any LDS release fence) also
// drains the vector-memory counter, because LDS-DMA loads count as LDS
// writes; that would stall on the slabs that are meant to stay in flight
// across the barrier.  The caller waits explicitly for the one slab it needs.
// The empty asm statements keep the compiler from moving memory accesses
// across the barrier.
__device__ inline void block_barrier_raw() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__host__ __device__ inline int dtype_size(int dt) { return dt == IRIS_DTYPE_F32 ? 4 : 2; }

// CU count of the current device, asked of the runtime once per device
// (launchers consult it on every call); 256 when it cannot be read.
int current_cu_count();

// ---- scoped atomics on flags -----------------------------------------------

__device__ inline void flag_add_release(IRIS_GLOBAL int32_t* p, int v, bool sys) {
  if (sys)
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  else
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ inline void flag_add_relaxed(IRIS_GLOBAL int32_t* p, int v, bool sys) {
  if (sys)
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  else
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Store that is written through to the coherence point of the agent (or of
// the system): nothing stays dirty in this XCD's L2.
template <typename T>
__device__ inline void store_through(IRIS_GLOBAL T* p, T v, bool sys) {
  if (sys)
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  else
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// CAS(expected -> desired) with acquire; returns the old value
// (tl.atomic_cas semantics, iris/iris.py:476-497).
__device__ inline int flag_cas_acquire(IRIS_GLOBAL int32_t* p, int expected, int desired, bool sys) {
  int e = expected;
  if (sys)
    __hip_atomic_compare_exchange_strong(p, &e, desired, __ATOMIC_ACQUIRE, __ATOMIC_ACQUIRE,
                                         __HIP_MEMORY_SCOPE_SYSTEM);
  else
    __hip_atomic_compare_exchange_strong(p, &e, desired, __ATOMIC_ACQUIRE, __ATOMIC_ACQUIRE,
                                         __HIP_MEMORY_SCOPE_AGENT);
  return e;
}

// Bounded wait for a tile's flag: spins on CAS(ws-1 -> 0) until the old value
// reaches ws-1 (gemm_one_shot_all_reduce.py:220-234) or `timeout` ticks of
// the 100 MHz wall clock have passed.  Returns true on success.  Every caller
// reaches an exit: a wait that gives up records IRIS_STATUS_SPIN_TIMEOUT.
__device__ inline bool wait_tile_flag(IRIS_GLOBAL int32_t* flag, int ws, bool sys, uint64_t timeout,
                                      uint32_t* status) {
  if (ws <= 1) return true;  // `while result < ws-1` never runs for ws == 1
  const uint64_t t0 = wall_clock64();
  for (;;) {
    const int old = flag_cas_acquire(flag, ws - 1, 0, sys);
    if (old >= ws - 1) return true;
    if (wall_clock64() - t0 > timeout) {
      if (status) atomicMax(status, (uint32_t)IRIS_STATUS_SPIN_TIMEOUT);
      return false;
    }
    __builtin_amdgcn_s_sleep(8);
  }
}

// Bounded wait until a tile's flag has reached `need`, without consuming it.
// Returns whether it has; a wait that gives up records IRIS_STATUS_SPIN_TIMEOUT.
// `mask` selects the bits of the flag that count.
__device__ inline bool wait_tile_ready(IRIS_GLOBAL int32_t* flag, int need, bool sys, uint64_t timeout,
                                       uint32_t* status, int mask = -1) {
  const uint64_t t0 = wall_clock64();
  for (;;) {
    const int v = sys ? __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM)
                      : __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((v & mask) >= need) return true;
    if (wall_clock64() - t0 > timeout) {
      if (status) atomicMax(status, (uint32_t)IRIS_STATUS_SPIN_TIMEOUT);
      return false;
    }
    __builtin_amdgcn_s_sleep(8);
  }
}

}  // namespace iris_amd
