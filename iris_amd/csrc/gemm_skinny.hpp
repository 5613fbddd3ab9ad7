// Shard GEMM for at most 16 rows of A (decode-time batches): C[M,N] = A[M,K] B[K,N]
// with the store epilogues of the persistent kernel (gemm_all_scatter.py:209-251,
// gemm_one_shot_all_reduce.py:197-218).
//
// With so few rows the product is a stream over B: every byte of B is used
// once, the matrix cores idle, and what matters is how many bytes a CU has in
// flight.  So nothing goes through LDS: a workgroup of eight waves owns 16
// columns of C, its waves share the K range out in blocks of 64, and a lane
// fetches its MFMA operands straight into registers, 32 contiguous bytes of a
// row of B (and of A) per block, every fetch of a wave issued before the
// first MFMA.  The eight partial 16x16 accumulators meet in LDS; wave w then
// stores the sum on destination rank w, w+8, ...
//
// A logical tile (BLOCK_SIZE_M x BLOCK_SIZE_N, one flag) spans several such
// workgroups.  They count their arrivals in locks[tile_id]; the last one to
// arrive re-arms the counter and publishes the tile's flag.
#pragma once

#include "gemm_registry.hpp"

namespace iris_amd {

constexpr int SKINNY_ROWS = 16;    // rows of A a launch can take
constexpr int SKINNY_COLS = 16;    // columns of C per workgroup
constexpr int SKINNY_WAVES = 8;
constexpr int SKINNY_THREADS = SKINNY_WAVES * 64;

// UN: K blocks (64 k each) whose fetches a wave has in flight together.
template <int DT, int OP, int ODT, int UN>
__global__ __launch_bounds__(SKINNY_THREADS) __attribute__((amdgpu_waves_per_eu(2, UN == 8 ? 2 : UN == 4 ? 4 : 8))) void
gemm_skinny_kernel(const GemmKArgs p) {
  static_assert(OP == OP_STORE16 || OP == OP_STORE32, "store epilogues only");
  using vec8 = typename Mfma<DT>::vec8;
  __shared__ f32x4 red[SKINNY_WAVES][64];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int lr = lane & 15, lq = lane >> 4;
  const int n0 = blockIdx.x * SKINNY_COLS;

  // Rows past the edge of either operand lie past the end of its buffer
  // descriptor and read as zero; chunks past K are parked out of range.
  const int rows_b = min(SKINNY_COLS, p.N - n0);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.b + (int64_t)n0 * p.sbn * 2), 0, (int)((((int64_t)rows_b - 1) * p.sbn + p.K) * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      (void*)p.a, 0, (int)((((int64_t)p.M - 1) * p.sam + p.K) * 2), 0x00020000);
  // Lane l holds row l%16 of its operand.  In K block kb, MFMA h (0, 1) takes
  // k = kb*64 + (l/16)*16 + h*8 .. +7 at MFMA position (l/16)*8 .. +7: the same
  // permutation of k for both operands, so the products pair up as they
  // should, and the two fetches of a lane are 32 contiguous bytes.
  const uint32_t ob = (uint32_t)(((int64_t)lr * p.sbn + lq * 16) * 2);
  const uint32_t oa = (uint32_t)(((int64_t)lr * p.sam + lq * 16) * 2);
  const int nb = (p.K + 63) / 64;

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int b0 = wave; b0 < nb; b0 += SKINNY_WAVES * UN) {
    vec8 fb[UN][2], fa[UN][2];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int kb = b0 + SKINNY_WAVES * u;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bool ok = kb < nb && kb * 64 + lq * 16 + h * 8 < p.K;
        const uint32_t koff = (uint32_t)(kb * 128 + h * 16);
        fb[u][h] = __builtin_bit_cast(
            vec8, __builtin_amdgcn_raw_buffer_load_b128(rb, ok ? (int)(ob + koff) : (int)0x80000000, 0, 0));
        fa[u][h] = __builtin_bit_cast(
            vec8, __builtin_amdgcn_raw_buffer_load_b128(ra, ok ? (int)(oa + koff) : (int)0x80000000, 0, 0));
      }
    }
    // every fetch is on its way before the first product waits for one
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) acc = Mfma<DT>::run(fb[u][h], fa[u][h], acc);
  }

  // acc: row m = l%16 of C, columns n0 + 4*(l/16) .. +3 (operands swapped, as
  // in the persistent kernel)
  red[wave][lane] = acc;
  __syncthreads();

  const int r_begin = p.dest_all ? 0 : p.cur_rank;
  const int r_end = p.dest_all ? p.ws : p.cur_rank + 1;
  const int m = lr, n = n0 + lq * 4;
  if (r_begin + wave < r_end && m < p.M && n < p.N) {
    f32x4 s = red[0][lane];
#pragma unroll
    for (int w = 1; w < SKINNY_WAVES; ++w) s += red[w][lane];  // wave order: the sum does not depend on timing
    constexpr int ES = OP == OP_STORE32 ? 4 : 2;
    const bool whole = p.vec_out && n + 4 <= p.N;
    for (int r = r_begin + wave; r < r_end; r += SKINNY_WAVES) {
      IRIS_GLOBAL char* dst = rank_ptr(p, p.out, r);
      if (whole) {
        IRIS_GLOBAL unsigned int* d = (IRIS_GLOBAL unsigned int*)(dst + ((int64_t)m * p.som + n) * ES);
        if constexpr (OP == OP_STORE32) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float f = s[e];  // (a bit cast of the element itself reads element 0)
            store_through(d + e, __builtin_bit_cast(unsigned int, f), p.sys != 0);
          }
        } else {
          store_through(d, pack2<ODT>(s[0], s[1]), p.sys != 0);
          store_through(d + 1, pack2<ODT>(s[2], s[3]), p.sys != 0);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (n + e >= p.N) continue;
          IRIS_GLOBAL char* d = dst + ((int64_t)m * p.som + (int64_t)(n + e) * p.son) * ES;
          const float f = s[e];
          if constexpr (OP == OP_STORE32)
            store_through((IRIS_GLOBAL unsigned int*)d, __builtin_bit_cast(unsigned int, f), p.sys != 0);
          else
            store_through((IRIS_GLOBAL unsigned short*)d, to16<ODT>(s[e]), p.sys != 0);
        }
      }
    }
  }
  if (p.flag_mode == 0) return;

  // The stores were write-through at the flags' scope: once every wave has
  // seen its own complete, the group's part of the tile is visible there.
  IRIS_WAIT_VMCNT(0);
  __syncthreads();
  if (tid == 0) {
    const int pid_n = n0 / p.BN;
    const int tile_id = tile_id_of(0, pid_n, p.num_pid_m, p.num_pid_n, p.G);
    const int cols = min(p.N, (pid_n + 1) * p.BN) - pid_n * p.BN;
    const int parts = (cols + SKINNY_COLS - 1) / SKINNY_COLS;
    bool last = true;
    if (parts > 1) {
      IRIS_GLOBAL int32_t* cnt = (IRIS_GLOBAL int32_t*)(p.locks + tile_id);
      last = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == parts - 1;
      if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
    }
    if (last) publish_tile(p, tile_id);
  }
}

// The kernel for (operand type, store op, blocks in flight), or null.
GemmKernelFn gemm_skinny_kernel_for(int dt, int op, int un);

}  // namespace iris_amd
