// Shard GEMM for a few rows of A (decode-time batches, 16 or 32 rows a workgroup): C[M,N] = A[M,K] B[K,N]
// with the epilogues of the persistent kernel (gemm_all_scatter.py:209-251,
// gemm_atomics_all_reduce.py:236-248, gemm_one_shot_all_reduce.py:197-218).
//
// With so few rows the product is a stream over B: every byte of B is used
// once, the matrix cores idle, and what matters is how many bytes a CU has in
// flight and how many bytes each cache-line access of its L1 brings.  A
// workgroup of eight waves owns 16 columns of C and its waves share the K
// range out in blocks of 64.  Every fetch of a wave is issued before its
// first MFMA:
//   * B, the stream, comes in with `buffer_load ... lds`, one instruction per
//     8 rows x 128 bytes (whole cache lines: twice the bytes per line access
//     of a fetch in MFMA operand layout, 16 rows x 64 bytes), into a region of
//     LDS private to the wave, 16-byte chunks XOR-ed by the row so that the
//     operand reads are conflict-free;
//   * A, rows that every workgroup reads and L2 holds, goes into registers:
//     straight in operand layout when there are very few of them, otherwise
//     lanes along a row like B, each block passing through 2 KiB of LDS on
//     its way to the MFMAs (a load in operand layout has neighbouring lanes
//     in different rows and merges nothing).
// The waves' partial 16x16 accumulators meet in LDS; wave w then stores the
// sum on destination rank w, w+8, ...
//
// A logical tile (BLOCK_SIZE_M x BLOCK_SIZE_N, one flag; BLOCK_SIZE_M covers
// every row) spans several such workgroups.  They count their arrivals in locks[tile_id]; the last one to
// arrive re-arms the counter and publishes the tile's flag.
#pragma once

#include "gemm_registry.hpp"

namespace iris_amd {

constexpr int SKINNY_ROWS = 16;    // rows of A per block (a workgroup takes RB blocks of them, blockIdx.y counts its share)
constexpr int SKINNY_MAX_ROWS = 32;  // rows of A a launch of single blocks can take: beyond, B is re-read too often
constexpr int SKINNY_COLS = 16;    // columns of C per block (a workgroup takes CB blocks of them)
constexpr int SKINNY_MID_MAX_ROWS = 64;   // rows of A a launch of 32-row workgroups can take ...
constexpr int SKINNY_MID_MIN_K = 2048;    // ... when K is at least this long
constexpr int SKINNY_WAVES = 8;
constexpr int SKINNY_THREADS = SKINNY_WAVES * 64;
constexpr int SKINNY_BLOCK_BYTES = 2048;                  // 16 rows of A or B x 64 k
// LDS of a workgroup of RB x CB blocks: a block of A per wave and row block (the waves' partial accumulators
// take its place once the K range is done), then every wave's UN K-blocks of B
constexpr int skinny_red_bytes(int rb, int cb) { return SKINNY_WAVES * rb * cb * 64 * 16; }
constexpr int skinny_a_bytes(int rb, int cb) {
  return SKINNY_WAVES * rb * SKINNY_BLOCK_BYTES > skinny_red_bytes(rb, cb) ? SKINNY_WAVES * rb * SKINNY_BLOCK_BYTES
                                                                            : skinny_red_bytes(rb, cb);
}
constexpr int skinny_lds_bytes(int un, int rb = 1, int cb = 1) {
  return skinny_a_bytes(rb, cb) + SKINNY_WAVES * un * cb * SKINNY_BLOCK_BYTES;
}

// From this many rows and this long a K on, A is fetched lanes-along-a-row
// and passed through LDS.  Below, a load in operand layout only touches the
// lanes of the rows that exist and is the cheaper way: [M,4096] x [4096,1376]
// 6.8 against 7.3 us at one row, 7.4 both ways at four, 8.2 against 7.5 at
// eight, 9.8 against 7.8 at sixteen; with K = 1376 (and 256 workgroups) the
// pass through LDS never pays (16 rows: 6.6 against 6.7 us).
constexpr int SKINNY_A_VIA_LDS_ROWS = 5;
constexpr int SKINNY_A_VIA_LDS_K = 2048;

// UN: K blocks (64 k each) whose fetches a wave has in flight together.
// A_LDS: how A reaches the MFMAs (see below).
// RB x CB: blocks of 16 rows x 16 columns a workgroup computes (1 x 1 for up
// to 32 rows; 2 x 1 up to 64 rows of a long K, always with A_LDS).
template <int DT, int OP, int ODT, int UN, bool A_LDS, int RB = 1, int CB = 1>
__global__ __launch_bounds__(SKINNY_THREADS) __attribute__((amdgpu_waves_per_eu(2, UN * CB >= 8 ? 2 : UN * CB >= 4 ? 4 : 8))) void
gemm_skinny_kernel(const GemmKArgs p) {
  constexpr bool ATOMIC = OP == OP_ATOMIC32 || OP == OP_ATOMIC16;
  constexpr bool F32 = OP == OP_STORE32 || OP == OP_ATOMIC32;
  constexpr int NB = RB * CB;
  static_assert(A_LDS || NB == 1, "several blocks a workgroup: A goes through LDS");
  static_assert(NB == 1 || NB == 2 || NB == 4, "blocks per workgroup");
  using vec8 = typename Mfma<DT>::vec8;
  extern __shared__ __attribute__((aligned(1024))) char skinny_lds[];
  IRIS_LDS char* lds = (IRIS_LDS char*)skinny_lds;
  // each wave's blocks of A ([SKINNY_WAVES][NB][64] partial accumulators at the end), then each wave's UN x CB blocks of B
  IRIS_LDS f32x4* red = (IRIS_LDS f32x4*)lds;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int lr = lane & 15, lq = lane >> 4;
  const int n0 = blockIdx.x * (SKINNY_COLS * CB);
  const int m0 = blockIdx.y * (SKINNY_ROWS * RB);
  IRIS_LDS char* wb = lds + skinny_a_bytes(RB, CB) + wave * (UN * CB * SKINNY_BLOCK_BYTES);
  IRIS_LDS char* wa = lds + wave * (RB * SKINNY_BLOCK_BYTES);

  // Rows past the edge of either operand lie past the end of its buffer
  // descriptor and read as zero; chunks past K are parked out of range.
  const int rows_b = min(SKINNY_COLS * CB, p.N - n0);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.b + (int64_t)n0 * p.sbn * 2), 0, (int)((((int64_t)rows_b - 1) * p.sbn + p.K) * 2), 0x00020000);
  const int rows_a = min(SKINNY_ROWS * RB, p.M - m0);
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.a + (int64_t)m0 * p.sam * 2), 0, (int)((((int64_t)rows_a - 1) * p.sam + p.K) * 2), 0x00020000);
  // B: lane l of fetch j of a block brings row 8j + l/8 and lands at byte
  // l*16 of the fetch's 1 KiB, i.e. at physical chunk l%8 of that row; the
  // chunk of the row it must bring there is (l%8) ^ (row/2 % 8).
  const int brow = lane >> 3;  // + 8j
  const int bchunk = (lane & 7) ^ ((brow >> 1) & 7);  // rows 8j + .. : (row/2)%8 = 4j + brow/2, and 4j flips bit 2
  // A_LDS: A comes in the same way, lanes along a row, but into registers: a
  // load in operand layout (lane l holds row l%16) has neighbouring lanes in
  // different rows, nothing for the memory pipeline to merge, and with 16 rows
  // costs eight times what the same bytes of B cost (2.5 against 0.3 us).  A
  // block of A then goes through a 2 KiB region of the wave, laid out like a
  // block of B, on its way to the MFMAs.  With very few rows the load in
  // operand layout is the cheaper one (!A_LDS).
  // The operand reads: lane l holds row l%16.  In K block kb, MFMA h (0, 1)
  // takes k = kb*64 + (l/16)*16 + h*8 .. +7 at MFMA position (l/16)*8 .. +7:
  // the same permutation of k for both operands.
  const uint32_t oa = (uint32_t)(((int64_t)lr * p.sam + lq * 16) * 2);
  const int nb = (p.K + 63) / 64;

  f32x4 acc[RB][CB];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int c = 0; c < CB; ++c) acc[i][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int b0 = wave; b0 < nb; b0 += SKINNY_WAVES * UN) {
    u32x4 va[UN][RB][2];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int kb = b0 + SKINNY_WAVES * u;
#pragma unroll
      for (int c = 0; c < CB; ++c)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int ch = bchunk ^ (j << 2);
          const bool ok = kb < nb && kb * 64 + ch * 8 < p.K;
          const uint32_t off = (uint32_t)(((int64_t)(c * 16 + brow + 8 * j) * p.sbn) * 2 + kb * 128 + ch * 16);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              rb, (IRIS_LDS void*)(wb + (u * CB + c) * SKINNY_BLOCK_BYTES + j * 1024), 16,
              ok ? (int)off : (int)0x80000000, 0, 0, 0);
        }
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if constexpr (A_LDS) {
            const int ch = bchunk ^ (j << 2);
            const bool ok = kb < nb && kb * 64 + ch * 8 < p.K;
            const uint32_t off = (uint32_t)(((int64_t)(i * 16 + brow + 8 * j) * p.sam) * 2 + kb * 128 + ch * 16);
            va[u][i][j] = __builtin_amdgcn_raw_buffer_load_b128(ra, ok ? (int)off : (int)0x80000000, 0, 0);
          } else {  // j is the MFMA (h) the 16 bytes are for
            const bool ok = kb < nb && kb * 64 + lq * 16 + j * 8 < p.K;
            va[u][i][j] =
                __builtin_amdgcn_raw_buffer_load_b128(ra, ok ? (int)(oa + kb * 128 + j * 16) : (int)0x80000000, 0, 0);
          }
        }
    }
    // every fetch is on its way; B has landed in this wave's own region once
    // the wave's counter says so (nobody else reads or writes it)
    IRIS_WAIT_VMCNT(0);
    asm volatile("" ::: "memory");
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      // (the wave's LDS operations execute in order: these writes land after
      // the previous block's reads and before this block's)
      if constexpr (A_LDS) {
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            *reinterpret_cast<IRIS_LDS u32x4*>(wa + i * SKINNY_BLOCK_BYTES + j * 1024 + lane * 16) = va[u][i][j];
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int pc = (lq * 2 + h) ^ ((lr >> 1) & 7);
        vec8 fb[CB];
#pragma unroll
        for (int c = 0; c < CB; ++c)
          fb[c] = *reinterpret_cast<const IRIS_LDS vec8*>(wb + (u * CB + c) * SKINNY_BLOCK_BYTES + lr * 128 + pc * 16);
#pragma unroll
        for (int i = 0; i < RB; ++i) {
          vec8 fa;
          if constexpr (A_LDS)
            fa = *reinterpret_cast<const IRIS_LDS vec8*>(wa + i * SKINNY_BLOCK_BYTES + lr * 128 + pc * 16);
          else
            fa = __builtin_bit_cast(vec8, va[u][i][h]);
#pragma unroll
          for (int c = 0; c < CB; ++c) acc[i][c] = Mfma<DT>::run(fb[c], fa, acc[i][c]);
        }
      }
    }
    // the reads above have returned before the next round overwrites the region
    IRIS_WAIT_LGKMCNT0();
    asm volatile("" ::: "memory");
  }

  // acc[i][c]: row m = i*16 + l%16 of the workgroup's rows, columns c*16 + 4*(l/16) .. +3 (operands swapped, as
  // in the persistent kernel).  The waves' partial sums meet in LDS, [wave][block][lane].
  if constexpr (A_LDS) __syncthreads();  // every wave is done with its blocks of A: the region becomes `red`
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int c = 0; c < CB; ++c) red[(wave * NB + i * CB + c) * 64 + lane] = acc[i][c];
  __syncthreads();
  if constexpr (NB > 1) {
    // With several blocks every destination's wave would add up all of them:
    // first each block is summed once, in wave order, by the 8 / NB waves that
    // share it (a part of the lanes each), and left in the first wave's place.
    constexpr int WPB = SKINNY_WAVES / NB, LPW = 64 / WPB;  // waves per block, lanes of a block per wave
    const int blk = wave / WPB, l0 = (wave % WPB) * LPW;
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    const bool mine = lane >= l0 && lane < l0 + LPW;
    if (mine) {
      s = red[blk * 64 + lane];
#pragma unroll
      for (int w = 1; w < SKINNY_WAVES; ++w) s += red[(w * NB + blk) * 64 + lane];  // wave order
    }
    __syncthreads();  // all partial sums have been read
    if (mine) red[blk * 64 + lane] = s;
    __syncthreads();
  }

  const int r_begin = p.dest_all ? 0 : p.cur_rank;
  const int r_end = p.dest_all ? p.ws : p.cur_rank + 1;
  if (r_begin + wave < r_end) {
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        const int m = m0 + i * 16 + lr, n = n0 + c * 16 + lq * 4;
        if (m >= p.M || n >= p.N) continue;
        f32x4 s = red[(i * CB + c) * 64 + lane];
        if constexpr (NB == 1) {
#pragma unroll
          for (int w = 1; w < SKINNY_WAVES; ++w) s += red[w * 64 + lane];  // wave order: the sum does not depend on timing
        }
        constexpr int ES = F32 ? 4 : 2;
        const bool whole = p.vec_out && n + 4 <= p.N;
        for (int r = r_begin + wave; r < r_end; r += SKINNY_WAVES) {
          IRIS_GLOBAL char* dst = rank_ptr(p, p.out, r);
          if constexpr (ATOMIC) {
            // 08: add into the destination (gemm_atomics_all_reduce.py:236-248)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if (n + e >= p.N) continue;
              IRIS_GLOBAL char* d = dst + ((int64_t)m * p.som + (int64_t)(n + e) * p.son) * ES;
              const float f = s[e];
              if constexpr (OP == OP_ATOMIC32) {
                __hip_atomic_fetch_add((IRIS_GLOBAL float*)d, f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              } else if (whole && (e & 1) == 0) {
                atomic_add16_pair<ODT>((IRIS_GLOBAL unsigned int*)d, pack2<ODT>(s[e], s[e + 1]));
                ++e;  // the pair took the next column too
              } else {
                atomic_add16_cas<ODT>((IRIS_GLOBAL unsigned short*)d, from16<ODT>(to16<ODT>(f)));
              }
            }
          } else if (whole) {
            IRIS_GLOBAL unsigned int* d = (IRIS_GLOBAL unsigned int*)(dst + ((int64_t)m * p.som + n) * ES);
            if constexpr (F32) {
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
              if constexpr (F32)
                store_through((IRIS_GLOBAL unsigned int*)d, __builtin_bit_cast(unsigned int, f), p.sys != 0);
              else
                store_through((IRIS_GLOBAL unsigned short*)d, to16<ODT>(s[e]), p.sys != 0);
            }
          }
        }
      }
  }
  if (p.flag_mode == 0) return;

  // The stores were write-through at the flags' scope: once every wave has
  // seen its own complete, the group's part of the tile is visible there.
  IRIS_WAIT_VMCNT(0);
  __syncthreads();
  if (wave == 0) {
    const int pid_n = n0 / p.BN;
    const int tile_id = tile_id_of(0, pid_n, p.num_pid_m, p.num_pid_n, p.G);
    const int cols = min(p.N, (pid_n + 1) * p.BN) - pid_n * p.BN;
    const int parts = ((cols + SKINNY_COLS * CB - 1) / (SKINNY_COLS * CB)) * gridDim.y;
    int last = 1;
    if (parts > 1) {
      IRIS_GLOBAL int32_t* cnt = (IRIS_GLOBAL int32_t*)(p.locks + tile_id);
      if (lane == 0) {
        last = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == parts - 1;
        if (last) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
      }
      last = __builtin_amdgcn_readfirstlane(last);
    }
    if (last) publish_tile(p, tile_id, lane);
  }
}

// The kernel for (operand type, store op, K blocks in flight, A through LDS, blocks of rows and of columns a
// workgroup), or null.
GemmKernelFn gemm_skinny_kernel_for(int dt, int op, int un, bool a_lds, int rb = 1, int cb = 1);

}  // namespace iris_amd
