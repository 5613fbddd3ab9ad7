// Measurement aid: what the matrix cores sustain on their own.
//
// A register-only loop of v_mfma_f32_16x16x32 (the instruction the shard GEMM
// uses) on operands taken from the caller's buffer: no LDS, no memory traffic
// inside the loop.  On a power-limited board the rate depends on how much the
// operand bits toggle, so the figure for random operands, not the data-sheet
// peak, is what a GEMM kernel on the same data can approach.
#include <hip/hip_runtime.h>

#include "../../../include/iris_amd_testing.h"
#include "../common.hpp"

namespace iris_amd {

template <int DT>
__global__ __launch_bounds__(512) void mfma_probe_kernel(const u32x4* operands, float* sink, int iters) {
  using V = typename std::conditional<DT == IRIS_DTYPE_BF16, bf16x8, f16x8>::type;
  // four A and four B fragments per lane, so that operands change from one MFMA to the next
  V a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = __builtin_bit_cast(V, operands[(threadIdx.x * 8 + i) & 4095]);
    b[i] = __builtin_bit_cast(V, operands[(threadIdx.x * 8 + 4 + i) & 4095]);
  }
  f32x4 acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if constexpr (DT == IRIS_DTYPE_BF16)
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j % 4], b[j / 4], acc[j], 0, 0, 0);
      else
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j % 4], b[j / 4], acc[j], 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
  sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Measurement aid: what a tile's worth of output stores costs next to the
// matrix cores, by how the stores are spread.  Every group of eight waves plays
// a GEMM program without its operand traffic: a "tile" is 16 K-steps of 64
// register-only MFMAs a wave (what a 256 x 256 x 1024 tile takes) and 16
// one-KiB stores a wave (its 128 KiB of bf16 output, whole lines, to a region
// of its own).  CHUNK stores are issued back to back, every CHUNK K-steps:
// 16 = the whole tile at once (an epilogue), 1 = one store a K-step, 0 = none.
// With `lockstep` the waves of a group meet at a barrier after every K-step,
// as the GEMM's waves do at a stage hand-over.
template <int CHUNK, int AUX>
__global__ __launch_bounds__(512) void store_probe_kernel(const u32x4* operands, float* sink, char* out,
                                                          unsigned long long out_bytes, int tiles, int lockstep) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x * 8 + i) & 4095]);
    b[i] = __builtin_bit_cast(bf16x8, operands[(threadIdx.x * 8 + 4 + i) & 4095]);
  }
  f32x4 acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const unsigned long long per_tile = (unsigned long long)gridDim.x * 8 * 16384;
  for (int t = 0; t < tiles; ++t) {
    // the wave's 16 KiB of this tile
    const unsigned long long base = (((unsigned long long)t * per_tile) % (out_bytes - per_tile + 1)) +
                                    ((unsigned long long)blockIdx.x * 8 + wave) * 16384;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)(out + base), 0, 16384, 0x00020000);
#pragma unroll
    for (int step = 0; step < 16; ++step) {
      if constexpr (CHUNK > 0) {
        if (step % CHUNK == 0) {
#pragma unroll
          for (int q = 0; q < CHUNK; ++q)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[(step + q) & 15]), rs,
                                                   (step + q) * 1024 + lane * 16, 0, AUX);
        }
      }
#pragma unroll
      for (int rep = 0; rep < 4; ++rep)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j % 4], b[j / 4], acc[j], 0, 0, 0);
      if (lockstep) __builtin_amdgcn_s_barrier();
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 16; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
  sink[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace iris_amd

extern "C" int iris_store_probe_launch(const void* operands, float* sink, void* out, uint64_t out_bytes, int32_t tiles,
                                       int32_t chunk, int32_t write_through, int32_t lockstep, int32_t num_groups,
                                       void* stream) {
  using namespace iris_amd;
  if (!operands || !sink || !out || tiles < 0 || num_groups <= 0) return hipErrorInvalidValue;
  if ((reinterpret_cast<uintptr_t>(operands) & 15) != 0 || (reinterpret_cast<uintptr_t>(out) & 15) != 0)
    return hipErrorInvalidValue;
  if (out_bytes < (uint64_t)num_groups * 8 * 16384) return hipErrorInvalidValue;  // one tile of every group
  void (*fn)(const u32x4*, float*, char*, unsigned long long, int, int) = nullptr;
  const bool wt = write_through != 0;
  switch (chunk) {
    case 0: fn = &store_probe_kernel<0, 0>; break;
    case 1: fn = wt ? &store_probe_kernel<1, AUX_SC1> : &store_probe_kernel<1, 0>; break;
    case 4: fn = wt ? &store_probe_kernel<4, AUX_SC1> : &store_probe_kernel<4, 0>; break;
    case 16: fn = wt ? &store_probe_kernel<16, AUX_SC1> : &store_probe_kernel<16, 0>; break;
    default: return hipErrorInvalidValue;
  }
  hipLaunchKernelGGL(fn, dim3(num_groups), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(operands), sink, static_cast<char*>(out),
                     (unsigned long long)out_bytes, tiles, lockstep);
  return hipGetLastError();
}

extern "C" int iris_mfma_probe_launch(const void* operands, float* sink, int32_t ab_dtype, int32_t iters,
                                      int32_t num_groups, void* stream) {
  if (!operands || !sink || iters < 0 || num_groups <= 0) return hipErrorInvalidValue;
  if ((reinterpret_cast<uintptr_t>(operands) & 15) != 0) return hipErrorInvalidValue;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (ab_dtype == IRIS_DTYPE_BF16)
    hipLaunchKernelGGL(iris_amd::mfma_probe_kernel<IRIS_DTYPE_BF16>, dim3(num_groups), dim3(512), 0, st,
                       static_cast<const iris_amd::u32x4*>(operands), sink, iters);
  else if (ab_dtype == IRIS_DTYPE_F16)
    hipLaunchKernelGGL(iris_amd::mfma_probe_kernel<IRIS_DTYPE_F16>, dim3(num_groups), dim3(512), 0, st,
                       static_cast<const iris_amd::u32x4*>(operands), sink, iters);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
