// Measurement aid: what the matrix cores sustain on their own.
//
// A register-only loop of v_mfma_f32_16x16x32 (the instruction the shard GEMM
// uses) on operands taken from the caller's buffer: no LDS, no memory traffic
// inside the loop.  On a power-limited board the rate depends on how much the
// operand bits toggle, so the figure for random operands, not the data-sheet
// peak, is what a GEMM kernel on the same data can approach.
#include <hip/hip_runtime.h>

#include "common.hpp"

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

}  // namespace iris_amd

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
