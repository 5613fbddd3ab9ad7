// Shard-GEMM kernel instantiations: fp32 operands, fp32 output (store and atomic-add epilogues).
#include "gemm_registry.hpp"

namespace iris_amd {

IRIS_GEMM_F32_VARIANTS(IRIS_GEMM_F32_INSTANTIATE, OP_STORE32)
IRIS_GEMM_F32_VARIANTS(IRIS_GEMM_F32_INSTANTIATE_FUSED, OP_STORE32)
IRIS_GEMM_F32_VARIANTS(IRIS_GEMM_F32_INSTANTIATE, OP_ATOMIC32)

static const GemmKernelEntry k_store[] = {IRIS_GEMM_F32_VARIANTS(IRIS_GEMM_F32_ENTRY, OP_STORE32)};
static const GemmKernelEntry k_atomic[] = {IRIS_GEMM_F32_VARIANTS(IRIS_GEMM_F32_ENTRY, OP_ATOMIC32)};

const GemmKernelEntry* gemm_entries_f32_store32(int* count) {
  *count = (int)(sizeof(k_store) / sizeof(k_store[0]));
  return k_store;
}

const GemmKernelEntry* gemm_entries_f32_atomic32(int* count) {
  *count = (int)(sizeof(k_atomic) / sizeof(k_atomic[0]));
  return k_atomic;
}

}  // namespace iris_amd
