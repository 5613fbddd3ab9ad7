// Shard-GEMM kernel instantiations: f16 operands, store16 epilogue.
#include "gemm_registry.hpp"

namespace iris_amd {

IRIS_GEMM_VARIANTS(IRIS_GEMM_INSTANTIATE, IRIS_DTYPE_F16, OP_STORE16)
IRIS_GEMM_VARIANTS(IRIS_GEMM_INSTANTIATE_FUSED, IRIS_DTYPE_F16, OP_STORE16)
IRIS_GEMM_INSTANTIATE_MERGED(IRIS_DTYPE_F16, OP_STORE16)

static const GemmKernelEntry k_entries[] = {IRIS_GEMM_VARIANTS(IRIS_GEMM_ENTRY, IRIS_DTYPE_F16, OP_STORE16)};

const GemmKernelEntry* gemm_entries_f16_store16(int* count) {
  *count = (int)(sizeof(k_entries) / sizeof(k_entries[0]));
  return k_entries;
}

}  // namespace iris_amd
