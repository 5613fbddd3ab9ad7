// Instantiations of the few-rows shard GEMM.
#include "gemm_skinny.hpp"

namespace iris_amd {

namespace {

template <int DT, int OP>
GemmKernelFn pick_un(int un, bool a_lds) {
  constexpr int ODT = (OP == OP_STORE32 || OP == OP_ATOMIC32) ? IRIS_DTYPE_F32 : DT;
  switch (un) {
    case 2: return a_lds ? &gemm_skinny_kernel<DT, OP, ODT, 2, true> : &gemm_skinny_kernel<DT, OP, ODT, 2, false>;
    case 4: return a_lds ? &gemm_skinny_kernel<DT, OP, ODT, 4, true> : &gemm_skinny_kernel<DT, OP, ODT, 4, false>;
    case 8: return a_lds ? &gemm_skinny_kernel<DT, OP, ODT, 8, true> : &gemm_skinny_kernel<DT, OP, ODT, 8, false>;
  }
  return nullptr;
}

}  // namespace

GemmKernelFn gemm_skinny_kernel_for(int dt, int op, int un, bool a_lds) {
  if (dt == IRIS_DTYPE_BF16) {
    if (op == OP_STORE16) return pick_un<IRIS_DTYPE_BF16, OP_STORE16>(un, a_lds);
    if (op == OP_STORE32) return pick_un<IRIS_DTYPE_BF16, OP_STORE32>(un, a_lds);
    if (op == OP_ATOMIC32) return pick_un<IRIS_DTYPE_BF16, OP_ATOMIC32>(un, a_lds);
    if (op == OP_ATOMIC16) return pick_un<IRIS_DTYPE_BF16, OP_ATOMIC16>(un, a_lds);
  } else if (dt == IRIS_DTYPE_F16) {
    if (op == OP_STORE16) return pick_un<IRIS_DTYPE_F16, OP_STORE16>(un, a_lds);
    if (op == OP_STORE32) return pick_un<IRIS_DTYPE_F16, OP_STORE32>(un, a_lds);
    if (op == OP_ATOMIC32) return pick_un<IRIS_DTYPE_F16, OP_ATOMIC32>(un, a_lds);
    if (op == OP_ATOMIC16) return pick_un<IRIS_DTYPE_F16, OP_ATOMIC16>(un, a_lds);
  }
  return nullptr;
}

}  // namespace iris_amd
