// Instantiations of the few-rows shard GEMM.
#include "gemm_skinny.hpp"

namespace iris_amd {

namespace {

template <int DT, int OP>
GemmKernelFn pick_un(int un, bool a_lds, int rb, int cb) {
  constexpr int ODT = (OP == OP_STORE32 || OP == OP_ATOMIC32) ? IRIS_DTYPE_F32 : DT;
  if (rb == 1 && cb == 1) {
    switch (un) {
      case 2: return a_lds ? &gemm_skinny_kernel<DT, OP, ODT, 2, true> : &gemm_skinny_kernel<DT, OP, ODT, 2, false>;
      case 4: return a_lds ? &gemm_skinny_kernel<DT, OP, ODT, 4, true> : &gemm_skinny_kernel<DT, OP, ODT, 4, false>;
      case 8: return a_lds ? &gemm_skinny_kernel<DT, OP, ODT, 8, true> : &gemm_skinny_kernel<DT, OP, ODT, 8, false>;
    }
  } else if (rb == 2 && cb == 1 && a_lds) {
    switch (un) {
      case 2: return &gemm_skinny_kernel<DT, OP, ODT, 2, true, 2, 1>;
      case 4: return &gemm_skinny_kernel<DT, OP, ODT, 4, true, 2, 1>;
      case 8: return &gemm_skinny_kernel<DT, OP, ODT, 8, true, 2, 1>;
    }
  }
  // (32 x 32 a workgroup, gemm_skinny_kernel<..., 2, 2>, works and is not built: LDS only holds four K blocks
  // of it a wave, a K of 4096 takes two rounds of fetches, and [128,4096] x [4096,1376] takes 18.4 us against
  // the persistent kernel's 13.4)
  return nullptr;
}

}  // namespace

GemmKernelFn gemm_skinny_kernel_for(int dt, int op, int un, bool a_lds, int rb, int cb) {
  if (dt == IRIS_DTYPE_BF16) {
    if (op == OP_STORE16) return pick_un<IRIS_DTYPE_BF16, OP_STORE16>(un, a_lds, rb, cb);
    if (op == OP_STORE32) return pick_un<IRIS_DTYPE_BF16, OP_STORE32>(un, a_lds, rb, cb);
    if (op == OP_ATOMIC32) return pick_un<IRIS_DTYPE_BF16, OP_ATOMIC32>(un, a_lds, rb, cb);
    if (op == OP_ATOMIC16) return pick_un<IRIS_DTYPE_BF16, OP_ATOMIC16>(un, a_lds, rb, cb);
  } else if (dt == IRIS_DTYPE_F16) {
    if (op == OP_STORE16) return pick_un<IRIS_DTYPE_F16, OP_STORE16>(un, a_lds, rb, cb);
    if (op == OP_STORE32) return pick_un<IRIS_DTYPE_F16, OP_STORE32>(un, a_lds, rb, cb);
    if (op == OP_ATOMIC32) return pick_un<IRIS_DTYPE_F16, OP_ATOMIC32>(un, a_lds, rb, cb);
    if (op == OP_ATOMIC16) return pick_un<IRIS_DTYPE_F16, OP_ATOMIC16>(un, a_lds, rb, cb);
  }
  return nullptr;
}

}  // namespace iris_amd
