// Table of compiled shard-GEMM kernels.  Each instantiation file defines the
// entries of one (operand type, epilogue op) pair; the launcher picks one
// entry per call.
#pragma once

#include "gemm_kernel.hpp"

namespace iris_amd {

using GemmKernelFn = void (*)(const GemmKArgs);

struct GemmKernelEntry {
  int dt;      // operand type: IRIS_DTYPE_F16 | IRIS_DTYPE_BF16 | IRIS_DTYPE_F32
  int op;      // StoreOp
  int cm, cn;  // compute tile
  int bk, wm, wn, stages;  // (bk in 16-bit units: half as many elements of fp32 operands)
  bool dma;    // LDS-DMA loader (needs K-contiguous, 16-byte aligned operands)
  bool splitk;  // the kernel can share a tile's K range with other programs
  bool split_owner;  // ... and its first part can add the others' partials itself (needed for stream-K runs)
  int threads;        // launch size: the multiplying waves and the fetching waves (if any)
  int fetch_waves;    // waves that only issue the stage loads (0: every wave fetches its share)
  int lds_bytes;
  GemmKernelFn fn;
  GemmKernelFn fn_split;  // split-K build, or null
  GemmKernelFn fn_fused;  // build with the one-shot reduce inside the program (store epilogues), or null
  GemmKernelFn fn_merged;  // build whose tiles are blocks of the caller's (store epilogues, 256 x 128 and 256 x 256), or null
  GemmKernelFn fn_split_merged;  // ... and its split-K build, or null
  GemmKernelFn fn_touch;         // unsplit build that touches lines of K-steps to come (the eight-wave 256 x 256 tile), or null
  GemmKernelFn fn_touch_merged;  // ... whose tiles are blocks of the caller's
  const char* name;
};

template <class Cfg, int OP, int ODT>
constexpr GemmKernelFn split_fn() {
  if constexpr (Cfg::SPLITK)
    return &gemm_persistent_kernel<Cfg, OP, ODT, true>;
  else
    return nullptr;
}

template <class Cfg, int OP, int ODT>
constexpr GemmKernelFn fused_fn() {
  // (the tiles with fetching waves have no such build: the reduce wants the registers their
  // fetch state takes, and the launcher takes the plain tile of the same shape instead)
  if constexpr ((OP == OP_STORE16 || OP == OP_STORE32) && Cfg::LW == 0)
    return &gemm_persistent_kernel<Cfg, OP, ODT, false, true>;
  else
    return nullptr;
}

// The launcher only merges the caller's tiles into 256 x 128 and 256 x 256 ones, for the store epilogues, and
// runs them with the table's first tile of either shape.
// (... and, for a range of the caller's columns launched on its own, with the 256 x 64 one as it is)
template <class Cfg>
constexpr bool merged_build = Cfg::CM == 256 && Cfg::DMA && Cfg::BK == 64 &&
                              ((Cfg::CN == 256 && Cfg::LW == 0 && Cfg::NW == 8) || (Cfg::CN == 128 && Cfg::LW == 4) ||
                               (Cfg::CN == 64 && Cfg::LW == 4 && Cfg::S == 3));
template <class Cfg, int OP, int ODT>
constexpr GemmKernelFn merged_fn() {
  if constexpr ((OP == OP_STORE16 || OP == OP_STORE32) && merged_build<Cfg>)
    return &gemm_persistent_kernel<Cfg, OP, ODT, false, false, true>;
  else
    return nullptr;
}

template <class Cfg, int OP, int ODT>
constexpr GemmKernelFn split_merged_fn() {
  if constexpr ((OP == OP_STORE16 || OP == OP_STORE32) && merged_build<Cfg> && Cfg::SPLITK)
    return &gemm_persistent_kernel<Cfg, OP, ODT, true, false, true>;
  else
    return nullptr;
}

// The eight-wave 256 x 256 tile's builds with the touches of Loader::touch (store epilogues).
template <class Cfg>
constexpr bool touch_build = Cfg::CM == 256 && Cfg::CN == 256 && Cfg::DMA && Cfg::BK == 64 && Cfg::LW == 0 && Cfg::NW == 8 &&
                             Cfg::S == 2 && Cfg::WM == 2;
template <int DT>
using TouchCfg = GemmCfg<DT, 256, 256, 64, 2, 4, 2, true, 0, true>;
template <class Cfg, int OP, int ODT, bool MERGED>
constexpr GemmKernelFn touch_fn() {
  if constexpr ((OP == OP_STORE16 || OP == OP_STORE32) && touch_build<Cfg>)
    return &gemm_persistent_kernel<TouchCfg<Cfg::DT>, OP, ODT, false, false, MERGED>;
  else
    return nullptr;
}

template <class Cfg, int OP>
constexpr GemmKernelEntry make_entry(const char* name) {
  constexpr int ODT = (OP == OP_STORE32 || OP == OP_ATOMIC32) ? IRIS_DTYPE_F32 : Cfg::DT;
  return GemmKernelEntry{Cfg::DT, OP,      Cfg::CM, Cfg::CN, Cfg::BK,        Cfg::WM,
                         Cfg::WN, Cfg::S,  Cfg::DMA, Cfg::SPLITK, Cfg::SPLIT_OWNER, Cfg::THREADS, Cfg::LW, Cfg::LDS_BYTES,
                         &gemm_persistent_kernel<Cfg, OP, ODT, false>, split_fn<Cfg, OP, ODT>(), fused_fn<Cfg, OP, ODT>(),
                         merged_fn<Cfg, OP, ODT>(), split_merged_fn<Cfg, OP, ODT>(), touch_fn<Cfg, OP, ODT, false>(),
                         touch_fn<Cfg, OP, ODT, true>(), name};
}

// The variants, in the launcher's order of preference: the first entry whose
// compute tile divides the logical tile (and whose loader fits the operands)
// wins.  `variant` k > 0 in iris_gemm_args forces entry k-1 (tuning runs).
// Columns: compute tile CM, CN, BK; waves WM x WN; stages; LDS-DMA loader;
// fetching waves; whether the tile also has a split-K build (must equal
// GemmCfg::SPLITK); name.
//
// The four-wave tiles come twice: with one fetching wave per SIMD beside the
// multiplying one (`_f4`: a K-step then costs the longer of fetch and multiply
// instead of their sum; [2048,4096] x [4096,1376] in 128 x 128 tiles 48 -> 40 us)
// and as deep a ring as LDS holds, since a fetching wave cannot refill the
// stage that is being multiplied (256 x 64 tiles in three stages instead of
// two: 57 -> 42 us on the same shape); and plain, which the launcher takes
// where the first loses: with the reduce inside the program (no such build)
// and for two programs per CU.
#define IRIS_GEMM_VARIANTS(X, DT, OP)                                     \
  X(DT, OP, 256, 256, 64, 2, 4, 2, true, 0, 1, "256x256x64_w2x4_s2")         \
  X(DT, OP, 256, 128, 64, 2, 2, 3, true, 4, 1, "256x128x64_w2x2_s3_f4")      \
  X(DT, OP, 128, 256, 64, 1, 4, 3, true, 4, 1, "128x256x64_w1x4_s3_f4")      \
  X(DT, OP, 128, 128, 64, 2, 2, 4, true, 4, 1, "128x128x64_w2x2_s4_f4")      \
  X(DT, OP, 256, 64, 64, 4, 1, 3, true, 4, 1, "256x64x64_w4x1_s3_f4")        \
  X(DT, OP, 128, 64, 64, 2, 2, 4, true, 4, 1, "128x64x64_w2x2_s4_f4")        \
  X(DT, OP, 64, 128, 64, 2, 2, 4, true, 4, 1, "64x128x64_w2x2_s4_f4")        \
  X(DT, OP, 64, 64, 128, 2, 2, 4, true, 4, 1, "64x64x128_w2x2_s4_f4")        \
  X(DT, OP, 256, 128, 64, 2, 2, 2, true, 0, 1, "256x128x64_w2x2_s2")         \
  X(DT, OP, 128, 256, 64, 1, 4, 2, true, 0, 1, "128x256x64_w1x4_s2")         \
  X(DT, OP, 128, 128, 64, 2, 2, 4, true, 0, 1, "128x128x64_w2x2_s4")         \
  X(DT, OP, 256, 64, 64, 4, 1, 2, true, 0, 1, "256x64x64_w4x1_s2")           \
  X(DT, OP, 64, 64, 64, 2, 2, 4, true, 0, 1, "64x64x64_w2x2_s4")             \
  X(DT, OP, 64, 64, 32, 2, 2, 1, false, 0, 0, "64x64x32_w2x2_generic")

// extra variants, compiled for the bf16 store op only (tuning runs, and the
// one-substep stage whose fragment buffers alternate from step to step)
#define IRIS_GEMM_TUNING_VARIANTS(X, DT, OP)                              \
  X(DT, OP, 256, 128, 32, 2, 4, 4, true, 0, 0, "256x128x32_w2x4_s4")         \
  X(DT, OP, 256, 128, 64, 2, 4, 2, true, 0, 1, "256x128x64_w2x4_s2")         \
  X(DT, OP, 128, 256, 64, 2, 4, 2, true, 0, 1, "128x256x64_w2x4_s2")         \
  X(DT, OP, 128, 128, 32, 2, 2, 4, true, 0, 0, "128x128x32_w2x2_s4")         \
  X(DT, OP, 64, 64, 64, 2, 2, 4, true, 4, 1, "64x64x64_w2x2_s4_f4")          \
  X(DT, OP, 256, 64, 64, 4, 1, 2, true, 4, 1, "256x64x64_w4x1_s2_f4")

#define IRIS_GEMM_ENTRY(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW, SPLIT, NAME) \
  make_entry<GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>, OP>(NAME),

// Explicit instantiation of an entry's kernels.  Taking their addresses in
// make_entry should be enough, but with the plain and the split-K build of a
// tile in one translation unit the compiler's host pass has been seen to
// reference one of the two without emitting it.
#define IRIS_GEMM_ODT(DT, OP) (((OP) == OP_STORE32 || (OP) == OP_ATOMIC32) ? IRIS_DTYPE_F32 : (DT))
#define IRIS_GEMM_INSTANTIATE_SPLIT_0(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW) \
  static_assert(!GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>::SPLITK, "split-K column of the variant table");
#define IRIS_GEMM_INSTANTIATE_SPLIT_1(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW)                                  \
  static_assert(GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>::SPLITK, "split-K column of the variant table"); \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>, OP,           \
                                                  IRIS_GEMM_ODT(DT, OP), true>(const GemmKArgs);
#define IRIS_GEMM_INSTANTIATE(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW, SPLIT, NAME)                    \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>, OP,    \
                                                  IRIS_GEMM_ODT(DT, OP), false>(const GemmKArgs); \
  IRIS_GEMM_INSTANTIATE_SPLIT_##SPLIT(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW)
// the store epilogues' build with the one-shot reduce inside the program
#define IRIS_GEMM_INSTANTIATE_FUSED(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW, SPLIT, NAME) \
  IRIS_GEMM_INSTANTIATE_FUSED_##LW(DT, OP, CM, CN, BK, WM, WN, S, DMA)
#define IRIS_GEMM_INSTANTIATE_FUSED_0(DT, OP, CM, CN, BK, WM, WN, S, DMA)                     \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA>, OP, \
                                                  IRIS_GEMM_ODT(DT, OP), false, true>(const GemmKArgs);
#define IRIS_GEMM_INSTANTIATE_FUSED_4(DT, OP, CM, CN, BK, WM, WN, S, DMA)

// the store epilogues' builds whose tiles are blocks of the caller's
#define IRIS_GEMM_INSTANTIATE_MERGED(DT, OP)                                                                        \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, 256, 256, 64, 2, 4, 2, true, 0>, OP,                \
                                                  IRIS_GEMM_ODT(DT, OP), false, false, true>(const GemmKArgs); \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, 256, 128, 64, 2, 2, 3, true, 4>, OP,                \
                                                  IRIS_GEMM_ODT(DT, OP), false, false, true>(const GemmKArgs); \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, 256, 256, 64, 2, 4, 2, true, 0>, OP,                \
                                                  IRIS_GEMM_ODT(DT, OP), true, false, true>(const GemmKArgs);  \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, 256, 128, 64, 2, 2, 3, true, 4>, OP,                \
                                                  IRIS_GEMM_ODT(DT, OP), true, false, true>(const GemmKArgs);  \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, 256, 64, 64, 4, 1, 3, true, 4>, OP,                 \
                                                  IRIS_GEMM_ODT(DT, OP), false, false, true>(const GemmKArgs); \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, 256, 64, 64, 4, 1, 3, true, 4>, OP,                 \
                                                  IRIS_GEMM_ODT(DT, OP), true, false, true>(const GemmKArgs);  \
  template __global__ void gemm_persistent_kernel<TouchCfg<DT>, OP, IRIS_GEMM_ODT(DT, OP), false, false, false>(  \
      const GemmKArgs);                                                                                           \
  template __global__ void gemm_persistent_kernel<TouchCfg<DT>, OP, IRIS_GEMM_ODT(DT, OP), false, false, true>(   \
      const GemmKArgs);

// fp32 operands (fp32 output only): a short table.  The tiles are the 16-bit ones' (a stage of BK 16-bit units holds
// BK / 2 elements of K; the names count elements); the matrix cores run fp32 at a sixteenth of the 16-bit rate, so any
// tile that keeps them fed will do, and none is split along K or merged.
template <class Cfg, int OP>
constexpr GemmKernelEntry make_entry_f32(const char* name) {
  static_assert(Cfg::DT == IRIS_DTYPE_F32 && (OP == OP_STORE32 || OP == OP_ATOMIC32), "fp32 operands, fp32 output");
  return GemmKernelEntry{Cfg::DT, OP, Cfg::CM, Cfg::CN, Cfg::BK, Cfg::WM, Cfg::WN, Cfg::S, Cfg::DMA, false, false,
                         Cfg::THREADS, Cfg::LW, Cfg::LDS_BYTES, &gemm_persistent_kernel<Cfg, OP, IRIS_DTYPE_F32, false>,
                         nullptr, fused_fn<Cfg, OP, IRIS_DTYPE_F32>(), nullptr, nullptr, nullptr, nullptr, name};
}
#define IRIS_GEMM_F32_VARIANTS(X, OP)                                                   \
  X(IRIS_DTYPE_F32, OP, 128, 128, 64, 2, 2, 4, true, 4, "128x128x32_w2x2_s4_f4_fp32")  \
  X(IRIS_DTYPE_F32, OP, 128, 128, 64, 2, 2, 4, true, 0, "128x128x32_w2x2_s4_fp32")     \
  X(IRIS_DTYPE_F32, OP, 64, 64, 64, 2, 2, 4, true, 0, "64x64x32_w2x2_s4_fp32")         \
  X(IRIS_DTYPE_F32, OP, 64, 64, 32, 2, 2, 1, false, 0, "64x64x16_w2x2_generic_fp32")
#define IRIS_GEMM_F32_ENTRY(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW, NAME) \
  make_entry_f32<GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>, OP>(NAME),
#define IRIS_GEMM_F32_INSTANTIATE(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW, NAME)                    \
  template __global__ void gemm_persistent_kernel<GemmCfg<DT, CM, CN, BK, WM, WN, S, DMA, LW>, OP, \
                                                  IRIS_DTYPE_F32, false>(const GemmKArgs);
#define IRIS_GEMM_F32_INSTANTIATE_FUSED(DT, OP, CM, CN, BK, WM, WN, S, DMA, LW, NAME) \
  IRIS_GEMM_INSTANTIATE_FUSED_##LW(DT, OP, CM, CN, BK, WM, WN, S, DMA)

#define IRIS_GEMM_DECLARE(TAG) const GemmKernelEntry* gemm_entries_##TAG(int* count);
IRIS_GEMM_DECLARE(f32_store32)
IRIS_GEMM_DECLARE(f32_atomic32)
IRIS_GEMM_DECLARE(bf16_store16)
IRIS_GEMM_DECLARE(bf16_store32)
IRIS_GEMM_DECLARE(bf16_atomic32)
IRIS_GEMM_DECLARE(bf16_atomic16)
IRIS_GEMM_DECLARE(f16_store16)
IRIS_GEMM_DECLARE(f16_store32)
IRIS_GEMM_DECLARE(f16_atomic32)
IRIS_GEMM_DECLARE(f16_atomic16)

}  // namespace iris_amd
