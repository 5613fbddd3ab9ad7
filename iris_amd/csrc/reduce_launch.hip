// C-ABI launchers of the one-shot reduce, the tile signal and the int32 fill
// (include/iris_amd.h).
#include <cstdio>
#include <cstdlib>

#include "reduce_kernel.hpp"

namespace iris_amd {
namespace {

using ReduceFn = void (*)(const ReduceKArgs);

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// The default kernel keeps three rows of strips in flight per lane and reads
// the partials with loads that are coherent at the flags' scope (sc1 for the
// agent, sc0 sc1 for the system), which spares the cache-invalidating fence
// after every flag wait (~35 us over the 1024 tiles of an [8192,8192] reduce).
template <int IN_DT, int OUT_DT>
ReduceFn pick_vec(int ws, int variant, bool sys, bool rows) {
  constexpr int AGENT = AUX_NT | AUX_SC1, SYSTEM = AUX_NT | AUX_SC1 | AUX_SC0;
  if (rows) {
    if (ws == 8) return sys ? &reduce_rows_kernel<IN_DT, OUT_DT, SYSTEM, 8> : &reduce_rows_kernel<IN_DT, OUT_DT, AGENT, 8>;
    return sys ? &reduce_rows_kernel<IN_DT, OUT_DT, SYSTEM, 0> : &reduce_rows_kernel<IN_DT, OUT_DT, AGENT, 0>;
  }
  if (ws != 8)
    return sys ? &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 0, 2, SYSTEM> : &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 0, 2, AGENT>;
  if (sys) return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 3, SYSTEM>;
  // variant: 0 default; 1..6 tuning points of (UNROLL, load cache policy)
  switch (variant) {
    case 1: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 2, AGENT>;
    case 2: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 2, SYSTEM>;
    case 3: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 2, AUX_NT>;  // plain loads behind an acquire fence
    case 4: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 4, AGENT>;
    case 5: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 2, AUX_SC1>;
    case 6: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 1, AGENT>;
    default: return &reduce_tiles_vec_kernel<IN_DT, OUT_DT, 8, 3, AGENT>;
  }
}

ReduceFn pick(int in_dt, int out_dt, int ws, int variant, bool sys, bool rows) {
  if (in_dt == IRIS_DTYPE_F32) {
    if (out_dt == IRIS_DTYPE_BF16) return pick_vec<IRIS_DTYPE_F32, IRIS_DTYPE_BF16>(ws, variant, sys, rows);
    if (out_dt == IRIS_DTYPE_F16) return pick_vec<IRIS_DTYPE_F32, IRIS_DTYPE_F16>(ws, variant, sys, rows);
    return pick_vec<IRIS_DTYPE_F32, IRIS_DTYPE_F32>(ws, variant, sys, rows);
  }
  if (in_dt == IRIS_DTYPE_BF16) {
    if (out_dt == IRIS_DTYPE_BF16) return pick_vec<IRIS_DTYPE_BF16, IRIS_DTYPE_BF16>(ws, variant, sys, rows);
    if (out_dt == IRIS_DTYPE_F32) return pick_vec<IRIS_DTYPE_BF16, IRIS_DTYPE_F32>(ws, variant, sys, rows);
    return nullptr;
  }
  if (in_dt == IRIS_DTYPE_F16) {
    if (out_dt == IRIS_DTYPE_F16) return pick_vec<IRIS_DTYPE_F16, IRIS_DTYPE_F16>(ws, variant, sys, rows);
    if (out_dt == IRIS_DTYPE_F32) return pick_vec<IRIS_DTYPE_F16, IRIS_DTYPE_F32>(ws, variant, sys, rows);
    return nullptr;
  }
  return nullptr;
}

bool valid_dtype(int dt) { return dt == IRIS_DTYPE_F32 || dt == IRIS_DTYPE_F16 || dt == IRIS_DTYPE_BF16; }

}  // namespace
}  // namespace iris_amd

using namespace iris_amd;

extern "C" int iris_one_shot_reduce_launch(const iris_reduce_args* a, void* stream) {
  if (!a) return hipErrorInvalidValue;
  if (a->M < 0 || a->N < 0 || a->block_m <= 0 || a->block_n <= 0 || a->group_size_m <= 0) return hipErrorInvalidValue;
  if (a->world_size <= 0 || a->cur_rank < 0 || a->cur_rank >= a->world_size) return hipErrorInvalidValue;
  if (a->world_size > 1 && !a->heap_bases) return hipErrorInvalidValue;
  if (a->wait_flags && a->world_size > 1 && !a->tile_completed) return hipErrorInvalidValue;
  if (!valid_dtype(a->c_dtype) || !valid_dtype(a->c_global_dtype)) return hipErrorInvalidValue;
  if (a->num_sms < 0 || a->num_xcds <= 0) return hipErrorInvalidValue;
  if (a->M == 0 || a->N == 0) return hipSuccess;
  if (!a->c || !a->c_global) return hipErrorInvalidValue;

  ReduceKArgs k{};
  k.c = static_cast<const char*>(a->c);
  k.cg = static_cast<char*>(a->c_global);
  k.flags = a->tile_completed;
  k.heap_bases = a->heap_bases;
  k.status = a->status;
  k.timeout = a->spin_timeout_ticks ? a->spin_timeout_ticks : 200000000ull;  // 2 s at 100 MHz
  k.scm = a->stride_cm;
  k.scn = a->stride_cn;
  k.sgm = a->stride_cm_global;
  k.sgn = a->stride_cn_global;
  k.M = a->M;
  k.N = a->N;
  k.BM = a->block_m;
  k.BN = a->block_n;
  k.G = a->group_size_m;
  k.num_pid_m = (a->M + a->block_m - 1) / a->block_m;
  k.num_pid_n = (a->N + a->block_n - 1) / a->block_n;
  k.total_tiles = k.num_pid_m * k.num_pid_n;
  k.cur_rank = a->cur_rank;
  k.ws = a->world_size;
  k.c_dt = a->c_dtype;
  k.cg_dt = a->c_global_dtype;
  k.sys = a->scope == IRIS_SCOPE_SYSTEM;
  k.wait_flags = a->wait_flags;
  if (a->flag_sem != IRIS_FLAG_SEM_WRITE_THROUGH && a->flag_sem != IRIS_FLAG_SEM_RELEASE_ACQUIRE)
    return hipErrorInvalidValue;
  k.acquire = a->flag_sem == IRIS_FLAG_SEM_RELEASE_ACQUIRE;

  // default grid: two blocks per CU, each walking its share of the tiles
  int grid = a->num_sms > 0 ? a->num_sms : 2 * current_cu_count();
  if (grid > k.total_tiles) grid = k.total_tiles;
  // the XCD remap is a permutation only when the grid splits evenly
  k.num_xcds = (a->num_xcds > 1 && grid % a->num_xcds == 0) ? a->num_xcds : 1;

  const int ies = dtype_size(k.c_dt), oes = dtype_size(k.cg_dt);
  // a lane moves 16 bytes of input at a time: 4 fp32 or 8 16-bit columns
  const int ve = 16 / ies;
  const bool vec = k.scn == 1 && k.sgn == 1 && aligned16(k.c) && aligned16(k.cg) && (k.scm * ies) % 16 == 0 &&
                   (k.sgm * oes) % 16 == 0 && k.BN % ve == 0 && k.N % ve == 0 && (k.BN * oes) % 16 == 0 &&
                   // lane offsets inside a tile are 32-bit
                   k.scm >= k.N && k.sgm >= k.N && ((int64_t)k.BM + 256) * k.scm * ies < (1ll << 31) &&
                   ((int64_t)k.BM + 256) * k.sgm * oes < (1ll << 31);
  // Row bands instead of tiles (variant 7 asks for them, 8 forbids them): an
  // item is 8192 elements per partial, whole rows when they are shorter.
  // They pay off when a row is long, from 16 KiB of input a row ...
  bool rows = false;
  if (vec && a->variant != 8) {
    const int item_vecs = ies == 4 ? 2048 : 1024;  // 16-byte strips per item: 8192 elements
    const int nv = k.N / ve;
    k.band_vecs = nv < item_vecs ? nv : item_vecs;
    int br = 1;
    if (nv < item_vecs)
      while (br * 2 * nv <= item_vecs && k.BM % (br * 2) == 0) br *= 2;
    k.band_rows = br;
    k.band_chunks = (nv + k.band_vecs - 1) / k.band_vecs;
    k.band_items = ((k.M + br - 1) / br) * k.band_chunks;
    const bool fits = k.BN >= 64 &&  // one lane per tile of the band for the flag wait: at most 129 tiles
                      (int64_t)br * k.scm * ies < (1ll << 31) && (int64_t)br * k.sgm * oes < (1ll << 31);
    // ... and when there is an item for every CU: with fewer, the tile walk has
    // more loads in flight
    rows = fits && (a->variant == 7 ||
                    (a->variant == 0 && (int64_t)k.N * ies >= 16384 && k.band_items >= current_cu_count()));
  }
  // (the tile kernel paces its walk only when a program has several tiles)
  k.pace = k.total_tiles > grid ? 1 : 0;
  ReduceFn fn = vec ? pick(k.c_dt, k.cg_dt, k.ws, a->variant, k.sys != 0, rows) : nullptr;
  if (!fn) {
    fn = &reduce_tiles_generic_kernel;
    rows = false;
  }
  if (rows) {
    grid = a->num_sms > 0 ? a->num_sms : 2 * current_cu_count();
    if (grid > k.band_items) grid = k.band_items;
  }
  // (the groups' count shares a 32-bit flag with a value below 2^16)
  k.reset_in_kernel = (rows && k.wait_flags && k.ws > 1 && grid < (1 << 15) && k.ws <= (1 << 15)) ? 1 : 0;
  hipLaunchKernelGGL(fn, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream), k);
  hipError_t err = hipGetLastError();
  if (err == hipSuccess && rows && k.wait_flags && k.ws > 1 && !k.reset_in_kernel) {
    hipLaunchKernelGGL(reset_consumed_flags_kernel, dim3((k.total_tiles + 255) / 256), dim3(256), 0,
                       static_cast<hipStream_t>(stream), k.flags, k.ws - 1, k.total_tiles);
    err = hipGetLastError();
  }
  return err;
}

extern "C" int iris_signal_tiles_launch(int32_t* tile_completed, const uint64_t* heap_bases, int32_t total_tiles,
                                        int32_t cur_rank, int32_t world_size, int32_t include_self, int32_t scope,
                                        void* stream) {
  if (total_tiles < 0 || world_size <= 0 || cur_rank < 0 || cur_rank >= world_size) return hipErrorInvalidValue;
  if (total_tiles == 0) return hipSuccess;
  if (!tile_completed || (world_size > 1 && !heap_bases)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(signal_tiles_kernel, dim3((total_tiles + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), tile_completed, heap_bases, total_tiles, cur_rank, world_size,
                     include_self, scope == IRIS_SCOPE_SYSTEM ? 1 : 0);
  return hipGetLastError();
}

extern "C" int iris_memset_i32_launch(int32_t* ptr, int32_t value, int64_t n_elements, void* stream) {
  if (n_elements < 0) return hipErrorInvalidValue;
  if (n_elements == 0) return hipSuccess;
  if (!ptr) return hipErrorInvalidValue;
  const int64_t blocks = (n_elements + 1023) / 1024;
  hipLaunchKernelGGL(memset_i32_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream), ptr,
                     value, n_elements);
  return hipGetLastError();
}

extern "C" int iris_tile_schedule_launch(int32_t* out, int32_t M, int32_t N, int32_t block_m, int32_t block_n,
                                         int32_t group_size_m, int32_t num_sms, int32_t num_xcds, void* stream) {
  if (M <= 0 || N <= 0 || block_m <= 0 || block_n <= 0 || group_size_m <= 0 || num_sms <= 0 || num_xcds <= 0 ||
      num_sms % num_xcds != 0 || !out)
    return hipErrorInvalidValue;
  const int npm = (M + block_m - 1) / block_m, npn = (N + block_n - 1) / block_n;
  hipLaunchKernelGGL(tile_schedule_kernel, dim3((num_sms + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), out, npm, npn, group_size_m, num_sms, num_xcds,
                     make_tile_divs(npm, npn, group_size_m));
  return hipGetLastError();
}

extern "C" void iris_tile_map_host(int32_t tile_id, int32_t M, int32_t N, int32_t block_m, int32_t block_n,
                                   int32_t group_size_m, int32_t* pid_m, int32_t* pid_n) {
  // (the GEMM kernels' arithmetic: multiply-high divisions by the launch's divisors)
  const int npm = (M + block_m - 1) / block_m, npn = (N + block_n - 1) / block_n;
  const TileCoord tc = tile_map_fast(tile_id, npm, npn, group_size_m, make_tile_divs(npm, npn, group_size_m));
  *pid_m = tc.pid_m;
  *pid_n = tc.pid_n;
}
