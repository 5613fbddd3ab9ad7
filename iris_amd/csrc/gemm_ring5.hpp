// Shard GEMM, 256 x 256 tile, with a ring of five half-stages.
//
// gemm_persistent_kernel keeps two 64 KiB stages (BK = 64) and 32 KiB of
// epilogue scratch in the CU's 160 KiB of LDS.  A stage can then only be
// refilled during the second half of the K-step before the one that reads it,
// and the path from L1 into LDS (about 45 bytes a clock) needs most of a
// K-step's MFMA time for the 64 KiB: the loads land late and the hand-over
// waits for them.
//
// Here LDS holds five slabs of 32 k (A 256 x 32 and B 256 x 32, 32 KiB each)
// and nothing else.  A K-step still
// covers 64 k, two slabs, behind one barrier, but of the two slabs that a
// hand-over frees and refills only the first is needed at the next hand-over:
// it is issued right away, four loads a wave, and has a whole step to land;
// the second is needed a step later and is issued at leisure, during the
// first half of the next step.
//
//   step g reads slabs 2g, 2g+1;  at its hand-over 2g+2 and 2g+3 have landed,
//   2g+4 may still be in flight;  the hand-over frees the slots of 2g and
//   2g+1, which take 2g+5 (issued in the rest of this step) and 2g+6 (issued
//   in the first half of step g+1).  Slab h lives in slot h mod 5, h counted
//   across the tiles of the program.
//
// The epilogue is the other kernel's (store_acc, through LDS): when a tile
// ends, the slot of the slab read last stays free until the next step's first
// half refills it, and there every wave writes only its own four 1 KiB
// blocks, which serve as the wave's scratch in between.
//
// Restrictions (the launcher checks them): LDS-DMA operands, one 256 x 256
// compute tile per logical tile, K a multiple of 64, store epilogues only.
#pragma once

#include "gemm_kernel.hpp"

namespace iris_amd {

template <int DT>
using Ring5Cfg = GemmCfg<DT, 256, 256, 32, 2, 4, 4, true>;  // S only sizes unused constants here
constexpr int RING5_SLOTS = 5;
template <int DT>
constexpr int ring5_lds_bytes() {
  return RING5_SLOTS * Ring5Cfg<DT>::STAGE;
}

template <int DT, int OP, int ODT>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_ring5_kernel(
    const GemmKArgs p) {
  using Cfg = Ring5Cfg<DT>;
  static_assert(OP == OP_STORE16 || OP == OP_STORE32, "store epilogues only");
  constexpr int L = Cfg::L;  // DMA loads a wave and slab
  constexpr int FAST_STORES = StoreCount<Cfg, OP>::FAST_STORES;
  // a wave's DMA blocks within a slot: blk = i * NW + wave, i = 0, 1 of A then of B
  constexpr int SCRATCH_STRIDE = Cfg::NW * 1024;
  static_assert(Cfg::A_LOADS == 2 && Cfg::B_LOADS == 2 && Cfg::A_BYTES == 2 * SCRATCH_STRIDE &&
                    Cfg::WS_BYTES == 4 * 1024,
                "the wave's four DMA blocks of a slot are its 32 scratch rows");
  static_assert(FAST_STORES + L <= 63, "vmcnt immediate");
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  IRIS_LDS char* lds = (IRIS_LDS char*)lds_raw;

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  const int pid = xcd_remap(blockIdx.x, p.num_sms, p.num_xcds);
  const int n_items = pid < p.total_tiles ? (p.total_tiles - pid + p.num_sms - 1) / p.num_sms : 0;
  const int nh = p.K / Cfg::BK;  // slabs per tile, even
  if (n_items == 0 || nh == 0) return;

  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  // fragment fetch: lane l reads row l%16 of a 16-row block, 16-byte chunk l/16
  const int lrow = lane & 15, lq = lane >> 4;
  const int xo = (lq ^ ((lrow / Cfg::RP) % Cfg::CPR)) * 16;
  const int a_lane = (wm * Cfg::TM + lrow) * Cfg::BK * 2 + xo;
  const int b_lane = Cfg::A_BYTES + (wn * Cfg::TN + lrow) * Cfg::BK * 2 + xo;

  f32x4 acc[Cfg::IM][Cfg::IN];
#pragma unroll
  for (int i = 0; i < Cfg::IM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::IN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  // Publication of a tile's flag waits for the tile's stores, which are left
  // in flight across the first hand-over of the next tile (pending_skip) and
  // are known complete at the second: memory operations complete in order,
  // and loads younger than the stores have been waited for by then.
  int pending_tile = -1, pending_skip = 0;

  int c_item = 0;
  Item c_it = decode_item<Cfg, false>(p, pid, 0);
  int c_slot = 0;  // slot of the slab the next step starts with

  Loader<Cfg> ld;
  int l_item = 0, l_h = 0, l_slot = 0;
  Item l_it = c_it;
  ld.setup(p, l_it, wave, lane, 0);
  // four loads of the cursor's slab have been issued: move on to the next slab
  auto advance_load_cursor = [&]() __attribute__((always_inline)) {
    l_slot = (l_slot == RING5_SLOTS - 1) ? 0 : l_slot + 1;
    if (++l_h == nh) {
      l_h = 0;
      if (++l_item < n_items) {
        l_it = decode_item<Cfg, false>(p, pid, l_item);
        ld.setup(p, l_it, wave, lane, 0);
      } else {
        ld.park();  // nothing left to load: the loads go on, and fetch nothing
      }
    }
  };
  auto issue_load = [&](int i) __attribute__((always_inline)) {
    ld.issue_at(p, lds + l_slot * Cfg::STAGE, l_h, wave, i);
  };

  auto epilogue = [&]() __attribute__((always_inline)) {
    if (pending_tile >= 0) {
      // a one-step tile: the previous tile has not been published yet
      IRIS_WAIT_VMCNT(0);
      __syncthreads();
      if (tid == 0) publish_tile(p, pending_tile);
      pending_tile = -1;
    }
    // The slot of the slab read last is free until the next step's first half
    // refills it, and there every wave writes only its own 1 KiB blocks (two of
    // A, two of B, 8 KiB apart): those four blocks are the wave's scratch.
    const int s_free = c_slot == 0 ? RING5_SLOTS - 1 : c_slot - 1;
    IRIS_LDS char* ws = lds + s_free * Cfg::STAGE + wave * 1024;
    const bool fast = store_acc<Cfg, OP, ODT, SCRATCH_STRIDE>(p, acc, ws, c_it.m0 + wm * Cfg::TM,
                                                              c_it.n0 + wn * Cfg::TN, c_it.m_end, c_it.n_end, lane);
    if (p.flag_mode != 0) {
      pending_tile = __builtin_amdgcn_readfirstlane(c_it.tile_id);
      pending_skip = fast ? 1 : 0;
    }
    if (p.ts_end && tid == 0)
      __hip_atomic_fetch_max((IRIS_GLOBAL unsigned long long*)(p.ts_end + c_it.tile_id),
                             (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (++c_item < n_items) c_it = decode_item<Cfg, false>(p, pid, c_item);
  };

  // ---- prologue: slabs 0..3 go out; 0 and 1 must have landed ---------------
#pragma unroll
  for (int s = 0; s < 4; ++s) {
#pragma unroll
    for (int i = 0; i < L; ++i) issue_load(i);
    advance_load_cursor();
  }
  IRIS_WAIT_VMCNT(2 * L);
  block_barrier_raw();
  Frags<Cfg> fr;
  load_all<Cfg>(lds + a_lane, lds + b_lane, fr, 0);
  IRIS_WAIT_LGKMCNT0();

  // One K-step: slabs in slots c_slot (its fragments are in registers, B in
  // buffer 0) and c_slot + 1.
  auto step = [&](auto first_tag) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_tag)::value;
    const int s1 = c_slot + 1 >= RING5_SLOTS ? c_slot + 1 - RING5_SLOTS : c_slot + 1;
    const int s2 = c_slot + 2 >= RING5_SLOTS ? c_slot + 2 - RING5_SLOTS : c_slot + 2;
    {
      // first half: multiply slab 2g, fetch the fragments of slab 2g+1, and
      // issue the slab that the previous hand-over left for later
      const IRIS_LDS char* sA = lds + s1 * Cfg::STAGE + a_lane;
      const IRIS_LDS char* sB = lds + s1 * Cfg::STAGE + b_lane;
#pragma unroll
      for (int i = 0; i < Cfg::IM; ++i) {
        mma_row<Cfg, FIRST>(acc, fr, 0, i);
        fr.a[i] = load_a<Cfg>(sA, i);
        load_b_share<Cfg>(sB, i, fr.b[1]);
        if (i % 2 == 1) issue_load(i / 2);
        __builtin_amdgcn_sched_barrier(0);
      }
      advance_load_cursor();
    }
    {
      // second half: multiply slab 2g+1; after its first block, hand over
      mma_row<Cfg, false>(acc, fr, 1, 0);
      __builtin_amdgcn_sched_barrier(0);
      // this wave's reads of slabs 2g and 2g+1 have returned
      IRIS_WAIT_LGKMCNT0();
      // slabs 2g+2 and 2g+3 have landed once only the slab issued during the
      // first half (and, behind a tile's end, the tile's stores before it)
      // is still outstanding
      const int pend = __builtin_amdgcn_readfirstlane(pending_tile);
      const int skip = __builtin_amdgcn_readfirstlane(pending_skip);
      if (pend >= 0 && skip != 0) {
        IRIS_WAIT_VMCNT(FAST_STORES + L);
      } else {
        IRIS_WAIT_VMCNT(L);
      }
      block_barrier_raw();
      if (pend >= 0) {
        if (skip == 0) {
          if (tid == 0) publish_tile(p, pend);
          pending_tile = -1;
        } else {
          pending_skip = 0;
        }
      }
      const IRIS_LDS char* sA = lds + s2 * Cfg::STAGE + a_lane;
      const IRIS_LDS char* sB = lds + s2 * Cfg::STAGE + b_lane;
      fr.a[0] = load_a<Cfg>(sA, 0);
      load_b_share<Cfg>(sB, 0, fr.b[0]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 1; i < Cfg::IM; ++i) {
        mma_row<Cfg, false>(acc, fr, 1, i);
        fr.a[i] = load_a<Cfg>(sA, i);
        load_b_share<Cfg>(sB, i, fr.b[0]);
        // the slot of slab 2g is free: the slab that the next hand-over needs goes out now
        if (i - 1 < L) issue_load(i - 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      advance_load_cursor();
    }
    c_slot = s2;
  };

  const int steps = nh / 2;
  for (int it = 0; it < n_items; ++it) {
    if (p.ts_begin && tid == 0)
      __hip_atomic_fetch_min((IRIS_GLOBAL unsigned long long*)(p.ts_begin + c_it.tile_id),
                             (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    step(std::true_type{});
    for (int k = 1; k < steps; ++k) step(std::false_type{});
    epilogue();
  }
  IRIS_WAIT_VMCNT(0);  // no load may still be writing this group's LDS when it exits
  if (pending_tile >= 0) {
    __syncthreads();
    if (tid == 0) publish_tile(p, pending_tile);
  }
}

}  // namespace iris_amd
