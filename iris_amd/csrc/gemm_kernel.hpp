// Persistent shard GEMM for gfx950 (MI355X) with the three tile-publishing
// epilogues.  One workgroup per CU walks its tiles
// `for tile_id in range(pid, total_tiles, NUM_SMS)`
// (examples/09_gemm_one_shot_all_reduce/gemm_one_shot_all_reduce.py:150) and,
// for every tile, runs the K loop of :174-195 on the matrix cores:
//
//   * A[M,K] and B[K,N] are both K-contiguous.  A CM x BK slab of A and a
//     CN x BK slab of B are copied HBM -> LDS with `buffer_load ... lds`
//     (16 bytes per lane, no register staging) into an S-deep ring of stages.
//     The ring is fed S-1 K-steps ahead and runs *across* tile boundaries, so
//     the next tile's first slabs are already in flight during an epilogue.
//   * LDS holds each slab row-major with the 16-byte chunks of a row XOR-ed
//     by the row index so that the `ds_read_b128` operand fetches of one MFMA
//     are bank-conflict free.
//   * v_mfma_f32_16x16x32 (bf16 or f16) with fp32 accumulators; operands are
//     swapped (B rows as SrcA, A rows as SrcB) so that a lane ends up with 4
//     consecutive columns of one output row.  Under the board's power limit
//     this shape sustains ~14% more than 32x32x16 on random operands
//     (measured: 1.91 vs 1.68 PFLOP/s for a register-only MFMA loop).
//   * Operand fragments are fetched from LDS one K-substep (32 k) ahead of
//     the MFMAs that use them: an A fragment's register is refilled right
//     after its last MFMA of the substep, B fragments are double-buffered.
//     The barrier that hands over the next stage sits inside a step's MFMA
//     stream, so neither LDS latency nor the barrier is paid with idle
//     matrix cores.
//   * The four-wave tiles run with four more waves, one per SIMD, that only
//     issue the stage loads and wait for them (GemmCfg::LW): a wave that is
//     held up at the issue of a load multiplies nothing meanwhile, and with
//     one wave per SIMD a K-step then costs fetch plus multiply instead of
//     the longer of the two.  All waves run the same control flow and meet
//     at the same barriers; only the work is told apart.
//   * The epilogue transposes the accumulators through a wave-private LDS
//     scratch so that global stores / atomics cover contiguous row segments.
//     Stores are write-through at the flags' scope; once they have completed
//     nothing is left in L2 for a release to write back, and a tile's flag is
//     published with a relaxed atomic.
//
// The logical tile (BLOCK_SIZE_M x BLOCK_SIZE_N, which fixes tile ids and
// flags) may be larger than the compute tile (CM x CN); a logical tile is
// then covered by several compute tiles and published once.
#pragma once

#include <type_traits>

#include "common.hpp"

namespace iris_amd {

constexpr int FLAG_MODE_MASK = 3, FLAG_RELEASE = 4;

struct GemmKArgs {
  const char* a;
  const char* b;
  char* out;  // c (ONE_SHOT producer) or c_global, already at its column offset
  int32_t* flags;
  const uint64_t* heap_bases;
  int64_t* ts_begin;
  int64_t* ts_end;
  int64_t sam, sak, sbk, sbn;  // A/B strides, elements
  int64_t som, son;            // strides of `out`, elements
  int M, N, K;
  int BM, BN, G;
  int num_sms, num_xcds, cur_rank, ws;
  // > 0: fewer work items than programs.  The reference remap would leave
  // whole XCDs idle then; instead each XCD takes xcd_per consecutive items
  // (neighbouring tiles, whose operand panels its L2 then fetches once).
  int xcd_per;
  int num_pid_m, num_pid_n, total_tiles;
  int sub_m, sub_n;  // compute tiles per logical tile
  // the launch's divisors, for the tile decode (see FastDiv)
  TileDivs tile_divs;
  FastDiv div_subs, div_sub_n;  // sub_m * sub_n, sub_n
  FastDiv div_split, div_nk;    // split_k; K-steps of a tile (stream-K runs)
  int dest_all;      // write `out` on every rank's heap (else on this rank only)
  // bits 1:0 -- 0: none, 1: +1 on every rank, 2: +1 on every other rank;  bit 2 (FLAG_RELEASE): the +1 is a
  // release at the flags' scope, as the reference's sem="release" (else relaxed, behind write-through stores)
  int flag_mode;
  int sys;           // flag atomics at system scope (else agent)
  int vec_out;       // 16-byte vector access allowed on `out`
  // > 0 (split-K launches with long parts; the value is total_tiles): the programs are numbered part by part
  // rather than tile by tile, so that an XCD's programs walk the same range of K over neighbouring tiles and
  // its L2 fetches each operand panel of that range once.  (Tile by tile, every program of an XCD walks a
  // different range and nothing is shared: the operands then come from HBM once per tile.)
  int part_major;
  // The launch covers tiles tile_base .. tile_base + total_tiles - 1 of the num_pid_m x num_pid_n grid.  Only the
  // split-K builds read it: a GEMM whose last round of tiles is split over the idle programs is an unsplit launch
  // from tile 0 and a split one from tile_base.  (The unsplit 256 x 256 kernel with one more scalar live across
  // its K loop ran 1.6 % slower on the headline shape.)
  int tile_base;
  // Split-K: a tile's K-steps are shared out over `split_k` programs.  Part 0
  // owns the tile: the others leave their fp32 accumulators in `partials`
  // (slot = global item index, `partial_stride` floats apart) and raise
  // `locks[slot]`; the owner adds them in part order and runs the epilogue.
  int split_k;  // >= 1
  int split_q, split_r;  // K-steps per part: nk / split_k and nk % split_k (the first split_r parts take one more)
  // Stream-K (with split_k == 1): the launch's total_tiles * nk K-steps, in
  // tile order, are cut into num_sms equal runs, split_q steps each and one
  // more for the first split_r programs; a run starts and ends anywhere in a
  // tile.  The program whose run holds a tile's first step owns the tile; the
  // programs that follow it hold the rest and hand it over through
  // partials[program] / locks[program] as split-K parts do.
  int stream_k;
  // Split-K with the sliced hand-over (split_k > 1 only): every part, the
  // first included, leaves its partial tile in `partials` as a row-major
  // fp32 matrix and raises locks[first slot]; once all have, part q sums rows
  // [q CM / split_k, (q + 1) CM / split_k) over the parts in part order and
  // runs the epilogue on them, so that no program does a whole tile's worth
  // of serial work; locks[first slot + 1] counts the parts that are done, and
  // the last one publishes the tile and re-arms both counters.
  int sliced;  // 1: as above; 2 (two parts only): each part keeps the half of the waves it owns, see dump_half
  float* partials;
  int32_t* locks;
  int64_t partial_stride;
  uint32_t* status;   // optional: IRIS_STATUS_SPIN_TIMEOUT when a wait for a partial or a tile flag gave up
  uint64_t timeout;   // bound of that wait, 100 MHz ticks
  // One-shot epilogue inside the program (the FUSED build of the kernel): once
  // a tile's partial is stored and signalled, the program waits for the
  // tile's flag on its own rank, sums the tile over all ranks' `out` buffers
  // and stores the result to `cg`.
  char* cg;
  int64_t sgm, sgn;  // strides of `cg`, elements
  int cg_dt;         // element type of `cg`
  int fused_vec;     // 16-byte strips allowed on `out` and `cg` in the in-program reduce

  // (Last, and the two fields of the split-K builds above among theirs: nothing the unsplit kernels read has
  // moved for them.  The unsplit 256 x 256 kernel is sensitive to where its arguments lie.)
  // merge_m * merge_n > 1: the launch's tiles (BM, BN, num_pid_m, num_pid_n, tile ids above) are merge_m x
  // merge_n of the caller's tiles; the flags stay the caller's, one per tile of BM / merge_m x BN / merge_n,
  // numbered over flag_num_pid_m x flag_num_pid_n tiles
  int merge_m, merge_n, flag_num_pid_m, flag_num_pid_n;

  // L2 prefetch hints (the 256 x 64 tile with fetching waves; 0: none).  The CUs of an XCD that work on one row of tiles
  // share its A panel, those on one column of tiles its B panel, and a line that the first of them asks for comes
  // from HBM while the others wait on the same miss.  With pf_dist > 0 a multiplying wave touches, every K-step,
  // one dword of its share of the lines that step k + pf_dist will need (every pf_sa-th row of A, every pf_sb-th
  // of B: the launch's tiles per XCD in either direction), so that the stage loads find them in L2.  Nothing
  // depends on the loaded values.
  // The touching build of the eight-wave 256 x 256 tile (GemmCfg::TOUCH) reads the same three: its touches are
  // issued by every wave, last in a K-step, for the step pf_dist beyond the load cursor (see Loader::touch), and
  // the shares are powers of two there.
  int pf_dist, pf_sa, pf_sb;
  // (MERGED builds) the launch covers the caller's columns of tiles from this one on: its flags sit that many
  // columns to the right in the caller's grid of flag_num_pid_m x flag_num_pid_n tiles
  int flag_pn_base;
  // Staggered start (the unsplit eight-wave 256 x 256 tile; 0: none).  The CUs of an XCD that finish their tiles
  // together send their 128 KiB of output stores each at the same moment, and a store that finds the XCD's write
  // path full holds its wave at issue, with the next tile's first MFMAs behind it.  With stagger_groups > 1 the
  // programs of an XCD start in that many groups, stagger_sleeps * 576 clocks apart, and stay that far apart for
  // the whole launch (they all do the same work): two groups 2 us apart take 3 % off the headline launch on zeros
  // and 1.5 % on data, the 2 us that the later group ends after the first included.
  int stagger_groups, stagger_sleeps;
};

template <int DT>
struct Mfma;
template <>
struct Mfma<IRIS_DTYPE_BF16> {
  using vec8 = bf16x8;
  __device__ static inline f32x4 run(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma<IRIS_DTYPE_F16> {
  using vec8 = f16x8;
  __device__ static inline f32x4 run(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

// fp32 operands.  The launcher hands such a launch over with K and the operands' strides counted in 16-bit units
// (two to an element), so that slabs, stages and loaders are the 16-bit kernels' byte for byte: a 16-byte chunk of a
// slab row holds four elements where it held eight.  A lane's fragment of a 32-unit substep is then four
// consecutive k of its row, and the substep's product is four v_mfma_f32_16x16x4_f32, the e-th over the lanes' e-th
// elements: lane group g contributes k = 4 g + e, so the four cover the substep's sixteen k once each (operands A
// and B pair up the same way, which is all a sum over k asks for).
template <>
struct Mfma<IRIS_DTYPE_F32> {
  using vec8 = f32x4;
  __device__ static inline f32x4 run(vec8 a, vec8 b, f32x4 c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
};

// LW_: waves that only fetch.  With one wave per SIMD a wave that is held up
// at the issue of a load (the memory pipeline takes a wave's loads at the
// rate it delivers them) runs no MFMA meanwhile, and the K loop costs the sum
// of fetch and multiply time.  LW_ = 4 adds one wave per SIMD that does
// nothing but issue the stage loads and wait for them; the WM x WN waves then
// issue no memory instruction in the K loop.
template <int DT_, int CM_, int CN_, int BK_, int WM_, int WN_, int S_, bool DMA_, int LW_ = 0, bool TOUCH_ = false>
struct GemmCfg {
  static constexpr int DT = DT_, CM = CM_, CN = CN_, BK = BK_, WM = WM_, WN = WN_, S = S_;
  static constexpr bool DMA = DMA_;
  static constexpr int NW = WM * WN, NT = NW * 64;  // the waves (threads) that multiply and store
  static constexpr int LW = LW_;
  static constexpr int NL = LW ? LW : NW;           // the waves that fetch
  // TOUCH_: a build of the eight-wave 256 x 256 tile that touches lines of K-steps to come (see Loader::touch)
  static constexpr bool TOUCH = TOUCH_;
  static_assert(!TOUCH_ || (DMA_ && LW_ == 0 && WM_ * WN_ == 8 && CM_ == 256 && CN_ == 256), "the touching build's tile");
  static constexpr int THREADS = (NW + LW) * 64;    // launch size
  static constexpr int TM = CM / WM, TN = CN / WN;
  static constexpr int IM = TM / 16, IN = TN / 16;  // 16x16 MFMA blocks of the wave tile
  static constexpr int CPR = BK / 8;    // 16-byte chunks per slab row
  static constexpr int RP = 16 / CPR;   // slab rows per 256 bytes
  static constexpr int RPB = 64 / CPR;  // slab rows per 1 KiB block (one wave-wide DMA)
  static constexpr int A_BYTES = CM * BK * 2, B_BYTES = CN * BK * 2;
  static constexpr int STAGE = A_BYTES + B_BYTES;
  static constexpr int A_LOADS = CM * CPR / (NL * 64), B_LOADS = CN * CPR / (NL * 64);
  static constexpr int L = A_LOADS + B_LOADS;  // loads of a fetching wave per stage
  static constexpr int KSUB = BK / 32;  // K-substeps (one MFMA depth) per stage
  // Every LDS-DMA tile with two substeps a stage has a split-K build.  In the
  // tiles with at most 64 accumulator registers a lane the first part of a tile
  // can add the other parts' partials to its accumulators (which is also how
  // stream-K runs hand over); the 128x64 wave tiles have no registers to spare
  // for that exchange and only take the sliced hand-over, in which a part's
  // accumulators are dead once its partial is written.
  static constexpr bool SPLITK = DMA_ && KSUB % 2 == 0 && IM * IN * 4 <= 128;
  static constexpr bool SPLIT_OWNER = SPLITK && IM * IN * 4 <= 64;
  // Waves per SIMD the register budget is sized for: 256 registers a wave.
  static constexpr int WPE = 2;
  // wave-private epilogue scratch: 32 rows x TN 16-bit elements
  static constexpr int WS_PITCH = TN * 2;
  static constexpr int WS_BYTES = 32 * WS_PITCH;
  static constexpr int U16 = TN / 8;       // 16-byte units per scratch row
  static constexpr int ERPB = 128 / TN;    // scratch rows per 256 bytes
  static constexpr int LDS_BYTES = S * STAGE + NW * WS_BYTES;
  static_assert(CM % (WM * 32) == 0 && CN % (WN * 32) == 0, "wave tile must be a multiple of 32x32");
  static_assert(BK == 32 || BK == 64 || BK == 128, "BK");
  static_assert((CM * CPR) % (NL * 64) == 0 && (CN * CPR) % (NL * 64) == 0, "slab must split evenly over lanes");
  static_assert(LW == 0 || (DMA && NW + LW <= 8), "fetching waves: LDS-DMA tiles of at most eight waves in all");
  static_assert(A_LOADS >= 1 && B_LOADS >= 1, "too many waves for this slab");
  static constexpr bool S_POW2 = (S & (S - 1)) == 0;  // (else the ring slot is counted along instead of masked out of g)
  static_assert(S >= 1, "ring depth");
  static_assert(!DMA || S >= 2, "the DMA ring needs a stage being read and one in flight");
  static_assert(L * (S - 1) <= 63, "vmcnt immediate");
  static_assert(IM * IN * 4 <= 128, "accumulators of a wave tile: at most 128 registers (two waves a SIMD)");
  static_assert(TN == 32 || TN == 64 || TN == 128, "wave tile width");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

// One compute tile of work.
struct Item {
  int tile_id;
  int m0, n0;        // origin of the compute tile
  int m_end, n_end;  // exclusive bounds (logical tile clipped to M, N)
  int lm0, ln0;      // origin of the logical tile
  bool last_sub;     // last compute tile of its logical tile
  bool first_sub;
};

// Split-K: item `item` of program `pid` is part `part` of tile `slot / split_k`
// and covers K-steps [k_begin, k_end).  Kept out of Item: these live in
// scalar registers across the K loop only where they are needed.
// part 0 owns the tile: its partial-sum slot is `slot`, and the other parts
// leave theirs in the slots that follow (their own `slot`).
struct KRange {
  int k_begin, k_end, part, slot;
};
// Stream-K: a program's run of global K-steps [g0, g1) starts at step k0 of
// tile `tile0`.  Computed once per program (it takes a division).
struct StreamRun {
  int tile0, k0, g1;
};
__host__ __device__ inline int stream_len(const GemmKArgs& p, int pid) { return p.split_q + (pid < p.split_r ? 1 : 0); }
__host__ __device__ inline StreamRun stream_run(const GemmKArgs& p, int pid, int nk) {
  StreamRun r;
  const int g0 = pid * p.split_q + (pid < p.split_r ? pid : p.split_r);
  r.g1 = g0 + stream_len(p, pid);
  r.tile0 = nk > 0 ? (int)fast_div((uint32_t)g0, p.div_nk) : 0;
  r.k0 = g0 - r.tile0 * nk;
  return r;
}
// Items (tiles touched) of the run.
__host__ __device__ inline int stream_items(const StreamRun& r, int nk) {
  return r.g1 > r.tile0 * nk + r.k0 ? (r.g1 - 1) / nk - r.tile0 + 1 : 0;
}
// Parts of a tile whose owner, program `pid`, stops at step k_end: itself and
// the programs that hold the rest (each run is at least one step long).
__host__ __device__ inline int stream_parts(const GemmKArgs& p, int pid, int k_end, int nk) {
  int parts = 1;
  for (int rem = nk - k_end, q = pid + 1; rem > 0; ++q, ++parts) rem -= stream_len(p, q);
  return parts;
}
// Split-K proper is the same thing with runs that never cross a tile: program
// pid is part pid % split_k of tile pid / split_k (one item per program).
__device__ inline StreamRun split_run(const GemmKArgs& p, int pid, int nk) {
  StreamRun r;
  r.tile0 = (int)fast_div((uint32_t)pid, p.div_split);
  const int part = pid - r.tile0 * p.split_k;
  r.k0 = part * p.split_q + min(part, p.split_r);
  r.g1 = r.tile0 * nk + r.k0 + (r.tile0 < p.total_tiles ? p.split_q + (part < p.split_r ? 1 : 0) : 0);
  return r;
}
template <class Cfg, bool SPLIT>
__device__ inline KRange k_range(const GemmKArgs& p, const StreamRun& sr, int pid, int item, int nk) {
  KRange r;
  if constexpr (SPLIT) {
    r.k_begin = item == 0 ? sr.k0 : 0;
    r.k_end = min(nk, sr.g1 - (sr.tile0 + item) * nk);
    r.part = r.k_begin == 0 ? 0 : 1;
    r.slot = pid;
  } else {
    r.slot = 0;
    r.part = 0;
    r.k_begin = 0;
    r.k_end = nk;
  }
  return r;
}

template <class Cfg, bool SPLIT>
__device__ inline Item decode_item(const GemmKArgs& p, const StreamRun& sr, int pid, int item) {
  const int subs = p.sub_m * p.sub_n;
  Item it;
  if constexpr (SPLIT) {
    // one compute tile per logical tile; the program's run touches tiles
    // tile0, tile0 + 1, ...
    it.tile_id = p.tile_base + sr.tile0 + item;
    const TileCoord tc = tile_map_fast(it.tile_id, p.num_pid_m, p.num_pid_n, p.G, p.tile_divs);
    it.lm0 = it.m0 = tc.pid_m * p.BM;
    it.ln0 = it.n0 = tc.pid_n * p.BN;
    it.m_end = min(p.M, it.lm0 + p.BM);
    it.n_end = min(p.N, it.ln0 + p.BN);
    it.first_sub = it.last_sub = true;
    return it;
  }
  const int ti = (int)fast_div((uint32_t)item, p.div_subs);
  const int s = item - ti * subs;
  it.tile_id = pid + ti * p.num_sms;  // (the unsplit builds only run launches whose tile_base is 0)
  const TileCoord tc = tile_map_fast(it.tile_id, p.num_pid_m, p.num_pid_n, p.G, p.tile_divs);
  it.lm0 = tc.pid_m * p.BM;
  it.ln0 = tc.pid_n * p.BN;
  const int sm = (int)fast_div((uint32_t)s, p.div_sub_n), sn = s - sm * p.sub_n;
  it.m0 = it.lm0 + sm * Cfg::CM;
  it.n0 = it.ln0 + sn * Cfg::CN;
  it.m_end = min(p.M, it.lm0 + p.BM);
  it.n_end = min(p.N, it.ln0 + p.BN);
  it.first_sub = (s == 0);
  it.last_sub = (s == subs - 1);
  return it;
}

// `ptr` as seen on rank r's heap (identity for the caller's own rank).
template <typename P>
__device__ inline IRIS_GLOBAL P* rank_ptr(const GemmKArgs& p, P* ptr, int r) {
  if (r == p.cur_rank || p.heap_bases == nullptr) return (IRIS_GLOBAL P*)ptr;
  // r and the bases are the same for the whole wave and the table does not
  // change while the kernel runs: scalar loads, which do not wait for stores
  const __attribute__((address_space(4))) uint64_t* hb =
      (const __attribute__((address_space(4))) uint64_t*)p.heap_bases;
  return translate(ptr, uniform_u64(hb[p.cur_rank]), uniform_u64(hb[r]));
}

// ---------------------------------------------------------------------------
// Slab loader
// ---------------------------------------------------------------------------

// Per-item loader state.  Lane `lane` of fetching wave `wave` (of NL) fetches,
// for load `i`, the 16-byte chunk that lands at byte  blk*1024 + lane*16  of
// the slab, blk = i*NL + wave.  That position is (row, physical chunk); the chunk of the
// row it must hold is  pc ^ ((row / RP) % CPR).
template <class Cfg>
struct Loader {
  __amdgpu_buffer_rsrc_t ra, rb;
  // Byte offset, at k0 == 0, of the 16-byte chunk this lane fetches with the
  // first A load and the first B load of a slab; load i of an operand is
  // i * NL * RPB rows further down (step_a / step_b bytes).  Rows below the
  // matrix edge lie past the end of the buffer descriptor and read as zero.
  // For the one K-step that can hold chunks past K, the K loop's last, the
  // offsets of those lanes are parked out of range when the load cursor
  // reaches the step (the masked tail of gemm_*:186-195), so the K-steps
  // issue their loads without any per-load arithmetic but one add.
  uint32_t va, vb;
  int step_a, step_b;
  int k_limit;  // K
  // (Cfg::TOUCH) byte offset of the row whose line this lane touches ahead of the loads, out of range for none
  uint32_t ta, tb;

  // The chunk of the row that a lane fetches is the same for every load:
  // the swizzle period divides the rows between two loads of a wave.
  static_assert((Cfg::NL * Cfg::RPB / Cfg::RP) % Cfg::CPR == 0, "the lane's chunk must not depend on the load");
  // first k of the chunk that this lane fetches at k0 == 0
  __device__ static inline int chunk_k(int wave, int lane) {
    const int row = wave * Cfg::RPB + lane / Cfg::CPR;
    return ((lane % Cfg::CPR) ^ ((row / Cfg::RP) % Cfg::CPR)) * 8;
  }

  // Offsets for the item's first step to be loaded, `k`.
  __device__ inline void setup(const GemmKArgs& p, const Item& it, int wave, int lane, int k) {
    // a tile that starts past the matrix edge (a masked sub-tile) reads nothing
    const int m0c = min(it.m0, p.M - 1), n0c = min(it.n0, p.N - 1);
    const int rows_a = it.m0 < p.M ? min(Cfg::CM, p.M - it.m0) : 0, rows_b = it.n0 < p.N ? min(Cfg::CN, p.N - it.n0) : 0;
    const char* abase = p.a + (int64_t)m0c * p.sam * 2;
    const char* bbase = p.b + (int64_t)n0c * p.sbn * 2;
    const uint32_t arec = rows_a > 0 ? (uint32_t)(((int64_t)(rows_a - 1) * p.sam + p.K) * 2) : 0;
    const uint32_t brec = rows_b > 0 ? (uint32_t)(((int64_t)(rows_b - 1) * p.sbn + p.K) * 2) : 0;
    ra = __builtin_amdgcn_make_buffer_rsrc((void*)abase, 0, arec, 0x00020000);
    rb = __builtin_amdgcn_make_buffer_rsrc((void*)bbase, 0, brec, 0x00020000);
    k_limit = p.K;
    const int row = wave * Cfg::RPB + lane / Cfg::CPR, ck = chunk_k(wave, lane);
    va = (uint32_t)(((int64_t)row * p.sam + ck) * 2);
    vb = (uint32_t)(((int64_t)row * p.sbn + ck) * 2);
    step_a = (int)((int64_t)Cfg::NL * Cfg::RPB * p.sam * 2);
    step_b = (int)((int64_t)Cfg::NL * Cfg::RPB * p.sbn * 2);
    if constexpr (Cfg::TOUCH) {
      // this program's share of the panels' rows: `first`, `first + share`, ... (the shares are powers of two)
      const int q = wave * 64 + lane;
      const int row_a = ((it.n0 / Cfg::CN) & (p.pf_sa - 1)) + p.pf_sa * q;
      const int row_b = ((it.m0 / Cfg::CM) & (p.pf_sb - 1)) + p.pf_sb * q;
      ta = row_a < rows_a ? (uint32_t)((int64_t)row_a * p.sam * 2) : 0x80000000u;
      tb = row_b < rows_b ? (uint32_t)((int64_t)row_b * p.sbn * 2) : 0x80000000u;
    }
    before_step(k, wave, lane);
  }
  // Touch, with one dword per lane, this program's share of the lines of K-step `k`, so that they are on their way
  // from HBM into the XCD's L2 before the stage loads of that step ask for them.  Two loads, one per operand,
  // always issued (a lane without a row holds an offset out of range), so that the waits that follow count the
  // same in every wave.  Loads return in order: the K-step issues them after its stage loads, and the next
  // hand-over leaves exactly these two in flight.  The dwords land in `scratch` (LDS that nothing reads inside a
  // K loop), not in a register, which the compiler would hand on before the load has returned.
  __device__ inline void touch(IRIS_LDS char* scratch, int k) const {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (IRIS_LDS void*)scratch, 4, ta, k * Cfg::BK * 2, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (IRIS_LDS void*)scratch, 4, tb, k * Cfg::BK * 2, 0, 0);
  }
  // The load cursor is about to load step `k`: park the chunks past K.
  __device__ inline void before_step(int k, int wave, int lane) {
    if (k_limit - k * Cfg::BK >= Cfg::BK) return;  // a full step: nothing to mask
    if (k * Cfg::BK + chunk_k(wave, lane) >= k_limit) va = vb = 0x80000000u;
  }
  // The program has no more steps to load: the loads are still issued, so
  // that every K-step keeps the same number of loads in flight, but fetch
  // nothing.
  __device__ inline void park() {
    va = vb = 0x80000000u;
    if constexpr (Cfg::TOUCH) ta = tb = 0x80000000u;
  }

  // Issue load `i` of K-step `k` into the stage at LDS address `stage`.  The
  // K offset rides in the scalar offset.
  __device__ inline void issue_at(const GemmKArgs& p, IRIS_LDS char* stage, int k, int wave, int i) const {
    const bool isA = i < Cfg::A_LOADS;
    const int j = isA ? i : i - Cfg::A_LOADS;
    const int k0 = k * Cfg::BK;
    IRIS_LDS char* dst = stage + (isA ? 0 : Cfg::A_BYTES) + (j * Cfg::NL + wave) * 1024;
    // (a parked offset stays out of range: j * step is far below 2 GiB)
    const uint32_t off = isA ? va + (uint32_t)(j * step_a) : vb + (uint32_t)(j * step_b);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(isA ? ra : rb, (IRIS_LDS void*)dst, 16, off, k0 * 2, 0, 0);
  }
  template <int I = 0>
  __device__ inline void issue(const GemmKArgs& p, IRIS_LDS char* stage, int k, int wave) const {
    if constexpr (I < Cfg::L) {
      issue_at(p, stage, k, wave, I);
      issue<I + 1>(p, stage, k, wave);
    }
  }
};

// Generic loader: any strides / alignment, element by element, synchronous.
// It writes the same slab layout.
template <class Cfg>
__device__ inline void load_slab_generic(const GemmKArgs& p, const Item& it, IRIS_LDS char* stage, int k,
                                         int tid) {
  const int k0 = k * Cfg::BK;
  const IRIS_GLOBAL unsigned short* A = (const IRIS_GLOBAL unsigned short*)p.a;
  const IRIS_GLOBAL unsigned short* B = (const IRIS_GLOBAL unsigned short*)p.b;
  for (int idx = tid; idx < (Cfg::CM + Cfg::CN) * Cfg::CPR; idx += Cfg::NT) {
    const bool isA = idx < Cfg::CM * Cfg::CPR;
    const int pos = isA ? idx : idx - Cfg::CM * Cfg::CPR;
    const int row = pos / Cfg::CPR, pc = pos % Cfg::CPR;
    const int ch = pc ^ ((row / Cfg::RP) % Cfg::CPR);
    u32x4 v;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      unsigned int w = 0;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int kk = k0 + ch * 8 + e * 2 + h;
        unsigned short x = 0;
        if (kk < p.K) {
          // (fp32 operands: 16-bit unit kk is half kk & 1 of element kk / 2, and the strides count units)
          const int64_t ke = Cfg::DT == IRIS_DTYPE_F32 ? kk >> 1 : kk, half = Cfg::DT == IRIS_DTYPE_F32 ? kk & 1 : 0;
          if (isA) {
            const int r = min(it.m0 + row, p.M - 1);
            x = A[(int64_t)r * p.sam + ke * p.sak + half];
          } else {
            const int r = min(it.n0 + row, p.N - 1);
            x = B[(int64_t)r * p.sbn + ke * p.sbk + half];
          }
        }
        w |= ((unsigned int)x) << (16 * h);
      }
      v[e] = w;
    }
    *reinterpret_cast<IRIS_LDS u32x4*>(stage + (isA ? 0 : Cfg::A_BYTES) + pos * 16) = v;
  }
}

// ---------------------------------------------------------------------------
// MFMA over one stage
// ---------------------------------------------------------------------------

// Operand fragments of a wave: one 16-row x 32-k block each (16 bytes a
// lane).  `a` holds the substep in use and is refilled block by block for the
// next one; `b` is double-buffered because every A block needs all of it.
template <class Cfg>
struct Frags {
  typename Mfma<Cfg::DT>::vec8 a[Cfg::IM], b[2][Cfg::IN];
};

template <class Cfg>
__device__ inline typename Mfma<Cfg::DT>::vec8 load_a(const IRIS_LDS char* sA, int i) {
  return *reinterpret_cast<const IRIS_LDS typename Mfma<Cfg::DT>::vec8*>(sA + i * 16 * Cfg::BK * 2);
}
template <class Cfg>
__device__ inline typename Mfma<Cfg::DT>::vec8 load_b(const IRIS_LDS char* sB, int j) {
  return *reinterpret_cast<const IRIS_LDS typename Mfma<Cfg::DT>::vec8*>(sB + j * 16 * Cfg::BK * 2);
}

// B fragments fetched next to A block i, so that all IN of them are spread
// over the IM blocks of a substep.
template <class Cfg>
__device__ inline void load_b_share(const IRIS_LDS char* sB, int i, typename Mfma<Cfg::DT>::vec8 (&b)[Cfg::IN]) {
  constexpr int PER = (Cfg::IN + Cfg::IM - 1) / Cfg::IM;
#pragma unroll
  for (int j = i * PER; j < (i + 1) * PER; ++j)
    if (j < Cfg::IN) b[j] = load_b<Cfg>(sB, j);
}

// Whole substep's fragments at once (pipeline prologue, generic loader).
template <class Cfg>
__device__ inline void load_all(const IRIS_LDS char* sA, const IRIS_LDS char* sB, Frags<Cfg>& f, int cb) {
#pragma unroll
  for (int j = 0; j < Cfg::IN; ++j) f.b[cb][j] = load_b<Cfg>(sB, j);
#pragma unroll
  for (int i = 0; i < Cfg::IM; ++i) f.a[i] = load_a<Cfg>(sA, i);
}

// acc[i][*] (+)= B fragments x A fragment i: the IN MFMAs of one 16-row block.
// FIRST: the block's first product of a tile, which defines the accumulator.
template <class Cfg, bool FIRST>
__device__ inline void mma_row(f32x4 (&acc)[Cfg::IM][Cfg::IN], const Frags<Cfg>& f, int cb, int i) {
#pragma unroll
  for (int j = 0; j < Cfg::IN; ++j) {
    if constexpr (FIRST) {
      const f32x4 z = {0, 0, 0, 0};
      acc[i][j] = Mfma<Cfg::DT>::run(f.b[cb][j], f.a[i], z);
    } else {
      acc[i][j] = Mfma<Cfg::DT>::run(f.b[cb][j], f.a[i], acc[i][j]);
    }
  }
}

// ---------------------------------------------------------------------------
// Epilogue
// ---------------------------------------------------------------------------

enum StoreOp { OP_STORE16 = 0, OP_STORE32 = 1, OP_ATOMIC32 = 2, OP_ATOMIC16 = 3 };

// 16-bit atomic add on `p` (element type DT) by CAS on the containing word.
template <int DT>
__device__ inline void atomic_add16_cas(IRIS_GLOBAL unsigned short* p, float v) {
  const uintptr_t addr = (uintptr_t)p;
  IRIS_GLOBAL unsigned int* w = (IRIS_GLOBAL unsigned int*)(addr & ~(uintptr_t)3);
  const int sh = (addr & 2) ? 16 : 0;
  unsigned int old = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  for (;;) {
    const unsigned short cur = (unsigned short)(old >> sh);
    const unsigned short nv = to16<DT>(from16<DT>(cur) + v);
    const unsigned int repl = (old & ~(0xFFFFu << sh)) | ((unsigned int)nv << sh);
    if (__hip_atomic_compare_exchange_strong(w, &old, repl, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT))
      break;
  }
}

// Packed 2 x 16-bit atomic add on a 4-byte aligned pair.
template <int DT>
__device__ inline void atomic_add16_pair(IRIS_GLOBAL unsigned int* p, unsigned int v) {
  if constexpr (DT == IRIS_DTYPE_BF16) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    __builtin_amdgcn_global_atomic_fadd_v2bf16((IRIS_GLOBAL bf16x2*)p,
                                               __builtin_bit_cast(bf16x2, v));
  } else {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    __builtin_amdgcn_global_atomic_fadd_v2f16((IRIS_GLOBAL f16x2*)p,
                                              __builtin_bit_cast(f16x2, v));
  }
}

// Write the wave's TM x TN accumulator block to `out` on the destination
// ranks, rows < m_end, columns < n_end, through the wave-private LDS scratch.
//
// Accumulator layout (operands swapped): for block (i, j), register r, lane l:
//   m = i*16 + l%16,   n = j*16 + 4*(l/16) + r.
//
// A pass moves 32 rows (two blocks) x CP columns: registers -> scratch (16-byte units of a
// row XOR-ed with the row index), then scratch -> memory with lanes running
// along a row so that one instruction covers contiguous bytes.
//
// OP_STORE16 : 16-bit elements of type ODT        OP_STORE32 : fp32 elements
// OP_ATOMIC32: fp32 atomic add                    OP_ATOMIC16: 16-bit atomic add
//
// Returns true when the wave issued exactly FAST_STORES memory instructions
// (every block took the 16-byte path to a single destination rank).
template <class Cfg, int OP>
struct StoreCount {
  static constexpr bool F32 = (OP == OP_STORE32 || OP == OP_ATOMIC32);
  static constexpr int NPASS = F32 ? 2 : 1;
  static constexpr int NV = 32 / (64 / Cfg::U16);
  static constexpr int FAST_STORES = (Cfg::TM / 32) * NPASS * NV;
};
template <class Cfg, int OP, int ODT>
__device__ __attribute__((always_inline)) inline bool store_acc(const GemmKArgs& p, const f32x4 (&acc)[Cfg::IM][Cfg::IN], IRIS_LDS char* ws,
                                 int wm0, int wn0, int m_end, int n_end, int lane) {  // lane: by value, see below
  constexpr bool F32 = (OP == OP_STORE32 || OP == OP_ATOMIC32);
  constexpr int ES = F32 ? 4 : 2;
  constexpr int CP = Cfg::WS_PITCH / ES;  // columns per pass
  constexpr int NPASS = Cfg::TN / CP;     // 1 (16-bit) or 2 (fp32)
  constexpr int NJ = CP / 16;             // 16-column accumulator blocks per pass
  constexpr int EPV = 16 / ES;            // elements per 16-byte unit
  // Everything below depends on the lane id.  It is made opaque here so that
  // the address arithmetic of the epilogue is computed in the epilogue and
  // not hoisted into registers that stay live across the K loop.
  asm volatile("" : "+v"(lane));
  const int lr = lane & 15, lq = lane >> 4;
  const int r_begin = p.dest_all ? 0 : p.cur_rank;
  const int r_end = p.dest_all ? p.ws : p.cur_rank + 1;
  bool all_fast = (OP == OP_STORE16 || OP == OP_STORE32) && p.vec_out && r_end - r_begin == 1;
  const bool single = r_end - r_begin == 1;
  IRIS_GLOBAL char* dst0 = rank_ptr(p, p.out, r_begin);
  // AUX: write-through at the flags' scope for the 16-byte stores, sc1 (agent)
  // or sc0 sc1 (system); chosen once, outside the loops
  auto blocks = [&](auto aux_tag) __attribute__((always_inline)) {
    constexpr int AUX = decltype(aux_tag)::value;
#pragma unroll
    for (int i = 0; i < Cfg::TM / 32; ++i) {
#pragma unroll
      for (int ps = 0; ps < NPASS; ++ps) {
        // ---- registers -> scratch
#pragma unroll
        for (int ib = 0; ib < 2; ++ib) {
          const int row = ib * 16 + lr;
          const int sw = (row / Cfg::ERPB) % Cfg::U16;
#pragma unroll
          for (int g = 0; g < NJ; ++g) {
            const f32x4 a4 = acc[i * 2 + ib][ps * NJ + g];
            if constexpr (F32) {
              const int u = (g * 4 + lq) ^ sw;
              *reinterpret_cast<IRIS_LDS f32x4*>(ws + row * Cfg::WS_PITCH + u * 16) = a4;
            } else {
              const int u = (g * 2 + (lq >> 1)) ^ sw;
              const u32x2 v = {pack2<ODT>(a4[0], a4[1]), pack2<ODT>(a4[2], a4[3])};
              *reinterpret_cast<IRIS_LDS u32x2*>(ws + row * Cfg::WS_PITCH + u * 16 + (lq & 1) * 8) = v;
            }
          }
        }
        // ---- scratch -> memory
        const int row0 = wm0 + i * 32, col0 = wn0 + ps * CP;
        const bool interior = (row0 + 32 <= m_end) && (col0 + CP <= n_end);
        // The 16-byte store path also takes ragged blocks whose valid columns
        // are whole 16-byte units: rows past m_end fall outside the block's
        // buffer descriptor and units past n_end are parked out of range.
        const int rows_ok = min(32, m_end - row0), cols_ok = min(CP, n_end - col0);
        const bool vec_block = (OP == OP_STORE16 || OP == OP_STORE32) && (cols_ok <= 0 || cols_ok % EPV == 0);
        all_fast = all_fast && (interior || vec_block);
#pragma nounroll
        for (int r = r_begin; r < r_end; ++r) {
          IRIS_GLOBAL char* dst = single ? dst0 : rank_ptr(p, p.out, r);
          if (OP == OP_ATOMIC32) {
            // one fp32 per lane, lanes along the row
            constexpr int ITER = 32 * CP / 64;
#pragma nounroll  // an atomic per iteration: nothing to gain, and unrolled address math spills
            for (int t = 0; t < ITER; ++t) {
              const int idx = t * 64 + lane;
              const int row = idx / CP, cc = idx % CP;
              const int u = (cc / 4) ^ ((row / Cfg::ERPB) % Cfg::U16);
              const float v =
                  *reinterpret_cast<const IRIS_LDS float*>(ws + row * Cfg::WS_PITCH + u * 16 + (cc % 4) * 4);
              const int m = row0 + row, n = col0 + cc;
              if (m < m_end && n < n_end)
                __hip_atomic_fetch_add((IRIS_GLOBAL float*)(dst + ((int64_t)m * p.som + (int64_t)n * p.son) * 4),
                                       v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
          } else if ((interior || vec_block) && p.vec_out) {
            if constexpr (OP == OP_ATOMIC16) {
              // one packed pair per lane, lanes along the row
              constexpr int ITER = 32 * (CP / 2) / 64;
#pragma nounroll
              for (int t = 0; t < ITER; ++t) {
                const int idx = t * 64 + lane;
                const int row = idx / (CP / 2), cc = (idx % (CP / 2)) * 2;
                const int u = (cc / 8) ^ ((row / Cfg::ERPB) % Cfg::U16);
                const unsigned int v =
                    *reinterpret_cast<const IRIS_LDS unsigned int*>(ws + row * Cfg::WS_PITCH + u * 16 + (cc % 8) * 2);
                const int m = row0 + row, n = col0 + cc;
                atomic_add16_pair<ODT>((IRIS_GLOBAL unsigned int*)(dst + ((int64_t)m * p.som + n) * 2), v);
              }
            } else {
              constexpr int RPI = 64 / Cfg::U16;  // rows per wave-wide 16-byte read
              constexpr int NV = 32 / RPI;
              // the 32 x CP block as a buffer: rows are p.som elements apart
              const bool any = rows_ok > 0 && cols_ok > 0;
              const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
                  (void*)(dst + ((int64_t)row0 * p.som + col0) * ES), 0,
                  any ? (int)(((rows_ok - 1) * p.som + cols_ok) * ES) : 0, 0x00020000);
              u32x4 v[NV];
              int off[NV];
#pragma unroll
              for (int t = 0; t < NV; ++t) {
                const int row = t * RPI + lane / Cfg::U16;
                const int u = lane % Cfg::U16;
                const int pu = u ^ ((row / Cfg::ERPB) % Cfg::U16);
                v[t] = *reinterpret_cast<const IRIS_LDS u32x4*>(ws + row * Cfg::WS_PITCH + pu * 16);
                off[t] = (u + 1) * EPV <= cols_ok ? (int)((row * p.som + u * EPV) * ES) : (int)0x80000000;
              }
#pragma unroll
              for (int t = 0; t < NV; ++t) __builtin_amdgcn_raw_buffer_store_b128(v[t], rs, off[t], 0, AUX);
            }
          } else {
            // ragged edge or unaligned destination: element by element
#pragma nounroll
            for (int idx = lane; idx < 32 * CP; idx += 64) {
              const int row = idx / CP, cc = idx % CP;
              const int u = (cc / EPV) ^ ((row / Cfg::ERPB) % Cfg::U16);
              const IRIS_LDS char* src = ws + row * Cfg::WS_PITCH + u * 16 + (cc % EPV) * ES;
              const int m = row0 + row, n = col0 + cc;
              if (m < m_end && n < n_end) {
                IRIS_GLOBAL char* d = dst + ((int64_t)m * p.som + (int64_t)n * p.son) * ES;
                if constexpr (OP == OP_STORE32)
                  store_through((IRIS_GLOBAL unsigned int*)d, *reinterpret_cast<const IRIS_LDS unsigned int*>(src),
                                p.sys != 0);
                else if constexpr (OP == OP_STORE16)
                  store_through((IRIS_GLOBAL unsigned short*)d,
                                *reinterpret_cast<const IRIS_LDS unsigned short*>(src), p.sys != 0);
                else
                  atomic_add16_cas<ODT>((IRIS_GLOBAL unsigned short*)d,
                                        from16<ODT>(*reinterpret_cast<const IRIS_LDS unsigned short*>(src)));
              }
            }
          }
        }
      }
    }
  };
  if ((OP == OP_STORE16 || OP == OP_STORE32) && p.sys)
    blocks(std::integral_constant<int, 17>{});
  else
    blocks(std::integral_constant<int, 16>{});
  return all_fast;
}

// Publish a finished logical tile: +1 on the tile's flag of every rank
// (flag_mode 1, the ready flag of the scatter epilogue) or of every *other*
// rank (flag_mode 2, the ONE_SHOT producer signal,
// gemm_one_shot_all_reduce.py:207-218, sem="release").  One wave calls it, all
// 64 lanes, after every wave of the group has waited for its stores of the
// tile to complete and the group has passed a barrier.  Those stores were
// write-through at the flag's scope, so they are already visible there and
// the increment itself can be relaxed: it is ordered after them by the waits.
// (This has been validated with producers and consumers on ONE device only; a
// launch may ask for the reference's release instead, FLAG_RELEASE.)
// Lane l takes ranks l, l + 64, ...: the ranks' heap bases come in with one
// vector load and the increments leave together (one thread walking the ranks
// waits for a scalar load per rank: 0.8 us for eight).
template <bool MERGED = false>
__device__ __attribute__((always_inline)) inline void publish_tile(const GemmKArgs& p, int tile_id, int lane) {
  // the caller's tiles the launch's tile covers: itself, or (the MERGED builds, which only run launches whose
  // tiles are blocks of the caller's) merge_m x merge_n of them, fewer at the edges.  A build of its own: the
  // unmerged 256 x 256 kernel with these four scalars live across its K loop ran 4 % slower.
  constexpr bool merged = MERGED;
  int first = tile_id, rows = 1, cols = 1, pm0 = 0, pn0 = 0;
  if constexpr (merged) {
    const TileCoord t = tile_map_fast(tile_id, p.num_pid_m, p.num_pid_n, p.G, p.tile_divs);
    pm0 = t.pid_m * p.merge_m;
    pn0 = t.pid_n * p.merge_n + p.flag_pn_base;
    rows = min(p.merge_m, p.flag_num_pid_m - pm0);
    cols = min(p.merge_n, p.flag_num_pid_n - pn0);
  }
  for (int i = 0; i < rows; ++i)
    for (int j = 0; j < cols; ++j) {
      if constexpr (merged) first = tile_id_of(pm0 + i, pn0 + j, p.flag_num_pid_m, p.flag_num_pid_n, p.G);
      IRIS_GLOBAL int32_t* own = (IRIS_GLOBAL int32_t*)(p.flags + first);
      for (int r = lane; r < p.ws; r += 64) {
        if ((p.flag_mode & FLAG_MODE_MASK) == 2 && r == p.cur_rank) continue;
        IRIS_GLOBAL int32_t* f = own;
        if (r != p.cur_rank && p.heap_bases != nullptr)
          f = translate(p.flags + first, p.heap_bases[p.cur_rank], p.heap_bases[r]);
        if (p.flag_mode & FLAG_RELEASE)
          flag_add_release(f, 1, p.sys != 0);  // gemm_one_shot_all_reduce.py:207-218 verbatim
        else
          flag_add_relaxed(f, 1, p.sys != 0);
      }
    }
}

// Split-K hand-over of a partial tile.  The partial keeps the accumulators'
// register order (block, thread, register): 16 bytes a lane, a wave writes or
// reads 1 KiB at a time, and nobody else needs to understand the layout.
template <class Cfg>
__device__ inline void dump_partial(const GemmKArgs& p, const f32x4 (&acc)[Cfg::IM][Cfg::IN], int slot, int tid) {
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.partials + (int64_t)slot * p.partial_stride), 0, Cfg::CM * Cfg::CN * 4, 0x00020000);
#pragma unroll
  for (int i = 0; i < Cfg::IM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::IN; ++j)
      // write-through to where every CU of the agent reads it
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][j]), rs,
                                             ((i * Cfg::IN + j) * Cfg::NT + tid) * 16, 0, 16);
}
// acc += partials of parts [q0, q0 + GROUP) of the tile whose part 0 is `slot0`,
// in part order; parts >= `parts` read as zero.  All loads of the group are in
// flight together.
template <class Cfg, int GROUP>
__device__ inline void add_partials(const GemmKArgs& p, f32x4 (&acc)[Cfg::IM][Cfg::IN], int slot0, int q0, int parts,
                                    int tid) {
  constexpr int NB = Cfg::IM * Cfg::IN;
  u32x4 v[GROUP][NB];
#pragma unroll
  for (int g = 0; g < GROUP; ++g) {
    const bool present = q0 + g < parts;
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)(p.partials + (int64_t)(slot0 + (present ? q0 + g : 0)) * p.partial_stride), 0,
        present ? Cfg::CM * Cfg::CN * 4 : 0, 0x00020000);
#pragma unroll
    for (int b = 0; b < NB; ++b)  // sc1: coherent at agent scope without a fence
      v[g][b] = __builtin_amdgcn_raw_buffer_load_b128(rs, (b * Cfg::NT + tid) * 16, 0, 16);
  }
#pragma unroll
  for (int g = 0; g < GROUP; ++g)
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b / Cfg::IN][b % Cfg::IN] += __builtin_bit_cast(f32x4, v[g][b]);
}

// Hand-over of a tile split in TWO parts: the first half of the multiplying waves belongs to part 0, the second
// half to part 1.  A part leaves the accumulators of the waves that are NOT its own in its slot, in register
// order (wave of the half, block, lane: 16 bytes a lane, 1 KiB a store), and each of its own waves adds what the
// other part left for the same wave and runs the epilogue on its wave tile.  Half a partial tile crosses memory
// per part, the other half never leaves its registers; p0 + p1 has the same bits whichever side adds.
template <class Cfg>
__device__ inline void dump_half(const GemmKArgs& p, const f32x4 (&acc)[Cfg::IM][Cfg::IN], int slot, int wv, int lane) {
  constexpr int NB = Cfg::IM * Cfg::IN;
  asm volatile("" : "+v"(lane));  // (offsets computed here, not kept in registers across the K loop)
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.partials + (int64_t)slot * p.partial_stride), 0, (Cfg::NW / 2) * NB * 1024, 0x00020000);
#pragma unroll
  for (int i = 0; i < Cfg::IM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::IN; ++j)
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][j]), rs,
                                             ((wv * NB + i * Cfg::IN + j) * 64 + lane) * 16, 0, AUX_SC1);
}
template <class Cfg>
__device__ inline void add_half(const GemmKArgs& p, f32x4 (&acc)[Cfg::IM][Cfg::IN], int slot, int wv, int lane) {
  constexpr int NB = Cfg::IM * Cfg::IN, CH = NB < 8 ? NB : 8;  // blocks in flight
  asm volatile("" : "+v"(lane));
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(p.partials + (int64_t)slot * p.partial_stride), 0, (Cfg::NW / 2) * NB * 1024, 0x00020000);
#pragma unroll
  for (int b0 = 0; b0 < NB; b0 += CH) {
    u32x4 v[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c)  // sc1: coherent at agent scope without a fence
      v[c] = __builtin_amdgcn_raw_buffer_load_b128(rs, ((wv * NB + b0 + c) * 64 + lane) * 16, 0, AUX_SC1);
#pragma unroll
    for (int c = 0; c < CH; ++c) acc[(b0 + c) / Cfg::IN][(b0 + c) % Cfg::IN] += __builtin_bit_cast(f32x4, v[c]);
  }
}

// Sliced hand-over, second half: rows [r0, r1) of the tile whose parts lie in
// slots slot0 .. slot0 + parts - 1 as row-major [CM, CN] fp32 matrices, summed
// in part order (the order in which an owner would add them) and handed to
// the epilogue operation: 16-byte strips of four columns, lanes along a row,
// two strips a lane and eight parts in flight.  The whole group works on the
// slice.  The destinations' heap bases come through ONE vector load, lane r
// holding rank r's (a scalar load per rank and strip, each waited for before
// the rank's stores could go out, cost more than everything else here).
template <class Cfg, int OP, int ODT>
__device__ inline void slice_epilogue(const GemmKArgs& p, const Item& it, int slot0, int parts, int r0, int r1,
                                      int tid) {  // tid: by value
  constexpr bool F32 = (OP == OP_STORE32 || OP == OP_ATOMIC32);
  constexpr int ES = F32 ? 4 : 2;
  constexpr int CN4 = Cfg::CN / 4, UN = 2, RG = 8;
  // (opaque, so that the lane's offsets are computed here and not kept in
  // registers across the K loop)
  asm volatile("" : "+v"(tid));
  const int nstrips = (r1 - r0) * CN4;
  const int r_begin = p.dest_all ? 0 : p.cur_rank;
  const int r_end = p.dest_all ? p.ws : p.cur_rank + 1;
  const int rows_ok = it.m_end - it.m0, cols_ok = it.n_end - it.n0;
  if (rows_ok <= 0 || cols_ok <= 0) return;
  const int64_t tile_off = ((int64_t)it.m0 * p.som + (int64_t)it.n0 * p.son) * ES;
  const uint32_t out_bytes = (uint32_t)(((int64_t)(rows_ok - 1) * p.som + cols_ok) * ES);
  const bool vec = p.vec_out && ((int64_t)(Cfg::CM - 1) * p.som + Cfg::CN) * ES < ((int64_t)1 << 31);
  // lane r of every wave: the heap base of rank r
  const bool table = p.heap_bases != nullptr && r_end - r_begin > 1 && p.ws <= 64;
  uint64_t lane_base = 0;
  if (table && (tid & 63) < p.ws) lane_base = p.heap_bases[tid & 63];
  for (int s0 = tid; s0 < nstrips; s0 += Cfg::NT * UN) {
    f32x4 sum[UN];
    int row[UN], col[UN];
    uint32_t poff[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int idx = s0 + u * Cfg::NT;
      const bool live = idx < nstrips;
      row[u] = r0 + idx / CN4;
      col[u] = (idx % CN4) * 4;
      poff[u] = live ? (uint32_t)((row[u] * Cfg::CN + col[u]) * 4) : DEAD_OFFSET;
      if (!live) row[u] = 0x40000000;  // past every edge
      sum[u] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int q0 = 0; q0 < parts; q0 += RG) {
      u32x4 v[RG][UN];
#pragma unroll
      for (int g = 0; g < RG; ++g) {
        const bool present = q0 + g < parts;
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(p.partials + (int64_t)(slot0 + (present ? q0 + g : 0)) * p.partial_stride), 0,
            present ? Cfg::CM * Cfg::CN * 4 : 0, 0x00020000);
#pragma unroll
        for (int u = 0; u < UN; ++u)  // sc1: coherent at agent scope without a fence
          v[g][u] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)poff[u], 0, AUX_SC1);
      }
#pragma unroll
      for (int g = 0; g < RG; ++g)
#pragma unroll
        for (int u = 0; u < UN; ++u) sum[u] += __builtin_bit_cast(f32x4, v[g][u]);
    }
    const uint64_t cur_base = table ? (((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(lane_base >> 32), p.cur_rank) << 32) |
                                       (uint32_t)__builtin_amdgcn_readlane((int)lane_base, p.cur_rank))
                                    : 0;
    auto rank_dst = [&](int r) __attribute__((always_inline)) -> IRIS_GLOBAL char* {
      if (table) {
        const uint64_t rb = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)(lane_base >> 32), r) << 32) |
                            (uint32_t)__builtin_amdgcn_readlane((int)lane_base, r);
        return (IRIS_GLOBAL char*)translate(p.out, cur_base, rb) + tile_off;
      }
      return rank_ptr(p, p.out, r) + tile_off;
    };
    // what each strip needs, decided once: `ncols` valid columns; strips that
    // are whole and may go out as one vector store have their offset, the
    // others' offsets are parked out of range, so that the loop over the
    // destinations is straight-line code
    int ncols[UN];
    uint32_t ooff[UN];
    bool ragged = false;
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      ncols[u] = row[u] < rows_ok ? max(0, min(4, cols_ok - col[u])) : 0;
      const bool whole = vec && ncols[u] == 4 && OP != OP_ATOMIC32;
      ooff[u] = whole ? (uint32_t)(((int64_t)row[u] * p.som + col[u]) * ES) : DEAD_OFFSET;
      ragged = ragged || (ncols[u] > 0 && !whole);
    }
    if constexpr (OP == OP_STORE32 || OP == OP_STORE16) {
      u32x4 w32[UN];
      u32x2 w16[UN];
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        w32[u] = __builtin_bit_cast(u32x4, sum[u]);
        w16[u] = u32x2{pack2<ODT>(sum[u][0], sum[u][1]), pack2<ODT>(sum[u][2], sum[u][3])};
      }
      auto all_ranks = [&](auto aux_tag) __attribute__((always_inline)) {
        constexpr int AUX = decltype(aux_tag)::value;
#pragma nounroll
        for (int r = r_begin; r < r_end; ++r) {
          const __amdgpu_buffer_rsrc_t rs = tile_rsrc(rank_dst(r), out_bytes);
#pragma unroll
          for (int u = 0; u < UN; ++u) {
            if constexpr (OP == OP_STORE32)
              __builtin_amdgcn_raw_buffer_store_b128(w32[u], rs, (int)ooff[u], 0, AUX);
            else
              __builtin_amdgcn_raw_buffer_store_b64(w16[u], rs, (int)ooff[u], 0, AUX);
          }
        }
      };
      if (p.sys)
        all_ranks(std::integral_constant<int, 17>{});
      else
        all_ranks(std::integral_constant<int, 16>{});
    } else if constexpr (OP == OP_ATOMIC16) {
#pragma nounroll
      for (int r = r_begin; r < r_end; ++r) {
        IRIS_GLOBAL char* dst = rank_dst(r);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          if (ooff[u] == DEAD_OFFSET) continue;
          atomic_add16_pair<ODT>((IRIS_GLOBAL unsigned int*)(dst + ooff[u]), pack2<ODT>(sum[u][0], sum[u][1]));
          atomic_add16_pair<ODT>((IRIS_GLOBAL unsigned int*)(dst + ooff[u] + 4), pack2<ODT>(sum[u][2], sum[u][3]));
        }
      }
    }
    if (ragged) {
      // ragged edge, odd strides or alignment, fp32 atomics: element by element
#pragma nounroll
      for (int r = r_begin; r < r_end; ++r) {
        IRIS_GLOBAL char* dst = rank_dst(r);
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          if (ooff[u] != DEAD_OFFSET) continue;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (e >= ncols[u]) continue;
            IRIS_GLOBAL char* d = dst + ((int64_t)row[u] * p.som + (int64_t)(col[u] + e) * p.son) * ES;
            if constexpr (OP == OP_STORE32)
              store_through((IRIS_GLOBAL unsigned int*)d, __builtin_bit_cast(unsigned int, sum[u][e]), p.sys != 0);
            else if constexpr (OP == OP_STORE16)
              store_through((IRIS_GLOBAL unsigned short*)d, to16<ODT>(sum[u][e]), p.sys != 0);
            else if constexpr (OP == OP_ATOMIC32)
              __hip_atomic_fetch_add((IRIS_GLOBAL float*)d, sum[u][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else
              atomic_add16_cas<ODT>((IRIS_GLOBAL unsigned short*)d, from16<ODT>(to16<ODT>(sum[u][e])));
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// One-shot reduce of one tile inside the GEMM program
// ---------------------------------------------------------------------------

// c_global[tile] = cast(sum over ranks 0..ws-1, in that order, of C_r[tile]):
// the tail of the reference program, gemm_one_shot_all_reduce.py:236-271.  The
// whole group works on the tile; a lane moves one 16-byte strip per rank, lanes
// run along a row, and RG ranks x UN rows are in flight per lane.  Absent ranks
// of the last group read through an empty descriptor: zeros, which leave an
// fp32 sum that started at +0 unchanged.  Loads are coherent at the flags'
// scope by themselves (sc1 / sc0 sc1) and the result is written through, like
// the reference's store with cache_modifier=".wt".
template <int IN_DT, int NT, int UN, bool SYS>
__device__ inline void fused_reduce_tile(const GemmKArgs& p, const Item& it, int tid) {  // tid: by value
  constexpr int IES = Vec<IN_DT>::ES, VE = Vec<IN_DT>::N;
  constexpr int RG = 4;
  constexpr int LAUX = SYS ? (AUX_NT | AUX_SC1 | AUX_SC0) : (AUX_NT | AUX_SC1);
  constexpr int SAUX = SYS ? (AUX_SC1 | AUX_SC0) : AUX_SC1;
  // (opaque, so that the lane's offsets are computed here and not kept in
  // registers across the K loop)
  asm volatile("" : "+v"(tid));
  const int m0 = it.lm0, n0 = it.ln0;
  const int rows = it.m_end - m0, cols = it.n_end - n0;
  const int oes = dtype_size(p.cg_dt);
  if (rows <= 0 || cols <= 0) return;
  if (p.fused_vec && cols % VE == 0) {
    const int cv = cols / VE;  // 16-byte strips per tile row
    const int tpr = min(cv, NT), rpp = NT / tpr;
    const int r0 = tid / tpr, cl = tid - r0 * tpr;
    const uint32_t in_bytes = ((uint32_t)(rows - 1) * (uint32_t)p.som + cols) * IES;
    const uint32_t out_bytes = ((uint32_t)(rows - 1) * (uint32_t)p.sgm + cols) * oes;
    const int64_t in0 = ((int64_t)m0 * p.som + n0) * IES;
    const __amdgpu_buffer_rsrc_t out_rs =
        tile_rsrc((const IRIS_GLOBAL char*)p.cg + ((int64_t)m0 * p.sgm + n0) * oes, out_bytes);
    for (int cc = 0; cc < cv; cc += tpr) {
      const int c = cc + cl;
      const bool live = r0 < rpp && c < cv;
      for (int rb = 0; rb < rows; rb += rpp * UN) {
        float acc[UN][VE];
        uint32_t ioff[UN], ooff[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          const uint32_t row = rb + r0 + u * rpp;
          ioff[u] = live ? (row * (uint32_t)p.som + c * VE) * IES : DEAD_OFFSET;
          ooff[u] = live ? (row * (uint32_t)p.sgm + c * VE) * oes : DEAD_OFFSET;
#pragma unroll
          for (int e = 0; e < VE; ++e) acc[u][e] = 0.f;
        }
        for (int rk0 = 0; rk0 < p.ws; rk0 += RG) {
          float v[RG][UN][VE];
#pragma unroll
          for (int g = 0; g < RG; ++g) {
            const bool present = rk0 + g < p.ws;
            const __amdgpu_buffer_rsrc_t rs =
                tile_rsrc((const IRIS_GLOBAL char*)rank_ptr(p, p.out, present ? rk0 + g : p.cur_rank) + in0,
                          present ? in_bytes : 0);
#pragma unroll
            for (int u = 0; u < UN; ++u) load_vec<IN_DT, LAUX>(rs, ioff[u], v[g][u]);
          }
#pragma unroll
          for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int u = 0; u < UN; ++u)
#pragma unroll
              for (int e = 0; e < VE; ++e) acc[u][e] += v[g][u][e];
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
          if (p.cg_dt == IRIS_DTYPE_F32)
            store_vec<IRIS_DTYPE_F32, VE, SAUX>(out_rs, ooff[u], acc[u]);
          else if (p.cg_dt == IRIS_DTYPE_BF16)
            store_vec<IRIS_DTYPE_BF16, VE, SAUX>(out_rs, ooff[u], acc[u]);
          else
            store_vec<IRIS_DTYPE_F16, VE, SAUX>(out_rs, ooff[u], acc[u]);
        }
      }
    }
  } else {
    // any strides, alignment and widths: element by element
    for (int idx = tid; idx < rows * cols; idx += NT) {
      const int r = idx / cols, cidx = idx - r * cols;
      const int64_t ioff = ((int64_t)(m0 + r) * p.som + (int64_t)(n0 + cidx) * p.son) * IES;
      float acc = 0.f;
      for (int rk = 0; rk < p.ws; ++rk) {
        const IRIS_GLOBAL char* src = (const IRIS_GLOBAL char*)rank_ptr(p, p.out, rk) + ioff;
        if constexpr (IN_DT == IRIS_DTYPE_F32) {
          const unsigned int w = SYS ? __hip_atomic_load((const IRIS_GLOBAL unsigned int*)src, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_SYSTEM)
                                     : __hip_atomic_load((const IRIS_GLOBAL unsigned int*)src, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT);
          acc += __builtin_bit_cast(float, w);
        } else {
          const unsigned short h = SYS ? __hip_atomic_load((const IRIS_GLOBAL unsigned short*)src, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_SYSTEM)
                                       : __hip_atomic_load((const IRIS_GLOBAL unsigned short*)src, __ATOMIC_RELAXED,
                                                           __HIP_MEMORY_SCOPE_AGENT);
          acc += from16<IN_DT>(h);
        }
      }
      IRIS_GLOBAL char* d = (IRIS_GLOBAL char*)p.cg + ((int64_t)(m0 + r) * p.sgm + (int64_t)(n0 + cidx) * p.sgn) * oes;
      if (p.cg_dt == IRIS_DTYPE_F32)
        store_through((IRIS_GLOBAL unsigned int*)d, __builtin_bit_cast(unsigned int, acc), SYS);
      else if (p.cg_dt == IRIS_DTYPE_BF16)
        store_through((IRIS_GLOBAL unsigned short*)d, to16<IRIS_DTYPE_BF16>(acc), SYS);
      else
        store_through((IRIS_GLOBAL unsigned short*)d, to16<IRIS_DTYPE_F16>(acc), SYS);
    }
  }
}

// ---------------------------------------------------------------------------
// The kernel
// ---------------------------------------------------------------------------

// SPLIT: the split-K build of the kernel (only launched with p.split_k > 1);
// the plain build carries none of its code or state.
// FUSED: the one-shot epilogue as the reference program runs it
// (gemm_one_shot_all_reduce.py:197-271): store the partial tile, signal the
// other ranks, wait for the tile's own flag, reduce it over all ranks and
// store the result, tile by tile, while other programs are in their K loops.
template <class Cfg, int OP, int ODT, bool SPLIT = false, bool FUSED = false, bool MERGED = false>
__global__ __launch_bounds__(Cfg::THREADS) __attribute__((amdgpu_waves_per_eu(Cfg::WPE, Cfg::WPE))) void
gemm_persistent_kernel(const GemmKArgs p) {
  static_assert(!MERGED || !FUSED, "blocks of the caller's tiles: no build with the reduce inside");
  extern __shared__ __attribute__((aligned(1024))) char lds_raw[];
  IRIS_LDS char* lds = (IRIS_LDS char*)lds_raw;
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;
  // Roles (wave-uniform).  Every wave runs the same control flow, so every
  // barrier below is met by all of them; only the work is told apart: the
  // first NW waves multiply and store, the fetching waves (if the tile has
  // any; otherwise every wave does both) issue the stage loads.
  const bool worker = Cfg::LW == 0 || wave < Cfg::NW;
  const bool fetcher = Cfg::LW == 0 || wave >= Cfg::NW;
  const int fwave = Cfg::LW == 0 ? wave : wave - Cfg::NW;  // index among the fetching waves
  int pid;
  if (p.xcd_per > 0) {
    // workgroups are dealt to the XCDs round-robin: this one is number j on XCD x
    const int x = blockIdx.x % p.num_xcds, j = blockIdx.x / p.num_xcds;
    pid = j < p.xcd_per ? x * p.xcd_per + j : p.num_sms * 2;  // (past every item: nothing to do)
  } else {
    pid = xcd_remap(blockIdx.x, p.num_sms, p.num_xcds);
  }
  if constexpr (SPLIT) {
    if (p.part_major > 0 && pid < p.part_major * p.split_k) {
      const int part = pid / p.part_major, tile = pid - part * p.part_major;
      pid = tile * p.split_k + part;
    }
  }

  if constexpr (Cfg::NW == 8 && Cfg::CM == 256 && Cfg::CN == 256 && !SPLIT && !FUSED) {
    // (workgroups are dealt to the XCDs in turn: blockIdx.x / num_xcds counts a program's place on its XCD)
    if (p.stagger_groups > 1) {
      const int group = (blockIdx.x / p.num_xcds) % p.stagger_groups;
      for (int i = 0; i < group * p.stagger_sleeps; ++i) __builtin_amdgcn_s_sleep(9);
    }
  }
  constexpr bool split = SPLIT;
  // The split build of a tile without the owner's hand-over only ever runs split-K proper (stream-K runs need
  // the owner's way): one (tile, part) item per program.  Saying so at compile time takes the item loop, the
  // load cursor's step into a next item and everything that would stay live across an epilogue for it
  // (the next item's first fragments, the loader's state) out of these builds, whose registers are full.
  constexpr bool ONE_ITEM = SPLIT && !Cfg::SPLIT_OWNER;
  const int nk = (p.K + Cfg::BK - 1) / Cfg::BK;
  const int work = split ? p.total_tiles * p.split_k : p.total_tiles;  // tiles, or (tile, part) pairs
  const int n_mine = pid < work ? (work - pid + p.num_sms - 1) / p.num_sms : 0;
  int n_items = split ? n_mine : n_mine * p.sub_m * p.sub_n;
  StreamRun sr{0, 0, 0};
  if constexpr (SPLIT) {
    if constexpr (ONE_ITEM) {
      sr = split_run(p, pid, nk);
      n_items = stream_items(sr, nk) > 0 ? 1 : 0;
    } else {
      sr = p.stream_k ? stream_run(p, pid, nk) : split_run(p, pid, nk);
      n_items = stream_items(sr, nk);
    }
  }
  const int total_steps = n_items * nk;  // > 0 iff there is anything to load

  const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
  IRIS_LDS char* ws = lds + Cfg::S * Cfg::STAGE + wave * Cfg::WS_BYTES;

  // operand fetch offsets inside a stage
  // lane l reads row l%16 of a 16-row block and the 16-byte chunk l/16 of the
  // substep's four (block bases are multiples of 16 rows, so the swizzle of a
  // row only depends on l%16)
  const int lrow = lane & 15, lq = lane >> 4;
  const int a_row_off = (wm * Cfg::TM + lrow) * Cfg::BK * 2;
  const int b_row_off = (wn * Cfg::TN + lrow) * Cfg::BK * 2;
  int xoff[Cfg::KSUB];
#pragma unroll
  for (int kk = 0; kk < Cfg::KSUB; ++kk) xoff[kk] = ((kk * 4 + lq) ^ ((lrow / Cfg::RP) % Cfg::CPR)) * 16;

  f32x4 acc[Cfg::IM][Cfg::IN];
#pragma unroll
  for (int i = 0; i < Cfg::IM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::IN; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

  // A tile's flag may only be published once every wave's stores of the tile
  // have completed.  Waiting for that right after issuing them would stall
  // the matrix cores, so the publication is deferred to the top of the next
  // K-step, where the whole group waits on its memory counter anyway.
  const bool defer_publish = !FUSED && Cfg::DMA && nk > 0 && p.flag_mode != 0;
  int pending_tile = -1;
  // 1: the pending tile's stores are exactly the FAST_STORES youngest memory
  // operations of this wave, so the next hand-over can wait for the loads
  // issued before them and leave the stores in flight one K-step longer
  int pending_skip = 0;
  constexpr int FAST_STORES = StoreCount<Cfg, OP>::FAST_STORES;
  static_assert(Cfg::L * (Cfg::S > 2 ? Cfg::S - 2 : 0) + FAST_STORES <= 63, "vmcnt immediate");

  int c_item = 0;  // compute cursor
  Item c_it;
  if (n_items > 0) c_it = decode_item<Cfg, SPLIT>(p, sr, pid, 0);

  // L2 prefetch hints (see GemmKArgs::pf_dist): the first two multiplying waves, one for A and one for B, hold a
  // descriptor of the current tile's panel and each lane the offset of the row whose line it touches.
  // (compiled into the 256 x 64 tile only: a test and a branch per K-step are felt by the small tiles, whose
  // steps take 0.2 us: [512,4096] x [4096,1376] in 64 x 64 x 128 tiles 19.9 -> 24.3 us)
  constexpr bool PF = Cfg::LW != 0 && Cfg::DMA && !FUSED && Cfg::CM == 256 && Cfg::CN == 64;
  // a third build of the K-step, without the hand-over's tests (see `step`; not with the reduce inside the program,
  // where the K loop is the smaller part and a third copy of the step adds to what the 128-accumulator tiles spill)
  constexpr bool LEAN_STEPS = Cfg::DMA && !FUSED;
  // the lean steps of the eight-wave 256 x 256 tile each end with the two touches of Loader::touch, which the
  // next lean step's hand-over leaves in flight
  constexpr bool PF8 = Cfg::TOUCH && LEAN_STEPS;
  constexpr int TOUCHES = PF8 ? 2 : 0;
  __amdgpu_buffer_rsrc_t pf_rs = __builtin_amdgcn_make_buffer_rsrc((void*)p.a, 0, 0, 0x00020000);
  uint32_t pf_off = 0x80000000u;
  auto prefetch_setup = [&](const Item& it) __attribute__((always_inline)) {
    if constexpr (PF) {
      if (p.pf_dist > 0 && wave < 2) {
        const bool isA = wave == 0;
        const int origin = isA ? it.m0 : it.n0, extent = isA ? p.M : p.N, span = isA ? Cfg::CM : Cfg::CN;
        const int64_t ld = isA ? p.sam : p.sbn;
        const int rows = origin < extent ? min(span, extent - origin) : 0;
        const char* base = (isA ? p.a : p.b) + (int64_t)min(origin, extent - 1) * ld * 2;
        pf_rs = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, rows > 0 ? (int)(((int64_t)(rows - 1) * ld + p.K) * 2) : 0,
                                                  0x00020000);
        // this program's share: rows `first`, `first + share`, ... of the panel
        const int share = isA ? p.pf_sa : p.pf_sb;
        const int first = (isA ? it.ln0 / p.BN : it.lm0 / p.BM) % share;
        const int row = first + share * lane;
        pf_off = row < rows ? (uint32_t)((int64_t)row * ld * 2) : 0x80000000u;
      }
    }
  };
  // ... and touch the lines of K-step `k` (steps from `k_end` on are left alone).  The dword a lane fetches must
  // land somewhere, and not in a register (the compiler would hand the register on before the load returns):
  // it goes, by LDS-DMA, into the wave's own epilogue scratch, which nothing reads inside a K loop.  The last
  // touch of a tile is issued pf_dist steps before its epilogue.
  auto prefetch_step = [&](int k, int k_end) __attribute__((always_inline)) {
    if constexpr (PF) {
      if (p.pf_dist > 0 && wave < 2 && k < k_end)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(pf_rs, (IRIS_LDS void*)ws, 4, pf_off, k * Cfg::BK * 2, 0, 0);
    }
  };

  // end of a compute tile: store it, and publish the logical tile it completes
  // FUSED: a wait for a peer's tile has timed out.  The peer is not resident (or gone): the tiles that follow
  // are still stored and signalled, but not waited for, so that a launch without its peers costs one timeout
  // and not one per tile.
  int peers_gone = 0;
  const GemmKArgs& p_outer = p;
  auto epilogue = [&]() __attribute__((always_inline)) {
    if constexpr (PF) {
      // (the prefetch hints' dwords land in this wave's scratch: all of them have, before the epilogue uses it;
      // the last was issued pf_dist K-steps ago, so nothing is waited for in practice)
      if (wave < 2) IRIS_WAIT_VMCNT(0);
    }
    if (defer_publish && pending_tile >= 0) {
      // a one-step tile: the previous tile has not been published yet
      IRIS_WAIT_VMCNT(0);
      __syncthreads();
      if (wave == 0) publish_tile<MERGED>(p, pending_tile, lane);
      pending_tile = -1;
    }
    if constexpr (SPLIT) {
      if (ONE_ITEM || p.sliced) {
        // (One item per program: whatever this hand-over reads of the launch's arguments is read here, from the
        // argument block, through a pointer the compiler cannot see through; held in scalar registers from the
        // kernel's entry on, those arguments pushed fragments of the K loop out of the 128-accumulator tiles'
        // registers: the split 256 x 256 tile stepped in 2.3 us instead of 1.5.)
        typedef const __attribute__((address_space(4))) GemmKArgs* KernArgPtr;
        KernArgPtr late_args = (KernArgPtr)__builtin_amdgcn_kernarg_segment_ptr();  // (the kernel's only parameter)
        asm volatile("" : "+s"(late_args));
        const GemmKArgs& p = ONE_ITEM ? *(const GemmKArgs*)late_args : p_outer;
        // split-K proper: program pid is part pid % split_k of tile pid / split_k
        const int parts = p.split_k;
        const int slot0 = __builtin_amdgcn_readfirstlane((int)fast_div((uint32_t)pid, p.div_split) * parts);
        const int part = pid - slot0;
        IRIS_LDS int* okslot = (IRIS_LDS int*)(lds + Cfg::S * Cfg::STAGE);  // wave 0's scratch, idle here
        // two parts, each keeping the half of the waves it owns (see dump_half)
        constexpr bool PAIR_BUILD = ONE_ITEM && Cfg::NW % 2 == 0;
        const bool pair = PAIR_BUILD && p.sliced == 2;
        const bool mine = (wave < Cfg::NW / 2) == (part == 0);
        const int wv = wave < Cfg::NW / 2 ? wave : wave - Cfg::NW / 2;
        if (pair) {
          if constexpr (PAIR_BUILD) {
            if (worker && !mine) dump_half<Cfg>(p, acc, pid, wv, lane);
          }
        } else {
          // the partial as a row-major [CM, CN] fp32 matrix in slot `pid`, through
          // the fp32 store epilogue (whole 128-byte lines, written through)
          // (only what store_acc reads: a copy of all the arguments would be made in memory)
          GemmKArgs q;
          q.out = (char*)(p.partials + (int64_t)pid * p.partial_stride);
          q.som = Cfg::CN;
          q.son = 1;
          q.dest_all = 0;
          q.vec_out = 1;
          q.sys = 0;
          q.heap_bases = nullptr;
          q.cur_rank = 0;
          q.ws = 1;
          if (worker)
            store_acc<Cfg, OP_STORE32, IRIS_DTYPE_F32>(q, acc, ws, wm * Cfg::TM, wn * Cfg::TN, Cfg::CM, Cfg::CN, lane);
        }
        IRIS_WAIT_VMCNT(0);  // this wave's part of the partial has been written
        __syncthreads();
        if (tid == 0) {
          flag_add_relaxed((IRIS_GLOBAL int32_t*)(p.locks + slot0), 1, false);
          *okslot = wait_tile_ready((IRIS_GLOBAL int32_t*)(p.locks + slot0), parts, false, p.timeout, p.status) ? 1 : 0;
        }
        __syncthreads();
        const int ok = *okslot;
        if (ok && worker) {
          if (pair) {
            if constexpr (PAIR_BUILD) {
              if (mine) {
                add_half<Cfg>(p, acc, slot0 + 1 - part, wv, lane);
                store_acc<Cfg, OP, ODT>(p, acc, ws, c_it.m0 + wm * Cfg::TM, c_it.n0 + wn * Cfg::TN, c_it.m_end,
                                        c_it.n_end, lane);
              }
            }
          } else {
            slice_epilogue<Cfg, OP, ODT>(p, c_it, slot0, parts, part * Cfg::CM / parts, (part + 1) * Cfg::CM / parts,
                                         tid);
          }
        }
        IRIS_WAIT_VMCNT(0);  // this wave's stores of the slice have completed
        __syncthreads();     // (and okslot is scratch again)
        if (wave == 0 && ok) {
          IRIS_GLOBAL int32_t* done = (IRIS_GLOBAL int32_t*)(p.locks + slot0 + 1);
          int before = 0;
          if (lane == 0) before = __hip_atomic_fetch_add(done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          before = __builtin_amdgcn_readfirstlane(before);
          if (before == parts - 1) {
            // every slice is in memory: publish, and leave both counters at 0
            if (p.flag_mode != 0) publish_tile<MERGED>(p, c_it.tile_id, lane);
            if (lane == 0) {
              flag_add_relaxed(done, -parts, false);
              flag_add_relaxed((IRIS_GLOBAL int32_t*)(p.locks + slot0), -parts, false);
            }
          }
        }
        if (p.ts_end && tid == 0)
          __hip_atomic_fetch_max((IRIS_GLOBAL unsigned long long*)(p.ts_end + c_it.tile_id),
                                 (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if constexpr (!ONE_ITEM) {
          if (++c_item < n_items) c_it = decode_item<Cfg, SPLIT>(p, sr, pid, c_item);
        }
        return;
      }
      // (the tiles without the owner's way are only launched with the sliced one)
      if constexpr (Cfg::SPLIT_OWNER) {
      const KRange kr = k_range<Cfg, SPLIT>(p, sr, pid, c_item, nk);
      if (kr.part != 0) {
        // not the owner: leave the partial, raise the lock once every wave's
        // stores have completed, and move on
        if (worker) dump_partial<Cfg>(p, acc, kr.slot, tid);
        IRIS_WAIT_VMCNT(0);
        __syncthreads();
        if (tid == 0) flag_add_relaxed((IRIS_GLOBAL int32_t*)(p.locks + kr.slot), 1, false);
        if (++c_item < n_items) c_it = decode_item<Cfg, SPLIT>(p, sr, pid, c_item);
        return;
      }
      // Wait for every other part at once: lane q of the group takes part q's
      // lock (1 -> 0, which also re-arms it for the next launch), each wait
      // bounded; then fetch the partials a few parts at a time.
      int ok = 1;
      const int parts = p.stream_k ? stream_parts(p, pid, kr.k_end, nk) : p.split_k;
      if (tid >= 1 && tid < parts)
        ok = wait_tile_flag((IRIS_GLOBAL int32_t*)(p.locks + kr.slot + tid), 2, false, p.timeout, p.status) ? 1 : 0;
      if (__syncthreads_and(ok)) {
        constexpr int GROUP = Cfg::IM * Cfg::IN * 4 <= 16 ? 4 : Cfg::IM * Cfg::IN * 4 <= 32 ? 2 : 1;
        if (worker)
          for (int q = 1; q < parts; q += GROUP) add_partials<Cfg, GROUP>(p, acc, kr.slot, q, parts, tid);
      }
      }
    }
    bool fast = true;  // (a fetching wave has no stores to count)
    if (worker)
      fast = store_acc<Cfg, OP, ODT>(p, acc, ws, c_it.m0 + wm * Cfg::TM, c_it.n0 + wn * Cfg::TN, c_it.m_end, c_it.n_end,
                                     lane);
    if constexpr (FUSED) {
      static_assert(!SPLIT && (OP == OP_STORE16 || OP == OP_STORE32), "the in-program reduce follows a plain store");
      if (c_it.last_sub) {
        constexpr int IN_DT = OP == OP_STORE32 ? IRIS_DTYPE_F32 : ODT;
        // (the arguments this part reads come from the argument block when it runs, not from registers held
        // across the K loop: see the split hand-over above)
        typedef const __attribute__((address_space(4))) GemmKArgs* KernArgPtr;
        KernArgPtr late_args = (KernArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("" : "+s"(late_args));
        const GemmKArgs& p = *(const GemmKArgs*)late_args;
        IRIS_LDS int* slot = (IRIS_LDS int*)(lds + Cfg::S * Cfg::STAGE);  // wave 0's scratch, idle by now
        IRIS_WAIT_VMCNT(0);  // this wave's stores of the partial tile have completed
        __syncthreads();
        int ok = 1;
        if (p.ws > 1) {
          if (wave == 0) publish_tile<MERGED>(p, c_it.tile_id, lane);  // +1 on every other rank (:207-218)
          if (tid == 0) {
            *slot = !peers_gone && wait_tile_flag((IRIS_GLOBAL int32_t*)(p.flags + c_it.tile_id), p.ws, p.sys != 0,
                                                  p.timeout, p.status)
                        ? 1
                        : 0;  // CAS(ws-1 -> 0) until it succeeds (:220-234), bounded
          }
          __syncthreads();
          ok = *slot;
          if (!ok) peers_gone = 1;
        }
        if (ok) {
          // rows in flight per lane (the accumulators' registers are free by now)
          constexpr int UN = 4;
          if (!worker) {
          } else if (p.sys)
            fused_reduce_tile<IN_DT, Cfg::NT, UN, true>(p, c_it, tid);
          else
            fused_reduce_tile<IN_DT, Cfg::NT, UN, false>(p, c_it, tid);
        }
        __syncthreads();  // the slot is scratch again
        if (p.ts_end && tid == 0)
          __hip_atomic_fetch_max((IRIS_GLOBAL unsigned long long*)(p.ts_end + c_it.tile_id),
                                 (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    } else if (c_it.last_sub) {
      if (defer_publish) {
        pending_tile = __builtin_amdgcn_readfirstlane(c_it.tile_id);
        // the count only holds for a tile that is a single compute tile
        pending_skip = (fast && c_it.first_sub) ? 1 : 0;
      } else if (p.flag_mode != 0) {
        IRIS_WAIT_VMCNT(0);  // this wave's stores of the tile have completed
        __syncthreads();
        if (wave == 0) publish_tile<MERGED>(p, c_it.tile_id, lane);
      }
      if (p.ts_end && tid == 0)
        __hip_atomic_fetch_max((IRIS_GLOBAL unsigned long long*)(p.ts_end + c_it.tile_id),
                               (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (++c_item < n_items) c_it = decode_item<Cfg, SPLIT>(p, sr, pid, c_item);
  };
  auto stamp_begin = [&]() __attribute__((always_inline)) {
    if (p.ts_begin && c_it.first_sub && tid == 0)
      __hip_atomic_fetch_min((IRIS_GLOBAL unsigned long long*)(p.ts_begin + c_it.tile_id),
                             (unsigned long long)wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  if (nk == 0) {
    // K == 0 leaves every tile all zeros: one epilogue per item, no loads
    for (int it = 0; it < n_items; ++it) epilogue();
  } else if constexpr (Cfg::DMA) {
    // ---- the (item, k) pipeline -------------------------------------------
    // Ring of S stages.  A step's last fragment fetch happens one substep
    // before its last MFMAs, so at the hand-over in step g every wave is done
    // reading stage g: it is refilled right there with step g+S.  While the
    // tail of step g is multiplied, stage g+1 has landed and stages
    // g+2..g+S are in flight.  The load cursor runs S steps ahead of the
    // compute cursor and crosses into the next item on its own.
    Loader<Cfg> ld;
    int l_item = 0, l_k = 0, l_kend = nk;  // load cursor
    Item l_it;
    auto advance_load_cursor = [&]() __attribute__((always_inline)) {
      if (++l_k == l_kend) {
        if (!ONE_ITEM && ++l_item < n_items) {
          l_it = decode_item<Cfg, SPLIT>(p, sr, pid, l_item);
          const KRange kr = k_range<Cfg, SPLIT>(p, sr, pid, l_item, nk);
          l_k = kr.k_begin;
          l_kend = kr.k_end;
          ld.setup(p, l_it, fwave, lane, l_k);
        } else {
          l_k = 0;
          l_kend = nk;
          ld.park();  // nothing left to load
        }
      } else {
        ld.before_step(l_k, fwave, lane);
      }
    };
    Frags<Cfg> fr;
    if (total_steps > 0) {
      if (fetcher) {
        l_it = c_it;  // (item 0, decoded above for the compute cursor)
        const KRange kr = k_range<Cfg, SPLIT>(p, sr, pid, 0, nk);
        l_k = kr.k_begin;
        l_kend = kr.k_end;
        ld.setup(p, l_it, fwave, lane, l_k);
#pragma unroll
        for (int s = 0; s < Cfg::S; ++s) {
          ld.issue(p, lds + s * Cfg::STAGE, l_k, fwave);
          advance_load_cursor();
        }
        // stage 0 has landed once at most S-1 younger slabs are outstanding
        IRIS_WAIT_VMCNT(Cfg::L * (Cfg::S - 1));
      }
      block_barrier_raw();
      if (worker) {
        load_all<Cfg>(lds + a_row_off + xoff[0], lds + Cfg::A_BYTES + b_row_off + xoff[0], fr, 0);
        IRIS_WAIT_LGKMCNT0();
      }
    }

    // One K-step (global step number g).  FIRST: the tile's first step, whose
    // first substep defines the accumulators.  PAR: B buffer the step starts
    // with (it only alternates between steps when KSUB is odd).
    //
    // A substep issues its MFMAs one 16-row block (IN MFMAs) at a time; right
    // after a block, its A fragment and a share of the B fragments are fetched
    // for the next substep, so every fetch has almost a whole substep of MFMAs
    // to land behind.  The step's last substep hands over: after its first
    // block the wave waits for its part of stage g+1, meets the other waves,
    // and from then on fetches from stage g+1 and refills stage g with step
    // g+S, a few DMA loads per block.  The program's very last step hands over
    // too; what it fetches is never used (loads past the last step fetch
    // nothing).
    int ring_slot = 0;  // slot of the step about to run (rings whose depth is no power of two)
    // LEAN: a step in the middle of a tile's K loop.  No tile waits to be published at its hand-over (the
    // previous tile's flag went up at this tile's second hand-over) and the load cursor's next step lies inside
    // the tile and is a full one, so the hand-over is a wait, the barrier and the refill, with no test between
    // them: the waves all pass it at the same time, and what it costs, every SIMD's matrix core waits out.
    auto step = [&](int g, auto first_tag, auto par_tag, auto lean_tag) __attribute__((always_inline)) {
      constexpr bool FIRST = decltype(first_tag)::value;
      constexpr int PAR = decltype(par_tag)::value;
      constexpr bool LEAN = decltype(lean_tag)::value;
      int slot_g, slot_n;  // ring slots of steps g and g+1
      if constexpr (Cfg::S_POW2) {
        slot_g = g & (Cfg::S - 1);
        slot_n = (g + 1) & (Cfg::S - 1);
      } else {
        slot_g = ring_slot;
        slot_n = ring_slot + 1 == Cfg::S ? 0 : ring_slot + 1;
        ring_slot = slot_n;
      }
      const IRIS_LDS char* stage = lds + slot_g * Cfg::STAGE;
      if (worker) {
#pragma unroll
        for (int kk = 0; kk < Cfg::KSUB - 1; ++kk) {
          const int cb = (PAR + kk) & 1;
          const IRIS_LDS char* sA = stage + a_row_off + xoff[kk + 1];
          const IRIS_LDS char* sB = stage + Cfg::A_BYTES + b_row_off + xoff[kk + 1];
#pragma unroll
          for (int i = 0; i < Cfg::IM; ++i) {
            if (FIRST && kk == 0)
              mma_row<Cfg, true>(acc, fr, cb, i);
            else
              mma_row<Cfg, false>(acc, fr, cb, i);
            fr.a[i] = load_a<Cfg>(sA, i);
            load_b_share<Cfg>(sB, i, fr.b[cb ^ 1]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
      {
        constexpr int kk = Cfg::KSUB - 1;
        constexpr int cb = (PAR + kk) & 1;
        constexpr bool F = FIRST && kk == 0;
        if (worker) {
          mma_row<Cfg, F>(acc, fr, cb, 0);
          __builtin_amdgcn_sched_barrier(0);
          // this wave's reads of stage g have returned (they were issued a
          // substep ago), so the stage may be refilled after the barrier
          IRIS_WAIT_LGKMCNT0();
        }
        // hand-over of stage g+1: wait for this wave's part of its slab
        // (S-2 younger slabs may stay in flight), then meet the other waves
        const int pend = LEAN ? -1 : __builtin_amdgcn_readfirstlane(pending_tile);
        const int skip = LEAN ? 0 : __builtin_amdgcn_readfirstlane(pending_skip);
        if constexpr (LEAN) {
          if (Cfg::LW == 0 || fetcher) IRIS_WAIT_VMCNT(Cfg::L * (Cfg::S - 2) + TOUCHES);
        } else if constexpr (Cfg::LW != 0) {
          if (fetcher) {
            IRIS_WAIT_VMCNT(Cfg::L * (Cfg::S - 2));
          } else if (pend >= 0 && skip == 0) {
            IRIS_WAIT_VMCNT(0);  // the previous tile's stores (all this wave has in flight)
          }
        } else if (pend >= 0 && skip == 0) {
          IRIS_WAIT_VMCNT(0);  // the previous tile's stores, too
        } else if (pend >= 0) {
          IRIS_WAIT_VMCNT(Cfg::L * (Cfg::S - 2) + FAST_STORES);  // the stores stay in flight
        } else {
          IRIS_WAIT_VMCNT(Cfg::L * (Cfg::S - 2));
        }
        block_barrier_raw();
        if constexpr (!LEAN) {
          if (pend >= 0) {
            if (skip == 0) {
              if (wave == 0) publish_tile<MERGED>(p, pend, lane);
              pending_tile = -1;
            } else {
              pending_skip = 0;
            }
          }
        }
        const IRIS_LDS char* nstage = lds + slot_n * Cfg::STAGE;
        const IRIS_LDS char* sA = nstage + a_row_off + xoff[0];
        const IRIS_LDS char* sB = nstage + Cfg::A_BYTES + b_row_off + xoff[0];
        IRIS_LDS char* rstage = lds + slot_g * Cfg::STAGE;
        if (worker) {
          fr.a[0] = load_a<Cfg>(sA, 0);
          load_b_share<Cfg>(sB, 0, fr.b[cb ^ 1]);
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 1; i < Cfg::IM; ++i) {
            mma_row<Cfg, F>(acc, fr, cb, i);
            fr.a[i] = load_a<Cfg>(sA, i);
            load_b_share<Cfg>(sB, i, fr.b[cb ^ 1]);
            // every wave is past its reads of stage g: refill it with step g+S,
            // the L loads shared out over the blocks
            if constexpr (Cfg::LW == 0) {
#pragma unroll
              for (int q = (i - 1) * Cfg::L / (Cfg::IM - 1); q < i * Cfg::L / (Cfg::IM - 1); ++q)
                ld.issue_at(p, rstage, l_k, wave, q);
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if constexpr (Cfg::LW != 0) {
          // every wave is past its reads of stage g: refill it with step g+S
          if (fetcher) {
            ld.issue(p, rstage, l_k, fwave);
            if constexpr (LEAN)
              ++l_k;
            else
              advance_load_cursor();
          }
        } else if constexpr (LEAN) {
          ++l_k;
        } else {
          advance_load_cursor();
        }
      }
    };
    // B buffer a step starts with: substeps alternate, so with an odd KSUB
    // it flips from step to step
    auto run_step = [&](int g, auto first_tag, auto lean_tag) __attribute__((always_inline)) {
      if constexpr (Cfg::KSUB % 2 == 0) {
        step(g, first_tag, std::integral_constant<int, 0>{}, lean_tag);
      } else {
        if (g & 1)
          step(g, first_tag, std::integral_constant<int, 1>{}, lean_tag);
        else
          step(g, first_tag, std::integral_constant<int, 0>{}, lean_tag);
      }
    };
    int g = 0;
    auto run_item = [&](int it) __attribute__((always_inline)) {
      stamp_begin();
      const KRange kr = k_range<Cfg, SPLIT>(p, sr, pid, it, nk);
      prefetch_setup(c_it);
      prefetch_step(kr.k_begin + p.pf_dist, kr.k_end);
      run_step(g, std::true_type{}, std::false_type{});
      ++g;
      const int steps = kr.k_end - kr.k_begin;
      // Steps [2, lean_end) are lean: the previous tile was published at the second hand-over, and the load
      // cursor, S steps ahead, moves on to a full step of this tile (the K loop's last step may be a partial one).
      const int lean_end = LEAN_STEPS ? steps - Cfg::S - 1 - ((p.K % Cfg::BK) != 0 ? 1 : 0) : 0;
      int k = 1;
      for (; k < steps && k < 2; ++k, ++g) {
        prefetch_step(kr.k_begin + k + p.pf_dist, kr.k_end);
        run_step(g, std::false_type{}, std::false_type{});
      }
      if constexpr (PF8) {
        // every lean step is entered with the two touches issued last
        if (k < lean_end) {
          const int dist = p.pf_dist;
          ld.touch(ws, min(l_k + dist, l_kend - 1));
          for (;;) {
            run_step(g, std::false_type{}, std::true_type{});
            ++k, ++g;
            if (k >= lean_end) break;
            ld.touch(ws, min(l_k + dist, l_kend - 1));
          }
        }
      } else if constexpr (LEAN_STEPS) {
        for (; k < lean_end; ++k, ++g) {
          prefetch_step(kr.k_begin + k + p.pf_dist, kr.k_end);
          run_step(g, std::false_type{}, std::true_type{});
        }
      }
      if constexpr (LEAN_STEPS && !PF8) {
        // Step lean_end is the one in which the load cursor crosses into the next tile (decode, loader set-up).
        // The S steps behind it load that tile's first steps and are lean again, when those are full steps and
        // the cursor does not cross a second time (behind the program's last tile it is parked on [0, nk)).
        if (k == lean_end && k < steps && (p.K % Cfg::BK) == 0) {
          int next_steps = nk;
          if constexpr (SPLIT) {
            if (it + 1 < n_items) {
              const KRange nr = k_range<Cfg, SPLIT>(p, sr, pid, it + 1, nk);
              next_steps = nr.k_end - nr.k_begin;
            }
          }
          prefetch_step(kr.k_begin + k + p.pf_dist, kr.k_end);
          run_step(g, std::false_type{}, std::false_type{});
          ++k, ++g;
          if (next_steps > Cfg::S) {
            for (; k < steps; ++k, ++g) {
              prefetch_step(kr.k_begin + k + p.pf_dist, kr.k_end);
              run_step(g, std::false_type{}, std::true_type{});
            }
          }
        }
      }
      for (; k < steps; ++k, ++g) {
        prefetch_step(kr.k_begin + k + p.pf_dist, kr.k_end);
        run_step(g, std::false_type{}, std::false_type{});
      }
      if constexpr (ONE_ITEM) IRIS_WAIT_VMCNT(0);  // (the loads past the last step fetch nothing, and nothing follows)
      epilogue();
    };
    if constexpr (ONE_ITEM) {
      if (n_items > 0) run_item(0);
    } else {
      for (int it = 0; it < n_items; ++it) run_item(it);
    }
    IRIS_WAIT_VMCNT(0);  // no load may still be writing this group's LDS when it exits
  } else {
    // ---- generic loader: one stage, synchronous ---------------------------
    Frags<Cfg> fr;
    for (int it = 0; it < n_items; ++it) {
      stamp_begin();
      const KRange kr = k_range<Cfg, SPLIT>(p, sr, pid, it, nk);
      for (int k = kr.k_begin; k < kr.k_end; ++k) {
        __syncthreads();  // previous step's readers are done with the stage
        load_slab_generic<Cfg>(p, c_it, lds, k, tid);
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < Cfg::KSUB; ++kk) {
          load_all<Cfg>(lds + a_row_off + xoff[kk], lds + Cfg::A_BYTES + b_row_off + xoff[kk], fr, 0);
#pragma unroll
          for (int i = 0; i < Cfg::IM; ++i) {
            if (k == kr.k_begin && kk == 0)
              mma_row<Cfg, true>(acc, fr, 0, i);
            else
              mma_row<Cfg, false>(acc, fr, 0, i);
          }
        }
      }
      epilogue();
    }
  }

  if (pending_tile >= 0) {
    IRIS_WAIT_VMCNT(0);
    __syncthreads();
    if (wave == 0) publish_tile<MERGED>(p, pending_tile, lane);
  }
}

}  // namespace iris_amd
