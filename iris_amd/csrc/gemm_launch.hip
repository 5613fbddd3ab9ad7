// C-ABI launcher of the persistent shard GEMM (include/iris_amd.h).
#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <memory>
#include <mutex>
#include <utility>
#include <vector>

#include "gemm_skinny.hpp"

namespace iris_amd {

namespace {

const GemmKernelEntry* entries_for(int dt, int op, int* count) {
  if (dt == IRIS_DTYPE_BF16) {
    switch (op) {
      case OP_STORE16: return gemm_entries_bf16_store16(count);
      case OP_STORE32: return gemm_entries_bf16_store32(count);
      case OP_ATOMIC32: return gemm_entries_bf16_atomic32(count);
      case OP_ATOMIC16: return gemm_entries_bf16_atomic16(count);
    }
  } else if (dt == IRIS_DTYPE_F16) {
    switch (op) {
      case OP_STORE16: return gemm_entries_f16_store16(count);
      case OP_STORE32: return gemm_entries_f16_store32(count);
      case OP_ATOMIC32: return gemm_entries_f16_atomic32(count);
      case OP_ATOMIC16: return gemm_entries_f16_atomic16(count);
    }
  } else if (dt == IRIS_DTYPE_F32) {
    switch (op) {
      case OP_STORE32: return gemm_entries_f32_store32(count);
      case OP_ATOMIC32: return gemm_entries_f32_atomic32(count);
    }
  }
  *count = 0;
  return nullptr;
}

// The plain build (every wave fetches its share) of the tile shape of `e`, an
// entry with fetching waves; null if `e` has none or the list holds no such build.
const GemmKernelEntry* plain_twin(const GemmKernelEntry* list, int count, const GemmKernelEntry& e) {
  if (e.fetch_waves == 0) return nullptr;
  for (int i = 0; i < count; ++i)
    if (list[i].dma && list[i].fetch_waves == 0 && list[i].cm == e.cm && list[i].cn == e.cn && list[i].wm == e.wm &&
        list[i].wn == e.wn)
      return &list[i];
  return nullptr;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// 16-byte vector access on a row-major [rows, cols] view of `es`-byte elements
bool vec_ok(const void* base, int64_t stride_m, int64_t stride_n, int es) {
  return stride_n == 1 && aligned16(base) && ((stride_m * es) % 16) == 0;
}

struct Plan {
  const GemmKernelEntry* entry = nullptr;
  GemmKArgs k{};
  int fused_reduce = 0;  // ONE_SHOT, CONSUME on its own or IRIS_PHASE_TWO_KERNELS: follow with the reduce kernel
  int in_program = 0;    // ONE_SHOT, IRIS_PHASE_FUSED: the build of the kernel that reduces each tile itself
  // the few-rows kernel instead of a table entry, one workgroup per 16 columns
  GemmKernelFn skinny = nullptr;
  int skinny_grid = 0, skinny_grid_y = 1, skinny_lds = 0;
  int skinny_rb = 1, skinny_cb = 1;  // blocks of 16 rows / 16 columns a workgroup of the few-rows kernel takes
  // a second launch of the entry's split-K build behind the first: the tiles of the last round, K shared out
  // over the programs that round would leave idle
  int last_round = 0;
  GemmKArgs k_last{};
  // the build that numbers its flags in a grid of its own (blocks of the caller's tiles, or a range of its columns)
  int remap_flags = 0;
  // a second plan behind this one: the columns of tiles this one leaves out
  std::shared_ptr<Plan> rest;
};

int dbg() {
  static int v = std::getenv("IRIS_AMD_DEBUG") ? 1 : 0;
  return v;
}

// A few rows: the product is a stream over B, and the kernel built for that
// takes it when the operands allow the 16-byte fetches, the logical tile
// covers every row, the tiles' arrival counters have a home, and (with more
// than 16 rows: two workgroups per 16 columns) every workgroup finds a place
// on the device at once, so that B comes from HBM once.  Fills the plan and
// returns true when the launch qualifies.
bool plan_few_rows(const iris_gemm_args& a, int op, bool dma_ok, Plan* plan) {
  GemmKArgs& k = plan->k;
  const int64_t lim = (int64_t)1 << 31;
  // Up to 32 rows: a workgroup per 16 rows x 16 columns.  Up to 64 rows of a long K, where the persistent
  // kernel would split K and pay for the hand-over: 32 rows x 16 columns a workgroup, as long as one round of
  // workgroups covers the matrix ([64,4096] x [4096,1376]: 172 workgroups, 11.5 us against 12.7).
  int rb = 1, cb = 1;
  if (a.M > SKINNY_MAX_ROWS) rb = 2;
  const int m_blocks = (a.M + SKINNY_ROWS * rb - 1) / (SKINNY_ROWS * rb);
  const int n_blocks = (a.N + SKINNY_COLS * cb - 1) / (SKINNY_COLS * cb);
  // fetches in flight per wave: enough for the whole K range, 8 blocks at most (4 with two blocks of columns:
  // LDS holds no more)
  const int per_wave = ((a.K + 63) / 64 + SKINNY_WAVES - 1) / SKINNY_WAVES;
  int un = per_wave <= 2 ? 2 : per_wave <= 4 ? 4 : 8;
  if (cb == 2 && un > 4) un = 4;
  const int wide = SKINNY_COLS * cb;
  const bool counters = (m_blocks == 1 && (a.block_n <= wide || a.N <= wide)) || k.flag_mode == 0 ||
                        (a.locks && k.total_tiles <= a.num_sms);
  bool room = true;
  if (rb > 1) {
    room = (int64_t)m_blocks * n_blocks <= (int64_t)current_cu_count() && a.M <= SKINNY_MID_MAX_ROWS &&
           a.K >= SKINNY_MID_MIN_K;
  } else if (m_blocks > 1) {
    const int per_cu = 160 * 1024 / skinny_lds_bytes(un) > 4 ? 4 : 160 * 1024 / skinny_lds_bytes(un);
    room = (int64_t)m_blocks * n_blocks <= (int64_t)current_cu_count() * per_cu;
  }
  const bool ok = room && a.K > 0 && dma_ok && !plan->in_program && a.block_m >= a.M && (a.block_n % wide) == 0 &&
                  !a.mm_begin_timestamp && !a.mm_end_timestamp && (a.split_k == 0 || a.split_k == 1) && counters &&
                  skinny_lds_bytes(un, rb, cb) <= 160 * 1024 &&
                  ((int64_t)SKINNY_ROWS * rb * a.stride_am + a.K) * 2 < lim &&
                  ((int64_t)wide * a.stride_bn + a.K) * 2 < lim;
  if (!ok) return false;
  const bool a_lds = rb > 1 || (a.M >= SKINNY_A_VIA_LDS_ROWS && a.K >= SKINNY_A_VIA_LDS_K);
  plan->skinny = gemm_skinny_kernel_for(a.ab_dtype, op, un, a_lds, rb, cb);
  if (!plan->skinny) return false;
  plan->skinny_lds = skinny_lds_bytes(un, rb, cb);
  plan->skinny_grid = n_blocks;
  plan->skinny_grid_y = m_blocks;
  plan->skinny_rb = rb;
  plan->skinny_cb = cb;
  k.split_k = 1;
  k.locks = a.locks;
  return true;
}

// Split-K and stream-K.  The owner of a tile waits for the programs that hold
// its other parts, so every part needs a program of its own that is resident
// at the same time: no more programs than the device has CUs.
hipError_t plan_split(const iris_gemm_args& a, const GemmKernelEntry& pick, bool in_program, GemmKArgs* kp) {
  GemmKArgs& k = *kp;
  k.split_k = 1;
  k.split_q = k.split_r = 0;
  k.partials = a.partials;
  k.locks = a.locks;
  k.partial_stride = a.partials_slot_elems;
  k.status = a.status;
  k.timeout = a.spin_timeout_ticks ? a.spin_timeout_ticks : 200000000ull;  // 2 s at 100 MHz
  k.stream_k = 0;
  if (a.split_k < 0 && a.split_k != IRIS_GEMM_SPLIT_STREAM_K) return hipErrorInvalidValue;
  if (a.split_handover < IRIS_GEMM_HANDOVER_AUTO || a.split_handover > IRIS_GEMM_HANDOVER_PAIR)
    return hipErrorInvalidValue;
  const int nk = (a.K + pick.bk - 1) / pick.bk;
  // the rules below were measured on K-steps of 64: `d` such steps to one of this tile
  const int d = pick.bk > 64 ? pick.bk / 64 : 1;
  if (in_program) {
    // the program that computes a tile also reduces it: K is never shared out
    return (a.split_k > 1 || a.split_k == IRIS_GEMM_SPLIT_STREAM_K) ? hipErrorInvalidValue : hipSuccess;
  }
  if (a.split_k != 1 && a.partials && a.locks) {
    const bool resident = a.num_sms <= current_cu_count();
    const bool any_way = resident && pick.splitk && pick.fn_split && k.sub_m == 1 && k.sub_n == 1 &&
                         (reinterpret_cast<uintptr_t>(a.partials) & 15) == 0 && (a.partials_slot_elems % 4) == 0;
    // Two parts of a 128-accumulator tile can meet with half a partial tile each (the pair hand-over: each part
    // keeps the accumulators of the waves it owns), so a slot of half a tile is enough for them; that is what a
    // caller who holds tiles half as wide has ([8192,14336] x [14336,448] in 256 x 64 tiles, run as 256 x 128).
    const bool pair_ok = any_way && !pick.split_owner && (pick.wm * pick.wn) % 2 == 0 &&
                         a.partials_slot_elems * 2 >= (int64_t)pick.cm * pick.cn;
    const bool possible = any_way && a.partials_slot_elems >= (int64_t)pick.cm * pick.cn;
    // Stream-K: every program takes the same number of K-steps (within one).
    // A run of at least four steps keeps the parts of a tile few.
    const int64_t steps = (int64_t)k.total_tiles * nk;
    const int run = (int)(steps / a.num_sms);
    const bool stream_ok = possible && pick.split_owner && run * d >= 4 && run >= 1 && steps < ((int64_t)1 << 30) &&
                           (nk + run - 1) / run + 1 <= 32;
    if (a.split_k == IRIS_GEMM_SPLIT_STREAM_K) {
      if (!stream_ok) return hipErrorInvalidValue;
      k.stream_k = 1;
    } else if (a.split_k > 1) {
      if (!(possible || (pair_ok && a.split_k == 2)) || a.split_k > nk || a.split_k > 64 ||
          (int64_t)k.total_tiles * a.split_k > a.num_sms)
        return hipErrorInvalidValue;
      k.split_k = a.split_k;
    } else if (possible || pair_ok) {
      if (k.total_tiles * 2 <= a.num_sms && nk * d >= 16) {
        // The hand-over of partials costs about as much as ten K-steps of a
        // small tile: as many parts as there are idle programs, at least four
        // K-steps each, and a K loop shorter than 32 steps is only split in
        // four or more parts (measured on [M, 1376] x [1376, 4096], 22 steps of
        // 128 x 128 tiles: 4 parts 16.4 against 19.5 us unsplit at 128 rows,
        // 2 parts 25.9 against 20.2 at 512).
        int sk = a.num_sms / k.total_tiles;
        if (sk > nk * d / 4) sk = nk * d / 4;
        if (sk > 16) sk = 16;
        if (!possible && sk > 2) sk = 2;  // (slots of half a tile: two parts)
        if (sk >= 4 || (sk > 1 && nk * d >= 32)) {
          k.split_k = sk;
        }
      }
      // Stream-K is only taken on request.  With the plain four-wave tiles it beat both the
      // unsplit and the split launch where the tiles left programs idle and the walk was long
      // (132 tiles of 64 steps on 256 programs: -17 %).  The tiles with fetching waves made
      // the K-steps a quarter shorter and left the hand-over as it was: on the same shapes
      // stream-K now ties with split-K (66 tiles: 27.9 against 27.6 us in three parts) or
      // loses (88 tiles: 33.2 against 31.9 in two parts; 132 tiles: 41.0 against 37.6 unsplit;
      // more tiles than programs: 80 against 54).  Nor does it pay where the walk is long and the last round
      // of tiles leaves most programs idle ([8192,36864] x [36864,576] in 288 tiles of 256 x 64 on 256
      // programs: 940 against 805 us): programs that start at different depths of K no longer fetch the
      // panels their neighbours fetch at the same time, and the operands come from HBM several times over.
    }
  } else if (a.split_k > 1 || a.split_k == IRIS_GEMM_SPLIT_STREAM_K) {
    return hipErrorInvalidValue;  // forced, but no workspace
  }
  if (k.split_k > 1) {
    k.split_q = nk / k.split_k;
    k.split_r = nk % k.split_k;
    // Many parts: every part reduces and stores a slice of the tile, instead
    // of the first part reading all the others' partials one after another.
    // Few parts: the owner's way, which has one hand-over less on its critical
    // path (measured on [128, 4096] x [4096, 1376] with 128 x 128 tiles: 16
    // parts 16.6 against 26.7 us, 8 parts 17.2 against 23.4, 4 parts 23.2
    // against 25.1, 2 parts 39 against 33; 64 x 64 tiles in 5 parts 16.2
    // against 14.9): sliced from eight parts up.
    // (the 128-accumulator tiles only have the sliced one)
    if (a.split_handover == IRIS_GEMM_HANDOVER_SLICED && k.split_k > pick.cm) return hipErrorInvalidValue;
    if (a.split_handover == IRIS_GEMM_HANDOVER_OWNER && !pick.split_owner) return hipErrorInvalidValue;
    const bool can_pair = k.split_k == 2 && !pick.split_owner && (pick.wm * pick.wn) % 2 == 0 &&
                          a.partials_slot_elems * 2 >= (int64_t)pick.cm * pick.cn;
    const bool can_slice = a.partials_slot_elems >= (int64_t)pick.cm * pick.cn;
    if (a.split_handover == IRIS_GEMM_HANDOVER_PAIR && !can_pair) return hipErrorInvalidValue;
    if (a.split_handover == IRIS_GEMM_HANDOVER_SLICED && !can_slice) return hipErrorInvalidValue;
    // (two parts of a 128-accumulator tile: the pair hand-over moves half the bytes of the sliced one)
    k.sliced = a.split_handover == IRIS_GEMM_HANDOVER_SLICED  ? 1
               : a.split_handover == IRIS_GEMM_HANDOVER_OWNER ? 0
               : a.split_handover == IRIS_GEMM_HANDOVER_PAIR  ? 2
               : can_pair                                     ? 2
                                                              : (!pick.split_owner || k.split_k >= 8) ? 1 : 0;
  }
  if (k.stream_k) {
    const int64_t steps = (int64_t)k.total_tiles * nk;
    k.split_q = (int)(steps / a.num_sms);
    k.split_r = (int)(steps % a.num_sms);
  }
  return hipSuccess;
}

// The launch's divisors as multiply-high constants, and how its items are dealt to the XCDs.
void launch_constants(const iris_gemm_args& a, const GemmKernelEntry& pick, GemmKArgs* kp) {
  GemmKArgs& k = *kp;
  const int nk = (a.K + pick.bk - 1) / pick.bk;
  const uint64_t items = (uint64_t)k.total_tiles * k.sub_m * k.sub_n + 1;
  k.tile_divs = make_tile_divs(k.num_pid_m, k.num_pid_n, k.G);
  k.div_subs = make_fast_div((uint32_t)(k.sub_m * k.sub_n), items);
  k.div_sub_n = make_fast_div((uint32_t)k.sub_n, items);
  k.div_split = make_fast_div((uint32_t)k.split_k, (uint64_t)a.num_sms + 1);
  k.div_nk = make_fast_div((uint32_t)(nk > 0 ? nk : 1), (uint64_t)k.total_tiles * (nk > 0 ? nk : 1) + 1);
  // Fewer (tile, part) items than programs: deal them to the XCDs evenly, in
  // consecutive runs, instead of filling the first XCDs and idling the rest.
  // (under stream-K every program has a run: the reference's XCD remap stays)
  const int64_t work = (int64_t)k.total_tiles * k.split_k;
  // parts of 32 K-steps or more: the programs part by part (see GemmKArgs::part_major; the short walks of
  // the decoder shapes were tuned tile by tile and stay so)
  k.part_major = (k.split_k > 1 && !k.stream_k && nk / k.split_k >= 32) ? k.total_tiles : 0;
  k.xcd_per = 0;
  if (!k.stream_k && a.num_xcds > 1 && work < a.num_sms) k.xcd_per = (int)((work + a.num_xcds - 1) / a.num_xcds);
  // L2 prefetch hints for long walks over K (the tiles with fetching waves read them): an XCD's share of a round
  // of tiles is a block of `rows` x `cols` neighbouring tiles, whose CUs share the A panels `cols` ways and the B
  // panels `rows` ways.  They pay on the 64-column tiles, whose K-steps are short enough to be bound by how
  // long a stage takes to arrive from HBM ([8192,14336] x [14336,448] in 256 x 64 tiles: 175 -> 161 us eight
  // steps ahead, 155 sixteen ahead); the wider tiles' steps are bound by the matrix cores' power budget on real
  // data and gain nothing (256 x 128: 427 -> 440 us on N(0, 0.02) data, 408 -> 380 us on zeros).
  // Staggered start (see GemmKArgs::stagger_groups): the unsplit eight-wave 256 x 256 tile, when every program has
  // two tiles or more, so that there are epilogues whose store bursts the stagger keeps apart (a launch of one
  // tile per program would only end later).  Two groups, 8 x 576 clocks = 2 us apart: [8192,1024] x [1024,8192]
  // 90.2 -> 87.6 us on zeros, 113.7 -> 112.0 on N(0, 0.02) data; [8192,1536] x [1536,4096] stored to eight ranks
  // 185.6 -> 182.6; [8192,7168] x [7168,4096] (two tiles a program, 112 K-steps each) unchanged.  Only for walks of
  // at most 64 K-steps: on a long walk the epilogues are little beside the K loop, and programs that fetch the
  // same panels two microseconds apart find less of them in their XCD's L2 ([8192,36864] x [36864,4608]: +2 %).
  k.stagger_groups = k.stagger_sleeps = 0;
  if (pick.cm == 256 && pick.cn == 256 && pick.wm * pick.wn == 8 && pick.fetch_waves == 0 && k.split_k == 1 &&
      !k.stream_k && a.num_xcds > 1 && k.sub_m == 1 && k.sub_n == 1 && k.total_tiles >= 2 * (int64_t)a.num_sms &&
      a.num_sms >= 2 * a.num_xcds && nk <= 64) {
    k.stagger_groups = 2;
    k.stagger_sleeps = 8;
  }
  k.pf_dist = k.pf_sa = k.pf_sb = 0;
  const int pf_dist = 8;
  if (pick.fetch_waves > 0 && pick.cm == 256 && pick.cn == 64 && !k.stream_k && k.sub_m == 1 && k.sub_n == 1 && nk >= 16 * pf_dist &&
      a.num_xcds > 1) {
    const int64_t per_xcd = k.xcd_per > 0 ? k.xcd_per : (k.num_sms / a.num_xcds);
    int64_t tiles_per_xcd = k.split_k > 1 ? (per_xcd + k.split_k - 1) / k.split_k : per_xcd;
    if (k.part_major > 0) tiles_per_xcd = per_xcd;  // (part by part: an XCD's programs are neighbouring tiles)
    const int g_rows = k.G < k.num_pid_m ? k.G : k.num_pid_m;
    int64_t cols = tiles_per_xcd / (g_rows > 0 ? g_rows : 1);
    if (cols < 1) cols = 1;
    if (cols > k.num_pid_n) cols = k.num_pid_n;
    int64_t rows = tiles_per_xcd / cols;
    if (rows < 1) rows = 1;
    // one touch instruction per operand covers 64 rows of the share: the share must thin the panel out enough
    if (cols * 64 >= pick.cm && rows * 64 >= pick.cn && cols * rows > 1) {
      k.pf_dist = pf_dist;
      k.pf_sa = (int)cols;
      k.pf_sb = (int)rows;
    }
  }
  // The same hints for the eight-wave 256 x 256 tile, whose every wave also loads: they are a build of their own
  // (GemmKernelEntry::fn_touch), taken where a round of tiles streams its operands from HBM.  Looping
  // [8192,14336] x [14336,2048] (294 MB of operands, one tile a program): 358 -> 339 us three steps ahead, 345 four,
  // 352 eight (an XCD's share of eight steps, 3 MB, no longer stays in its 4 MB L2), 411 when every program touches
  // all its lines instead of its share; on zeros 337 -> 296.  [8192,28672] x [28672,4096] (two tiles a program)
  // 1393 -> 1344.  Where the operands stay in the 256 MB last-level cache the touches only add L2 requests:
  // [8192,12288] x [12288,2048] (252 MB) +3 %, [8192,7168] x [7168,4096] +2 %; and an XCD whose tiles are two rows
  // of sixteen (group size 2) fetches half as many lines again per step and is bound by that, not by latency
  // ([8192,36864] x [36864,4608]: +5 %).  So: at least 272 MB of operands per round of tiles, and an XCD block of at
  // least four tiles either way.
  if (a.touch_ahead != IRIS_GEMM_TOUCH_OFF && pick.fn_touch && k.split_k == 1 && !k.stream_k && k.sub_m == 1 && k.sub_n == 1) {
    const int64_t per_xcd = a.num_xcds > 1 ? (k.xcd_per > 0 ? k.xcd_per : (k.num_sms / a.num_xcds)) : k.num_sms;
    const int g_rows = k.G < k.num_pid_m ? k.G : k.num_pid_m;
    int64_t cols = per_xcd / (g_rows > 0 ? g_rows : 1);
    if (cols < 1) cols = 1;
    if (cols > k.num_pid_n) cols = k.num_pid_n;
    int64_t rows = per_xcd / cols;
    if (rows < 1) rows = 1;
    // (the kernel takes its share of a panel's rows with a mask: powers of two)
    int sa = 1, sb = 1;
    while (sa * 2 <= cols && sa < 64) sa *= 2;
    while (sb * 2 <= rows && sb < 64) sb *= 2;
    const int64_t rounds = (k.total_tiles + k.num_sms - 1) / k.num_sms;
    const int64_t operand_bytes = ((int64_t)a.M + a.N) * a.K * 2;
    const bool streams = nk >= 32 && sa >= 4 && sb >= 4 && operand_bytes >= rounds * ((int64_t)272 << 20);
    if (a.touch_ahead == IRIS_GEMM_TOUCH_ON || streams) {
      k.pf_dist = 3;
      k.pf_sa = sa;
      k.pf_sb = sb;
    }
  }
}

// Validate `a` and build the launch plan.  Returns hipSuccess,
// hipErrorInvalidValue, or a pseudo-success with entry == nullptr when there
// is no GEMM work to do.
hipError_t make_plan_body(const iris_gemm_args& a, Plan* plan);

// A long GEMM whose tiles are a few more than a multiple of the programs spends a whole round on those few:
// 288 tiles on 256 programs take two rounds for 1.125 rounds of work.  Where a tile's walk over K is long
// and the caller brought the split-K workspace, the plan becomes two launches on the stream: the full rounds
// as they are, then the tiles of the last round with K shared out over the programs it would leave idle
// (every part at the same depths of K as its neighbours', so the operand panels are still fetched together;
// stream-K, which would even out the rounds too, loses that and is slower here).
void split_last_round(const iris_gemm_args& a, Plan* plan) {
  GemmKArgs& k = plan->k;
  const GemmKernelEntry* e = plan->entry;
  plan->last_round = 0;
  if (!e || plan->skinny || plan->in_program || k.split_k != 1 || k.stream_k || k.sub_m != 1 || k.sub_n != 1) return;
  if (k.merge_m * k.merge_n > 1 || plan->remap_flags) return;  // (the second launch would raise flags of its own grid)
  if (a.split_k != 0 || a.variant != 0 || a.mm_begin_timestamp || a.mm_end_timestamp) return;
  if (!a.partials || !a.locks || !e->splitk || !e->fn_split || k.num_sms != a.num_sms) return;
  if (a.num_sms > current_cu_count() || a.partials_slot_elems < (int64_t)e->cm * e->cn) return;
  const int programs = a.num_sms, rounds = k.total_tiles / programs, last = k.total_tiles - rounds * programs;
  if (rounds < 1 || last == 0 || last * 2 > programs) return;
  const int nk = (a.K + e->bk - 1) / e->bk;
  // parts of at least 32 K-steps: the build with fetching waves of a split 128-accumulator tile needs them
  // to pay for its spills, and the second launch's start must be little beside a part's walk
  int parts = programs / last;
  if (parts > 16) parts = 16;
  if (parts > nk / 32) parts = nk / 32;
  if (parts < 2) return;
  iris_gemm_args forced = a;
  forced.split_k = parts;
  GemmKArgs t = k;
  t.tile_base = rounds * programs;
  t.total_tiles = last;
  if (plan_split(forced, *e, false, &t) != hipSuccess || t.split_k != parts) return;
  launch_constants(forced, *e, &t);
  k.total_tiles = rounds * programs;
  launch_constants(a, *e, &k);
  plan->k_last = t;
  plan->last_round = 1;
}

// How a plain launch's tiles are blocked: merge_m x merge_n of the caller's tiles as one 256 x 256 or 256 x 128
// tile, when the `tiles_n` columns of tiles suffice for it.  Returns false for "the caller's tiles as they are".
bool choose_merge(const iris_gemm_args& a, int64_t tiles_n, int* merge_m, int* merge_n) {
  *merge_m = *merge_n = 1;
  const int64_t tiles_m = (a.M + a.block_m - 1) / a.block_m;
  const int mm = 256 / a.block_m;  // 1 or 2
  const int64_t rows = (tiles_m + mm - 1) / mm;
  // 256 x 256 or 256 x 128, whichever finishes first among those that give (almost) every program a tile: rounds
  // of tiles times the tile's time (a 256 x 256 tile does twice the work at 1.25 times the rate, as measured)
  double best = 0;
  for (int width = 256; width >= 128; width /= 2) {
    const int mn = width / a.block_n;
    const int64_t merged_tiles = rows * ((tiles_n + mn - 1) / mn);
    // (seven programs in eight busy is enough: [8192,14336] x [14336,1792] as 224 tiles of 256 x 256 in one
    // round against 448 of 256 x 128 in two)
    if (mm * mn == 1 || merged_tiles * 8 < (int64_t)a.num_sms * 7) continue;
    const double cost = (double)((merged_tiles + a.num_sms - 1) / a.num_sms) * (width == 256 ? 1.6 : 1.0);
    if (best == 0 || cost < best) best = cost, *merge_m = mm, *merge_n = mn;
  }
  if (*merge_m * *merge_n > 1) return true;
  if (!a.partials || !a.locks || a.K < 4096) return false;
  // No block of the caller's tiles gives every program one.  Blocks that give every OTHER program one do, with
  // each block's K range shared by two programs; their hand-over takes slots of half a (merged) tile, which is
  // what the caller's workspace holds when the blocks are pairs of its tiles ([8192,14336] x [14336,448] in
  // 256 x 64 tiles: 175 -> 114 us).
  for (int width = 256; width >= 128; width /= 2) {
    const int mn = width / a.block_n;
    const int64_t merged_tiles = rows * ((tiles_n + mn - 1) / mn);
    if (mm * mn == 1 || mn < 1) continue;
    if (merged_tiles * 2 > a.num_sms || merged_tiles * 16 < (int64_t)a.num_sms * 7) continue;
    if (a.partials_slot_elems * 2 < (int64_t)256 * width) continue;
    *merge_m = mm, *merge_n = mn;
    return true;
  }
  return false;
}

// The plan for the caller's tiles blocked merge_m x merge_n; false when the launcher has no kernel for it.
bool plan_merged(const iris_gemm_args& a, int merge_m, int merge_n, Plan* plan) {
  iris_gemm_args b = a;
  b.block_m = a.block_m * merge_m;
  b.block_n = a.block_n * merge_n;
  Plan merged;
  const hipError_t err = make_plan_body(b, &merged);
  // (only the persistent kernels publish merged tiles: unsplit, or split in parts)
  const bool unsplit = merged.k.split_k == 1 && merged.entry && merged.entry->fn_merged;
  const bool parts = merged.k.split_k > 1 && merged.entry && merged.entry->fn_split_merged;
  if (err != hipSuccess || !merged.entry || merged.skinny || !(unsplit || parts) || merged.k.stream_k || merged.in_program)
    return false;
  *plan = merged;
  plan->remap_flags = 1;
  plan->k.merge_m = merge_m;
  plan->k.merge_n = merge_n;
  plan->k.flag_num_pid_m = (a.M + a.block_m - 1) / a.block_m;
  plan->k.flag_num_pid_n = (a.N + a.block_n - 1) / a.block_n;
  plan->k.flag_pn_base = 0;
  if (merge_m * merge_n > 1) split_last_round(b, plan);
  return true;
}

// `a` restricted to columns [col0, col0 + cols) of B and of the output (whole tiles of the caller).
iris_gemm_args column_range(const iris_gemm_args& a, int64_t col0, int64_t cols) {
  iris_gemm_args b = a;
  b.N = (int32_t)cols;
  b.b = static_cast<const char*>(a.b) + col0 * a.stride_bn * 2;
  if (a.epilogue == IRIS_EPI_ALL_SCATTER) {
    // (the launcher adds cur_rank * N columns to c_global: of the range's N, so the difference goes in here;
    // the pointer is only ever used with that offset added)
    const int64_t shift = (int64_t)a.cur_rank * (a.N - cols) + col0;
    b.c_global = static_cast<char*>(a.c_global) + shift * a.stride_cn_global * dtype_size(a.c_global_dtype);
  } else {
    b.c = static_cast<char*>(a.c) + col0 * a.stride_cn * dtype_size(a.c_dtype);
    b.c_global = static_cast<char*>(a.c_global) + col0 * a.stride_cn_global * dtype_size(a.c_global_dtype);
  }
  return b;
}

// The plan of a launch.  A caller's tile that is narrow or short (the reference scripts' 256 x 64; 128 x 128)
// makes a large GEMM wait for its operands: a 256 x 64 tile fetches 256 rows of A every K-step for 64 columns'
// worth of work.  Where there are enough of them, the launch computes a block of the caller's tiles as one
// 256 x 128 or 256 x 256 tile and raises each one's flag: tile ids and flags are the caller's, which program
// computes a tile was never observable ([8192,8192] x [8192,1024] in 256 x 64 tiles: 739-762 -> 928 TFLOP/s
// over the eight ranks of the reference's 07 benchmark).
hipError_t make_plan_units(const iris_gemm_args& a, Plan* plan);

// fp32 operands (the reference scripts' --datatype fp32; the output is fp32 too): the kernels count K and the
// operands' strides in 16-bit units, two to an element, and everything between this function and the MFMAs
// (loaders, slabs, stages, K tail, the 2 GiB windows of the buffer descriptors) is the 16-bit kernels' as it is.
hipError_t make_plan(const iris_gemm_args& a, Plan* plan) {
  if (a.ab_dtype != IRIS_DTYPE_F32) return make_plan_units(a, plan);
  const int64_t lim = (int64_t)1 << 30;
  if (a.K < 0 || a.K >= lim) return hipErrorInvalidValue;
  iris_gemm_args b = a;
  b.K = 2 * a.K;
  b.stride_am = 2 * a.stride_am;
  b.stride_ak = 2 * a.stride_ak;
  b.stride_bk = 2 * a.stride_bk;
  b.stride_bn = 2 * a.stride_bn;
  return make_plan_units(b, plan);
}

hipError_t make_plan_units(const iris_gemm_args& a, Plan* plan) {
  const bool plain = a.variant == 0 && a.split_k == 0 && !a.mm_begin_timestamp && !a.mm_end_timestamp &&
                     !(a.epilogue == IRIS_EPI_ONE_SHOT && a.phase != IRIS_PHASE_PRODUCE) &&
                     a.epilogue != IRIS_EPI_ATOMIC_ADD && a.num_sms > 0 && (a.block_m == 128 || a.block_m == 256) &&
                     (a.block_n == 64 || a.block_n == 128) && a.M >= 256;
  const bool plain_two_kernels = a.variant == 0 && a.split_k == 0 && !a.mm_begin_timestamp && !a.mm_end_timestamp &&
                                 a.epilogue == IRIS_EPI_ONE_SHOT && a.phase == IRIS_PHASE_TWO_KERNELS && a.num_sms > 0 &&
                                 (a.block_m == 128 || a.block_m == 256) && (a.block_n == 64 || a.block_n == 128) &&
                                 a.M >= 256;
  if (plain || plain_two_kernels) {
    const int64_t tiles_n = (a.N + a.block_n - 1) / a.block_n;
    int merge_m = 1, merge_n = 1;
    if (choose_merge(a, tiles_n, &merge_m, &merge_n)) {
      if (plan_merged(a, merge_m, merge_n, plan)) return hipSuccess;
    } else if (plain && a.N % a.block_n == 0) {
      // The columns of tiles are one or a few too many for a blocking that pays: [8192,36864] x [36864,576] is nine
      // columns of 256 x 64 tiles, eight of which block into 128 pairs with K in two parts.  The launch then
      // takes the columns that block first and the remaining ones as a launch of their own behind it.
      for (int width = 256; width >= 128; width /= 2) {
        const int mn = width / a.block_n;
        const int64_t main_n = tiles_n / mn * mn, rest_n = tiles_n - main_n;
        if (mn < 2 || main_n == 0 || rest_n == 0 || rest_n * 4 > main_n) continue;
        const iris_gemm_args am = column_range(a, 0, main_n * a.block_n);
        if (!choose_merge(am, main_n, &merge_m, &merge_n)) continue;
        Plan first;
        if (!plan_merged(am, merge_m, merge_n, &first)) continue;
        const iris_gemm_args ar = column_range(a, main_n * a.block_n, rest_n * a.block_n);
        auto rest = std::make_shared<Plan>();
        // (the remaining columns as the caller's tiles; their flags sit at their place in the caller's grid)
        if (!plan_merged(ar, 1, 1, rest.get())) continue;
        first.k.flag_num_pid_n = (int)tiles_n;
        rest->k.flag_num_pid_n = (int)tiles_n;
        rest->k.flag_pn_base = (int)main_n;
        *plan = first;
        plan->rest = rest;
        return hipSuccess;
      }
    }
  }
  const hipError_t err = make_plan_body(a, plan);
  plan->k.merge_m = plan->k.merge_n = 1;
  plan->k.flag_num_pid_m = plan->k.num_pid_m;
  plan->k.flag_num_pid_n = plan->k.num_pid_n;
  plan->k.flag_pn_base = 0;
  if (err == hipSuccess) split_last_round(a, plan);
  return err;
}

hipError_t make_plan_body(const iris_gemm_args& a, Plan* plan) {
  if (a.M < 0 || a.N < 0 || a.K < 0) return hipErrorInvalidValue;
  if (a.block_m <= 0 || a.block_n <= 0 || a.group_size_m <= 0) return hipErrorInvalidValue;
  if (a.num_sms <= 0 || a.num_xcds <= 0 || (a.num_sms % a.num_xcds) != 0) return hipErrorInvalidValue;
  if (a.world_size <= 0 || a.cur_rank < 0 || a.cur_rank >= a.world_size) return hipErrorInvalidValue;
  if (a.world_size > 1 && a.heap_bases == nullptr) return hipErrorInvalidValue;
  if (a.ab_dtype != IRIS_DTYPE_BF16 && a.ab_dtype != IRIS_DTYPE_F16 && a.ab_dtype != IRIS_DTYPE_F32)
    return hipErrorInvalidValue;

  int op, out_dt;
  GemmKArgs& k = plan->k;
  k = GemmKArgs{};
  switch (a.epilogue) {
    case IRIS_EPI_ALL_SCATTER:
      if (!a.c_global) return hipErrorInvalidValue;
      out_dt = a.c_global_dtype;
      op = out_dt == IRIS_DTYPE_F32 ? OP_STORE32 : OP_STORE16;
      k.out = static_cast<char*>(a.c_global) +
              (int64_t)a.cur_rank * a.N * a.stride_cn_global * dtype_size(out_dt);
      k.som = a.stride_cm_global;
      k.son = a.stride_cn_global;
      k.dest_all = 1;
      k.flag_mode = a.notify ? 1 : 0;
      break;
    case IRIS_EPI_ATOMIC_ADD:
      if (!a.c_global) return hipErrorInvalidValue;
      out_dt = a.c_global_dtype;
      op = out_dt == IRIS_DTYPE_F32 ? OP_ATOMIC32 : OP_ATOMIC16;
      k.out = static_cast<char*>(a.c_global);
      k.som = a.stride_cm_global;
      k.son = a.stride_cn_global;
      k.dest_all = 1;
      k.flag_mode = 0;
      break;
    case IRIS_EPI_ONE_SHOT:
      if (!a.c || !a.c_global) return hipErrorInvalidValue;
      if (a.phase != IRIS_PHASE_PRODUCE && a.phase != IRIS_PHASE_CONSUME && a.phase != IRIS_PHASE_FUSED &&
          a.phase != IRIS_PHASE_TWO_KERNELS)
        return hipErrorInvalidValue;
      out_dt = a.c_dtype;
      op = out_dt == IRIS_DTYPE_F32 ? OP_STORE32 : OP_STORE16;
      k.out = static_cast<char*>(a.c);
      k.som = a.stride_cm;
      k.son = a.stride_cn;
      k.dest_all = 0;
      k.flag_mode = 2;
      plan->in_program = a.phase == IRIS_PHASE_FUSED ? 1 : 0;
      plan->fused_reduce = (a.phase == IRIS_PHASE_CONSUME || a.phase == IRIS_PHASE_TWO_KERNELS) ? 1 : 0;
      if (!(a.phase & IRIS_PHASE_PRODUCE)) return hipSuccess;  // consumer only: no GEMM
      if (plan->in_program) {
        const int gdt = a.c_global_dtype;
        if (gdt != IRIS_DTYPE_F32 && gdt != IRIS_DTYPE_F16 && gdt != IRIS_DTYPE_BF16) return hipErrorInvalidValue;
        k.cg = static_cast<char*>(a.c_global);
        k.sgm = a.stride_cm_global;
        k.sgn = a.stride_cn_global;
        k.cg_dt = gdt;
      }
      break;
    default:
      return hipErrorInvalidValue;
  }
  if (out_dt != IRIS_DTYPE_F32 && out_dt != a.ab_dtype) return hipErrorInvalidValue;
  if (a.touch_ahead != IRIS_GEMM_TOUCH_AUTO && a.touch_ahead != IRIS_GEMM_TOUCH_ON && a.touch_ahead != IRIS_GEMM_TOUCH_OFF)
    return hipErrorInvalidValue;
  if (a.flag_sem != IRIS_FLAG_SEM_WRITE_THROUGH && a.flag_sem != IRIS_FLAG_SEM_RELEASE_ACQUIRE)
    return hipErrorInvalidValue;
  if (k.flag_mode != 0 && a.flag_sem == IRIS_FLAG_SEM_RELEASE_ACQUIRE) k.flag_mode |= FLAG_RELEASE;
  if (k.flag_mode != 0 && a.world_size > 1 && !a.tile_completed) return hipErrorInvalidValue;
  if ((k.flag_mode & FLAG_MODE_MASK) == 1 && !a.tile_completed) return hipErrorInvalidValue;
  if (a.M == 0 || a.N == 0) return hipSuccess;  // nothing to compute
  if (!a.a || !a.b) {
    if (a.K > 0) return hipErrorInvalidValue;
  }

  k.a = static_cast<const char*>(a.a);
  k.b = static_cast<const char*>(a.b);
  k.flags = a.tile_completed;
  k.heap_bases = a.heap_bases;
  k.ts_begin = a.mm_begin_timestamp;
  k.ts_end = a.mm_end_timestamp;
  k.sam = a.stride_am;
  k.sak = a.stride_ak;
  k.sbk = a.stride_bk;
  k.sbn = a.stride_bn;
  k.M = a.M;
  k.N = a.N;
  k.K = a.K;
  k.BM = a.block_m;
  k.BN = a.block_n;
  k.G = a.group_size_m;
  k.num_sms = a.num_sms;
  k.num_xcds = a.num_xcds;
  k.cur_rank = a.cur_rank;
  k.ws = a.world_size;
  k.num_pid_m = (a.M + a.block_m - 1) / a.block_m;
  k.num_pid_n = (a.N + a.block_n - 1) / a.block_n;
  k.total_tiles = k.num_pid_m * k.num_pid_n;
  k.sys = a.scope == IRIS_SCOPE_SYSTEM;
  k.vec_out = vec_ok(k.out, k.som, k.son, dtype_size(out_dt)) ? 1 : 0;
  if (plan->in_program) {
    // 16-byte strips in the in-program reduce: aligned rows on both sides, tile
    // origins on strip boundaries, rows at least as long as the matrix is wide
    // and 32-bit offsets inside a tile
    const int ies = dtype_size(out_dt), oes = dtype_size(k.cg_dt), ve = 16 / ies;
    k.fused_vec = k.vec_out && vec_ok(k.cg, k.sgm, k.sgn, oes) && a.block_n % ve == 0 && (a.block_n * oes) % 16 == 0 &&
                  k.som >= a.N && k.sgm >= a.N && ((int64_t)a.block_m + 64) * k.som * ies < (1ll << 31) &&
                  ((int64_t)a.block_m + 64) * k.sgm * oes < (1ll << 31);
  }

  int count = 0;
  const GemmKernelEntry* list = entries_for(a.ab_dtype, op, &count);
  if (!list) return hipErrorInvalidValue;

  // Operands fit the LDS-DMA loader when both are K-contiguous with 16-byte
  // aligned rows and K is a multiple of 8; a compute tile's rows must stay
  // within a 2 GiB window of its buffer descriptor.
  // (an fp32 launch arrives here with K and the operands' strides in 16-bit units: make_plan)
  const int unit = a.ab_dtype == IRIS_DTYPE_F32 ? 2 : 1;
  const bool dma_ok = a.stride_ak == unit && a.stride_bk == unit && (a.stride_am % 8) == 0 && (a.stride_bn % 8) == 0 &&
                      aligned16(a.a) && aligned16(a.b) && (a.K % 8) == 0 && a.stride_am > 0 && a.stride_bn > 0;
  auto fits = [&](const GemmKernelEntry& e) {
    if (!e.dma) return true;
    if (!dma_ok) return false;
    const int64_t lim = (int64_t)1 << 31;
    return ((int64_t)e.cm * a.stride_am + a.K) * 2 < lim && ((int64_t)e.cn * a.stride_bn + a.K) * 2 < lim;
  };

  if (a.variant == 0 || a.variant == IRIS_GEMM_VARIANT_FEW_ROWS) {
    if (plan_few_rows(a, op, dma_ok, plan)) return hipSuccess;
    if (a.variant == IRIS_GEMM_VARIANT_FEW_ROWS) return hipErrorInvalidValue;
  }

  const GemmKernelEntry* pick = nullptr;
  if (a.variant == IRIS_GEMM_VARIANT_PERSISTENT) {
    // the default choice among the persistent kernels
  } else if (a.variant > 0) {
    if (a.variant > count) return hipErrorInvalidValue;
    const GemmKernelEntry& e = list[a.variant - 1];
    if (!fits(e)) return hipErrorInvalidValue;
    pick = &e;
  }
  if (!pick) {
    // first entry whose compute tile divides the logical tile; the rows and
    // columns a small matrix cannot fill are not worth a tall compute tile
    for (int i = 0; i < count && !pick; ++i) {
      const GemmKernelEntry& e = list[i];
      if (!fits(e)) continue;
      if (plan->in_program && !e.fn_fused) continue;
      // (a caller's split needs a K-step per part: a tile with a deeper step may not have them)
      if (a.split_k > 1 && a.split_k > (a.K + e.bk - 1) / e.bk && e.bk > 64) continue;
      if (a.block_m % e.cm != 0 || a.block_n % e.cn != 0) continue;
      // (up to half a tall tile may be padding: its rows cost matrix-core time only, and
      // the tall tiles are the ones whose K range can be shared out over idle programs)
      if (e.cm > 64 && e.cm >= 4 * a.M) continue;
      if (e.cn > 64 && e.cn >= 4 * a.N) continue;
      // An atomic epilogue is bound by the chip's atomic rate (329 G fp32
      // adds a second, 51 us for 4096 x 4096), and while a program walks its
      // K loop it sends none: with two half tiles per logical tile the
      // second's K loop runs while the first's atomics drain (-7 % per launch).
      if ((op == OP_ATOMIC32 || op == OP_ATOMIC16) && e.cm * e.cn > 256 * 128) continue;
      pick = &e;
    }
    // otherwise the generic tile, with masked sub-tiles
    for (int i = count - 1; i >= 0 && !pick; --i)
      if (!list[i].dma && list[i].cm == 64 && list[i].cn == 64) pick = &list[i];
  }
  if (!pick) return hipErrorInvalidValue;
  if (plan->in_program && !pick->fn_fused) return hipErrorInvalidValue;
  // compute tiles per logical tile; a matrix smaller than one logical tile
  // has nothing beyond its own edge
  const int span_m = a.block_m < a.M ? a.block_m : a.M, span_n = a.block_n < a.N ? a.block_n : a.N;
  k.sub_m = (span_m + pick->cm - 1) / pick->cm;
  k.sub_n = (span_n + pick->cn - 1) / pick->cn;
  plan->entry = pick;

  const hipError_t err = plan_split(a, *pick, plan->in_program != 0, &k);
  launch_constants(a, *pick, &k);
  // (under stream-K every program has a run: the reference's XCD remap stays)
  if (err != hipSuccess || k.stream_k) return err;
  // A tile whose stages take at most half a CU's LDS runs one wave per SIMD
  // and has every instruction of a K-step on its critical path.  A launch
  // that owns the whole device (one program per CU or more) and has at least
  // two such tiles per program is given two programs per CU, each other's
  // cover: which program computes which tile is not observable, the tiles'
  // flags are.  (64 x 64 tiles, 256 -> 512 programs: [512,1376] x [1376,4096]
  // 25.0 -> 17.8 us, [2048,4096] x [4096,1376] 80 -> 65 us.)
  const int64_t items = (int64_t)k.total_tiles * k.sub_m * k.sub_n;
  // (Two programs of a tile with fetching waves are slower than one, so such a launch takes
  // the plain tile of the same shape: [512,1376] x [1376,4096] 20.6 -> 17.1 us.)
  const GemmKernelEntry* twin = a.variant > 0 ? nullptr : plain_twin(list, count, *pick);
  const bool two_ok = pick->fetch_waves == 0 || twin;
  if (!plan->in_program && k.split_k == 1 && two_ok && (twin ? twin : pick)->lds_bytes * 2 <= 160 * 1024 &&
      a.num_sms >= current_cu_count() && a.num_sms <= 2 * current_cu_count() && items >= 2 * (int64_t)a.num_sms &&
      !a.mm_begin_timestamp && !a.mm_end_timestamp) {
    k.num_sms = 2 * a.num_sms;
    if (twin) plan->entry = twin;
  }
  // (A split launch of a 128-accumulator tile runs the `_f4` build too: its split build handles one (tile, part)
  // item per program and keeps nothing live across the epilogue, which leaves it 40 registers to spare.  Before
  // that it spilled around the hand-over, now and then inside the K loop, and such launches took the plain tile:
  // [8192,12288] x [12288,512] as 128 tiles of 256 x 128 in two parts 145 us, against 131 or 181 as the spills fell.)
  return hipSuccess;
}

hipError_t ensure_lds(GemmKernelFn fn, int lds_bytes) {
  // dynamic LDS above 64 KiB must be opted into once per function and device
  static std::mutex m;
  static std::vector<std::pair<int, GemmKernelFn>> done;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  std::lock_guard<std::mutex> lock(m);
  for (const auto& d : done)
    if (d.first == dev && d.second == fn) return hipSuccess;
  err = hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (err == hipSuccess) done.emplace_back(dev, fn);
  return err;
}

iris_reduce_args reduce_args_from(const iris_gemm_args& a) {
  iris_reduce_args r{};
  r.c = a.c;
  r.c_global = a.c_global;
  r.tile_completed = a.tile_completed;
  r.heap_bases = a.heap_bases;
  r.status = a.status;
  r.M = a.M;
  r.N = a.N;
  r.stride_cm = a.stride_cm;
  r.stride_cn = a.stride_cn;
  r.stride_cm_global = a.stride_cm_global;
  r.stride_cn_global = a.stride_cn_global;
  r.block_m = a.block_m;
  r.block_n = a.block_n;
  r.group_size_m = a.group_size_m;
  r.num_sms = a.num_sms;
  r.num_xcds = a.num_xcds;
  r.cur_rank = a.cur_rank;
  r.world_size = a.world_size;
  r.c_dtype = a.c_dtype;
  r.c_global_dtype = a.c_global_dtype;
  r.scope = a.scope;
  r.wait_flags = 1;
  r.variant = 0;
  r.spin_timeout_ticks = a.spin_timeout_ticks;
  r.flag_sem = a.flag_sem;
  return r;
}

}  // namespace
}  // namespace iris_amd

using namespace iris_amd;

namespace {

// Whether the plan's launch is the build that touches lines of K-steps to come (launch_constants decides; a
// launch that splits K has no such build).
bool plan_touches(const Plan& plan) {
  const GemmKernelEntry* e = plan.entry;
  return e && !plan.skinny && !plan.in_program && plan.k.split_k == 1 && !plan.k.stream_k && plan.k.pf_dist > 0 && e->fn_touch;
}

// The build of the picked kernel that the plan launches.
GemmKernelFn plan_fn(const Plan& plan) {
  const GemmKernelEntry* e = plan.entry;
  if (plan.in_program) return e->fn_fused;
  const bool split = plan.k.split_k > 1 || plan.k.stream_k;
  const bool touch = plan_touches(plan);
  if (plan.remap_flags) return split ? e->fn_split_merged : touch ? e->fn_touch_merged : e->fn_merged;
  return split ? e->fn_split : touch ? e->fn_touch : e->fn;
}

// Enqueue what `plan` describes on `stream`.  (`args` is the caller's launch: only a reduce kernel behind the GEMM
// reads it.)
hipError_t run_plan(const Plan& plan, const iris_gemm_args& args, void* stream) {
  hipError_t err = hipSuccess;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (plan.skinny) {
    if (dbg())
      std::fprintf(stderr, "[iris_amd] gemm few-rows M=%d N=%d K=%d tiles=%d grid=%dx%d\n", plan.k.M, plan.k.N, plan.k.K,
                   plan.k.total_tiles, plan.skinny_grid, plan.skinny_grid_y);
    if (plan.skinny_lds > 64 * 1024) {
      err = ensure_lds(plan.skinny, plan.skinny_lds);
      if (err != hipSuccess) return err;
    }
    hipLaunchKernelGGL(plan.skinny, dim3(plan.skinny_grid, plan.skinny_grid_y), dim3(SKINNY_THREADS), plan.skinny_lds, s,
                       plan.k);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
  } else if (plan.entry) {
    const GemmKernelEntry* e = plan.entry;
    const GemmKernelFn fn = plan_fn(plan);
    if (e->lds_bytes > 64 * 1024) {
      err = ensure_lds(fn, e->lds_bytes);
      if (err != hipSuccess) return err;
    }
    if (dbg())
      std::fprintf(stderr, "[iris_amd] gemm %s%s M=%d N=%d K=%d tiles=%d grid=%d sub=%dx%d lds=%d\n", e->name,
                   plan.in_program ? "+reduce" : "", plan.k.M, plan.k.N, plan.k.K, plan.k.total_tiles, plan.k.num_sms,
                   plan.k.sub_m, plan.k.sub_n, e->lds_bytes);
    hipLaunchKernelGGL(fn, dim3(plan.k.num_sms), dim3(e->threads), e->lds_bytes, s, plan.k);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    if (plan.last_round) {
      if (e->lds_bytes > 64 * 1024) {
        err = ensure_lds(e->fn_split, e->lds_bytes);
        if (err != hipSuccess) return err;
      }
      if (dbg())
        std::fprintf(stderr, "[iris_amd] gemm %s: last round, tiles %d..%d in %d parts\n", e->name,
                     plan.k_last.tile_base, plan.k_last.tile_base + plan.k_last.total_tiles - 1, plan.k_last.split_k);
      hipLaunchKernelGGL(e->fn_split, dim3(plan.k_last.num_sms), dim3(e->threads), e->lds_bytes, s, plan.k_last);
      err = hipGetLastError();
      if (err != hipSuccess) return err;
    }
  }
  if (plan.rest) {
    err = run_plan(*plan.rest, args, stream);
    if (err != hipSuccess) return err;
  }
  if (plan.fused_reduce) {
    // The consumer half of the one-shot epilogue runs as a second kernel on
    // the same stream: it waits for each tile's flag, sums the partials and
    // stores the result, exactly what the tail of the reference program does
    // for that tile (gemm_one_shot_all_reduce.py:220-271).
    const iris_reduce_args r = reduce_args_from(args);
    return static_cast<hipError_t>(iris_one_shot_reduce_launch(&r, stream));
  }
  return hipSuccess;
}

}  // namespace

extern "C" int iris_gemm_launch(const iris_gemm_args* args, void* stream) {
  if (!args) return hipErrorInvalidValue;
  Plan plan;
  hipError_t err = make_plan(*args, &plan);
  if (err != hipSuccess) return err;
  return run_plan(plan, *args, stream);
}

// ---------------------------------------------------------------------------
// The launch that allocates nothing: the split-K / stream-K / few-rows
// workspace (partial tiles and their locks) lives in a device array of this
// library instead of in buffers of the caller.
// ---------------------------------------------------------------------------

namespace {

constexpr size_t NOALLOC_LOCK_BYTES = 4096;  // int32[1024]: one lock per program or tile
constexpr size_t NOALLOC_PARTIAL_BYTES =
    (size_t)IRIS_GEMM_NOALLOC_MAX_PROGRAMS * IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS * sizeof(float);
constexpr size_t NOALLOC_BYTES = NOALLOC_LOCK_BYTES + NOALLOC_PARTIAL_BYTES;

}  // namespace

// locks first, then one partial-tile slot per program.  Every device the
// library runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[NOALLOC_BYTES];

namespace {

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* p, int32_t v, int n) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) p[i] = v;
}

// Device address of `scratch` on the current device, looked up once per
// device.  (In host code the array's name is only a handle for this lookup.)
hipError_t scratch_address(unsigned char** out) {
  static std::mutex m;
  static unsigned char* ptr[64] = {};
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(m);
  if (!ptr[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (!p) return hipErrorInvalidSymbol;
    ptr[dev] = static_cast<unsigned char*>(p);
  }
  *out = ptr[dev];
  return hipSuccess;
}

}  // namespace

extern "C" int iris_gemm_launch_noalloc(const iris_gemm_args* args, void* stream) {
  if (!args) return hipErrorInvalidValue;
  if (args->num_sms > IRIS_GEMM_NOALLOC_MAX_PROGRAMS) {
    std::fprintf(stderr, "[iris_amd] iris_gemm_launch_noalloc: num_sms %d exceeds the workspace's %d programs\n",
                 args->num_sms, IRIS_GEMM_NOALLOC_MAX_PROGRAMS);
    return hipErrorInvalidValue;
  }
  const int64_t tile_elems = (int64_t)args->block_m * args->block_n;
  const bool forced = args->split_k > 1 || args->split_k == IRIS_GEMM_SPLIT_STREAM_K;
  if (forced && tile_elems > IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS) {
    std::fprintf(stderr,
                 "[iris_amd] iris_gemm_launch_noalloc: a split of K was asked for, and a %d x %d tile exceeds the "
                 "workspace's %d elements per partial tile\n",
                 args->block_m, args->block_n, IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS);
    return hipErrorInvalidValue;
  }
  unsigned char* base = nullptr;
  hipError_t err = scratch_address(&base);
  if (err != hipSuccess) return err;

  iris_gemm_args a = *args;
  a.locks = reinterpret_cast<int32_t*>(base);
  // tiles beyond the slot size run unsplit, exactly as without a workspace
  a.partials = tile_elems <= IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS ? reinterpret_cast<float*>(base + NOALLOC_LOCK_BYTES) : nullptr;
  a.partials_slot_elems = a.partials ? IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS : 0;
  Plan plan;
  err = make_plan(a, &plan);
  if (err != hipSuccess) return err;
  // The array keeps what the last call left: the locks must start at zero (a
  // wait that timed out leaves one raised).  A fill kernel, not a memset, so
  // that the call can be recorded into a HIP graph.
  auto needs_locks = [](const Plan& q) {
    return (q.skinny && q.k.flag_mode != 0) || (q.entry && (q.k.split_k > 1 || q.k.stream_k || q.last_round));
  };
  const bool uses_locks = needs_locks(plan) || (plan.rest && needs_locks(*plan.rest));
  if (uses_locks) {
    hipLaunchKernelGGL(fill_i32_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream), a.locks, 0,
                       (int)(NOALLOC_LOCK_BYTES / sizeof(int32_t)));
    err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  return run_plan(plan, a, stream);
}

extern "C" int iris_gemm_split_k(const iris_gemm_args* args, int* split_k) {
  if (!args || !split_k) return hipErrorInvalidValue;
  Plan plan;
  hipError_t err = make_plan(*args, &plan);
  if (err != hipSuccess) return err;
  *split_k = plan.entry && !plan.skinny ? (plan.k.stream_k ? IRIS_GEMM_SPLIT_STREAM_K : plan.k.split_k) : 1;
  return hipSuccess;
}

extern "C" int iris_gemm_kernel_info(const iris_gemm_args* args, int* n_regs, int* n_spills) {
  if (!args) return hipErrorInvalidValue;
  Plan plan;
  hipError_t err = make_plan(*args, &plan);
  if (err != hipSuccess) return err;
  if (n_regs) *n_regs = 0;
  if (n_spills) *n_spills = 0;
  if (!plan.entry && !plan.skinny) return hipSuccess;
  hipFuncAttributes attr;
  err = hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(plan.skinny ? plan.skinny : plan_fn(plan)));
  if (err != hipSuccess) return err;
  if (n_regs) *n_regs = attr.numRegs;
  if (n_spills) *n_spills = static_cast<int>(attr.localSizeBytes);
  return hipSuccess;
}

extern "C" int iris_gemm_variant_name(int ab_dtype, int out_is_f32, int atomic, int variant, char* buf, size_t len) {
  const int op = atomic ? (out_is_f32 ? OP_ATOMIC32 : OP_ATOMIC16) : (out_is_f32 ? OP_STORE32 : OP_STORE16);
  int count = 0;
  const GemmKernelEntry* list = entries_for(ab_dtype, op, &count);
  if (!list || variant < 1 || variant > count || !buf || len == 0) return hipErrorInvalidValue;
  std::snprintf(buf, len, "%s", list[variant - 1].name);
  return hipSuccess;
}

extern "C" int iris_gemm_plan_name(const iris_gemm_args* args, char* buf, size_t len) {
  if (!args || !buf || len == 0) return hipErrorInvalidValue;
  Plan plan;
  hipError_t err = make_plan(*args, &plan);
  if (err != hipSuccess) return err;
  const char* few = plan.skinny_rb == 2 ? "few_rows_32xN" : "few_rows_16xN";
  std::snprintf(buf, len, "%s%s%s", plan.skinny ? few : plan.entry ? plan.entry->name : "",
                plan.entry && plan.k.stream_k                   ? "+stream_k"
                : plan.entry && plan.in_program                 ? "+reduce"
                : plan.entry && plan.k.num_sms > args->num_sms ? "+two_per_cu"
                                                                : "",
                !plan.entry                            ? ""
                : plan.k.merge_m * plan.k.merge_n == 2 ? "+two_tiles_each"
                : plan.k.merge_m * plan.k.merge_n == 4 ? "+four_tiles_each"
                : plan.k.merge_m * plan.k.merge_n == 8 ? "+eight_tiles_each"
                                                       : "");
  if (plan_touches(plan)) {
    const size_t n = std::strlen(buf);
    std::snprintf(buf + n, len > n ? len - n : 0, "+touch_ahead");
  }
  if (plan.last_round) {
    const size_t n = std::strlen(buf);
    std::snprintf(buf + n, len > n ? len - n : 0, "+last_round_in_%d_parts", plan.k_last.split_k);
  }
  if (plan.rest) {
    const size_t n = std::strlen(buf);
    std::snprintf(buf + n, len > n ? len - n : 0, "+last_%d_columns_apart", plan.rest->k.N);
  }
  return hipSuccess;
}

extern "C" int iris_stream_k_schedule_host(int32_t total_tiles, int32_t k_steps, int32_t num_programs, int32_t pid,
                                           int32_t* items, int32_t cap, int32_t* n_items) {
  if (total_tiles <= 0 || k_steps <= 0 || num_programs <= 0 || pid < 0 || pid >= num_programs || !n_items ||
      (int64_t)total_tiles * k_steps >= ((int64_t)1 << 30))
    return hipErrorInvalidValue;
  GemmKArgs k{};
  const int64_t steps = (int64_t)total_tiles * k_steps;
  k.split_q = (int)(steps / num_programs);
  k.split_r = (int)(steps % num_programs);
  if (k.split_q < 1) return hipErrorInvalidValue;  // the kernel is never launched with empty runs
  k.div_nk = make_fast_div((uint32_t)k_steps, (uint64_t)steps + 1);
  const StreamRun sr = stream_run(k, pid, k_steps);
  const int n = stream_items(sr, k_steps);
  *n_items = n;
  for (int i = 0; i < n && i < cap && items; ++i) {
    // the kernel's k_range for a split build, and the owner's count of parts
    const int k_begin = i == 0 ? sr.k0 : 0;
    const int k_end = sr.g1 - (sr.tile0 + i) * k_steps < k_steps ? sr.g1 - (sr.tile0 + i) * k_steps : k_steps;
    items[4 * i + 0] = sr.tile0 + i;
    items[4 * i + 1] = k_begin;
    items[4 * i + 2] = k_end;
    items[4 * i + 3] = k_begin == 0 ? stream_parts(k, pid, k_end, k_steps) : 0;
  }
  return hipSuccess;
}
