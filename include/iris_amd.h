/*
 * iris_amd.h -- C-ABI of the MI355X-native fused GEMM + tile-publishing path.
 *
 * Two shared libraries implement it:
 *
 *   libfinegrained_allocator.so   torch pluggable-allocator entry points
 *   libiris_amd.so                HIP runtime helpers + kernel launchers
 *
 * Everything is `extern "C"`, takes plain pointers and integers, allocates
 * nothing (except the two allocator calls whose job that is), never
 * synchronises the stream and never takes ownership of a buffer.  A HIP
 * stream is passed as `void*` (a `hipStream_t`); NULL is the default stream.
 * Unless stated otherwise a function returns a `hipError_t` as `int`
 * (0 == hipSuccess); `iris_hip_error_string` turns it into text.
 *
 * Reference citations are relative to the ROCm/iris tree.
 */
#ifndef IRIS_AMD_H_
#define IRIS_AMD_H_

#include <stddef.h>
#include <stdint.h>
#include <sys/types.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------ */
/* Pluggable allocator (libfinegrained_allocator.so)                         */
/* Replaces csrc/finegrained_alloc/finegrained_allocator.hip:28-55, bound by */
/* torch.cuda.memory.CUDAPluggableAllocator at iris/__init__.py:40-45.       */
/* On a HIP error both print "[finegrained_allocator] Hip error: ..." to     */
/* stderr and exit(EXIT_FAILURE), as the reference does (:11-16).            */
/* ------------------------------------------------------------------------ */
void* finegrained_hipMalloc(ssize_t size, int device, void* stream);
void finegrained_hipFree(void* ptr, ssize_t size, int device, void* stream);

/* ------------------------------------------------------------------------ */
/* HIP runtime helpers (libiris_amd.so); replace iris/_hip.py                */
/* ------------------------------------------------------------------------ */
/* hipGetErrorString; iris/_hip.py:12-16 */
const char* iris_hip_error_string(int err);
/* iris/_hip.py:62-65 */
int iris_hip_device_count(int* count);
/* iris/_hip.py:68-69 */
int iris_hip_set_device(int device);
/* iris/_hip.py:72-75 */
int iris_hip_get_device(int* device);
/* hipDeviceAttributeMultiprocessorCount; iris/_hip.py:78-87 */
int iris_hip_cu_count(int device, int* cu_count);
/* hipDeviceAttributeWallClockRate, kHz; iris/_hip.py:107-114 */
int iris_hip_wall_clock_rate(int device, int* khz);
/* hipExtMallocWithFlags(hipDeviceMallocFinegrained); iris/_hip.py:117-121 */
int iris_hip_malloc_finegrained(void** ptr, size_t size);
/* hipMalloc / hipFree; iris/_hip.py:124-131 */
int iris_hip_malloc(void** ptr, size_t size);
int iris_hip_free(void* ptr);
/* hipIpcGetMemHandle, 64-byte handle; iris/_hip.py:56-59 */
int iris_hip_ipc_get_handle(void* handle64, void* ptr);
/* hipIpcOpenMemHandle(..., hipIpcMemLazyEnablePeerAccess); iris/_hip.py:23-53 */
int iris_hip_ipc_open_handle(void** ptr, const void* handle64);
/* hipDeviceSynchronize: the device half of Iris.barrier, iris/iris.py:272-276 */
int iris_hip_device_synchronize(void);
/* name of the gfx target the current device reports ("gfx950"); buf gets a
 * NUL-terminated string of at most len-1 characters */
int iris_hip_arch_name(int device, char* buf, size_t len);

/* ------------------------------------------------------------------------ */
/* Kernel launchers (libiris_amd.so)                                         */
/* ------------------------------------------------------------------------ */

/* element types */
#define IRIS_DTYPE_F32 0
#define IRIS_DTYPE_F16 1
#define IRIS_DTYPE_BF16 2
/* integer element types: only iris_p2p_bench_launch (and the unit-test kernels of iris_amd_testing.h) take them */
#define IRIS_DTYPE_I8 3
#define IRIS_DTYPE_I16 4
#define IRIS_DTYPE_I32 5
#define IRIS_DTYPE_I64 6

/* epilogues of the persistent shard GEMM */
#define IRIS_EPI_ALL_SCATTER 0 /* examples/07_gemm_all_scatter/gemm_all_scatter.py:209-251 */
#define IRIS_EPI_ATOMIC_ADD 1  /* examples/08_gemm_atomics_all_reduce/gemm_atomics_all_reduce.py:206-248 */
#define IRIS_EPI_ONE_SHOT 2    /* examples/09_gemm_one_shot_all_reduce/gemm_one_shot_all_reduce.py:197-271 */

/* phases of IRIS_EPI_ONE_SHOT (bit mask) */
#define IRIS_PHASE_PRODUCE 1 /* store partial tile + signal the other ranks  (:197-218) */
#define IRIS_PHASE_CONSUME 2 /* wait for the tile's flag, reduce, store       (:220-271) */
#define IRIS_PHASE_FUSED 3   /* both, in one program and tile by tile, as the reference kernel: every rank's
                              * launch must be on its device at the same time (a program waits for its peers) */
#define IRIS_PHASE_TWO_KERNELS 7 /* both, as two kernels on the stream: the producer GEMM, then the reduce kernel
                                  * (iris_one_shot_reduce_launch) behind it */

/* flag scopes */
#define IRIS_SCOPE_AGENT 0  /* all "ranks" live on this GPU */
#define IRIS_SCOPE_SYSTEM 1 /* the reference's scope="sys" */
#define IRIS_SCOPE_WORKGROUP 2 /* scope="cta"; only the unit-test kernels of iris_amd_testing.h take it */

/* How a tile's flag orders the tile's data (iris_gemm_args.flag_sem, iris_reduce_args.flag_sem).
 * WRITE_THROUGH (the default): the tile is stored with write-through stores at the flags' scope, the producer
 * waits for their acknowledgement and raises the flag with a relaxed atomic; the consumer polls relaxed and reads
 * with loads that are coherent at that scope.  No cache write-back and no invalidate per tile.  This scheme has
 * been validated with producers and consumers running side by side on ONE device (at both scopes); it has not
 * been run across devices.
 * RELEASE_ACQUIRE: the reference's semantics verbatim -- atomic_add(flag, 1, sem="release") on the producer
 * side, sem="acquire" on the consumer's wait (gemm_one_shot_all_reduce.py:207-234).  What a launch across
 * devices should use until the default has been validated there; costs an L2 write-back per published tile. */
#define IRIS_FLAG_SEM_WRITE_THROUGH 0
#define IRIS_FLAG_SEM_RELEASE_ACQUIRE 1

/* status word values (max-reduced by the kernels into *status) */
#define IRIS_STATUS_OK 0
#define IRIS_STATUS_SPIN_TIMEOUT 1 /* a flag wait gave up; that tile was not reduced */

/* Special values of iris_gemm_args.variant.  A launch with at most 32 rows of
 * A (64 when K >= 2048) whose operands are K-contiguous normally takes a kernel
 * of its own that streams B (one workgroup per 16 or 32 rows x 16 columns of C,
 * all fetches in flight);
 * FEW_ROWS insists on it (hipErrorInvalidValue when the launch does not
 * qualify), PERSISTENT keeps the default choice among the persistent kernels.
 * The reference has one Triton kernel for every M (gemm_all_scatter.py:95). */
#define IRIS_GEMM_VARIANT_FEW_ROWS 1000
#define IRIS_GEMM_VARIANT_PERSISTENT 1001

/* iris_gemm_args.touch_ahead.  The eight-wave 256 x 256 tile has a build whose programs touch, one dword per 128-byte
 * line, their share of the operand lines that the K-steps three ahead will load, so that the lines are in the
 * XCD's L2 when the stage loads ask for them.  It pays where a round of tiles streams its operands from HBM (more
 * bytes than the 256 MB last-level cache holds) and costs a few per cent where they are cache-resident: AUTO lets
 * the launcher decide by the launch's bytes per round of tiles, ON takes the build wherever the picked tile has it
 * (unsplit launches of that tile with a store epilogue on more than one XCD), OFF never.  The results are the same
 * bits either way.  The reference has no counterpart (its loads are the Triton compiler's, gemm_*:170-199). */
#define IRIS_GEMM_TOUCH_AUTO 0
#define IRIS_GEMM_TOUCH_ON 1
#define IRIS_GEMM_TOUCH_OFF 2

/* Special value of iris_gemm_args.split_k: cut the launch's K-steps (all
 * tiles, in tile order) into num_sms equal runs that start and end anywhere
 * in a tile, the stream-K schedule the reference's wrappers describe and size
 * their `P` / `locks` buffers for (matmul_wrapper.py:73-92,
 * images/stream_k.excalidraw.svg) but do not implement.  Needs partials and
 * locks; hipErrorInvalidValue when the launch cannot be cut this way.  Only
 * taken on request (split_k = 0 chooses between an unsplit and a split-K
 * launch); iris_gemm_split_k reports this value for such a launch. */
#define IRIS_GEMM_SPLIT_STREAM_K (-1)
/* iris_gemm_args.split_handover */
#define IRIS_GEMM_HANDOVER_AUTO 0
#define IRIS_GEMM_HANDOVER_OWNER 1
#define IRIS_GEMM_HANDOVER_SLICED 2
#define IRIS_GEMM_HANDOVER_PAIR 3

/*
 * Arguments of one persistent shard-GEMM launch.  It is the argument list of
 * the reference kernels (gemm_*:95-132) plus what their Triton launch passes
 * implicitly (element types, stream).  Strides are in elements.
 */
typedef struct iris_gemm_args {
  const void* a;        /* A  [M, K]                                   gemm_*:96  */
  const void* b;        /* B  [K, N]                                   gemm_*:97  */
  void* c;              /* this rank's partial C [M, N] (ONE_SHOT)      gemm_*:98  */
  void* c_global;       /* published result                            gemm_*:99  */
  int32_t* tile_completed; /* one flag per tile, on the heap            gemm_*:103 */
  const uint64_t* heap_bases; /* device uint64[world_size]              gemm_*:125 */
  int64_t* mm_begin_timestamp; /* optional int64[total_tiles]           gemm_*:130 */
  int64_t* mm_end_timestamp;   /* optional int64[total_tiles]           gemm_*:131 */
  uint32_t* status;     /* optional device word, see IRIS_STATUS_*                */
  int32_t M, N, K;      /*                                              gemm_*:104-106 */
  int64_t stride_am, stride_ak; /*                                      gemm_*:107-108 */
  int64_t stride_bk, stride_bn; /*                                      gemm_*:109-110 */
  int64_t stride_cm, stride_cn; /*                                      gemm_*:111-112 */
  int64_t stride_cm_global, stride_cn_global; /*                        gemm_*:113-114 */
  int32_t block_m, block_n, block_k; /* BLOCK_SIZE_*                    gemm_*:116-118 */
  int32_t group_size_m; /* GROUP_SIZE_M                                 gemm_*:119 */
  int32_t num_sms;      /* NUM_SMS == grid size                         gemm_*:120 */
  int32_t num_xcds;     /* NUM_XCDS                                     gemm_*:122 */
  int32_t cur_rank, world_size; /*                                      gemm_*:126-127 */
  int32_t ab_dtype;     /* IRIS_DTYPE_F16 | IRIS_DTYPE_BF16; IRIS_DTYPE_F32 with fp32 outputs */
  int32_t c_dtype;      /* element type of c                                      */
  int32_t c_global_dtype; /* element type of c_global                             */
  int32_t epilogue;     /* IRIS_EPI_*                                             */
  int32_t phase;        /* IRIS_PHASE_* (ONE_SHOT only)                           */
  int32_t notify;       /* ALL_SCATTER: publish a ready flag per tile   gemm_*:128 (NOTIFY_REMOTES) */
  int32_t scope;        /* IRIS_SCOPE_*                                           */
  int32_t variant;      /* 0 = default kernel choice; >0 selects a tuning variant, or IRIS_GEMM_VARIANT_* */
  uint64_t spin_timeout_ticks; /* bound on a flag wait in 100 MHz ticks; 0 = default (2 s) */
  /* Split-K workspace: the `P` and `locks` buffers that matmul.apply receives
   * (matmul_wrapper.py:29-31,73-92; allocated at benchmark.py:136-142).  With both
   * given, a launch whose tiles would leave most programs idle shares each
   * tile's K range over several programs: partial tiles go through `partials`
   * in fp32, `locks` (all zero before the first launch, left all zero) orders
   * the hand-over.  Results differ from the unsplit ones only in fp32
   * summation order. */
  float* partials;      /* [num_sms][partials_slot_elems] fp32, or NULL           */
  int32_t* locks;       /* int32[num_sms], or NULL (a tile in n parts uses the n words of its programs) */
  int64_t partials_slot_elems; /* >= block_m * block_n                            */
  int32_t split_k;      /* 0 = let the launcher decide, 1 = never, n > 1 = force n, IRIS_GEMM_SPLIT_STREAM_K */
  /* How the parts of a split tile meet (split-K proper; stream-K runs always
   * hand over to the tile's first part): IRIS_GEMM_HANDOVER_AUTO lets the
   * launcher decide, _OWNER: the first part adds the others' partials and runs
   * the epilogue, _SLICED: every part leaves its partial, then sums and stores
   * its share of the tile's rows, _PAIR (two parts of a 256 x 128, 128 x 256 or
   * 256 x 256 compute tile only): each part keeps the accumulators of half the
   * waves and leaves the other half's for the other part, so that slots of
   * half a tile are enough.  All add the partials in part order: the results
   * are bit-identical. */
  int32_t split_handover;
  int32_t flag_sem;     /* IRIS_FLAG_SEM_*: how a tile's flag orders its data                    */
  int32_t touch_ahead;  /* IRIS_GEMM_TOUCH_*                                                     */
} iris_gemm_args;

/*
 * Launch the persistent shard GEMM with the epilogue `args->epilogue`.
 * Replaces `gemm_kernel[(grids,)](...)` at matmul_wrapper.py:109-150 (the same file in
 * examples/07_gemm_all_scatter, 08_gemm_atomics_all_reduce and 09_gemm_one_shot_all_reduce).
 * Returns hipErrorInvalidValue for shapes/strides/types it does not take.
 */
int iris_gemm_launch(const iris_gemm_args* args, void* stream);

/*
 * iris_gemm_launch for callers that cannot allocate device memory and have no
 * workspace to pass: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference
 * (whose wrappers allocate `P` and `locks` with torch, benchmark.py:136-142).
 * `args->partials`, `args->locks` and `args->partials_slot_elems` are ignored:
 * the split-K / stream-K partial tiles and the locks (also the few-rows
 * kernel's arrival counters) live in a device array inside the library,
 * IRIS_GEMM_NOALLOC_MAX_PROGRAMS slots of IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS
 * floats plus 4 KiB of locks (16 MiB + 4 KiB per device, held until the process
 * ends).  The call allocates and frees nothing; it clears the locks with a
 * fill kernel on `stream` before the GEMM when the launch uses them.
 * Limits: num_sms > IRIS_GEMM_NOALLOC_MAX_PROGRAMS is rejected; a forced split
 * (split_k > 1 or IRIS_GEMM_SPLIT_STREAM_K) with block_m * block_n >
 * IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS is rejected; both print the reason to
 * stderr and return hipErrorInvalidValue.  With split_k == 0 a larger tile
 * runs unsplit, as iris_gemm_launch does without a workspace.
 * Every call on a device shares that device's array: calls that overlap on
 * one device (two streams, two threads) race on it.  The first call on a
 * device looks the array's address up (hipGetSymbolAddress) and should be made
 * outside a graph capture.
 */
#define IRIS_GEMM_NOALLOC_MAX_PROGRAMS 256
#define IRIS_GEMM_NOALLOC_MAX_TILE_ELEMS 16384 /* 128 x 128, the largest tile with a split-K build */
int iris_gemm_launch_noalloc(const iris_gemm_args* args, void* stream);

/* Registers and spills of the kernel `iris_gemm_launch` would pick for `args`
 * (what the reference reads from kk.n_regs / kk.n_spills,
 * matmul_wrapper.py:152-155).  *spills is the scratch bytes per lane. */
int iris_gemm_kernel_info(const iris_gemm_args* args, int* n_regs, int* n_spills);
/* The split-K factor `iris_gemm_launch` would use for `args` (1 = unsplit). */
int iris_gemm_split_k(const iris_gemm_args* args, int* split_k);

/* Name of the kernel `iris_gemm_launch` would run for `args` ("" when there is
 * no GEMM work): a tuning variant's name, or "few_rows_16xN" / "few_rows_32xN",
 * followed by "+stream_k", "+reduce" (the in-program reduce) or "+two_per_cu"
 * (two programs a CU), and by "+two_tiles_each" / "+four_tiles_each" /
 * "+eight_tiles_each" where the launch computes a block of that many of the
 * caller's tiles as one (each tile keeps its own id and flag), and by
 * "+last_round_in_N_parts" where a second launch shares K of the last round's
 * tiles out over the programs that round would leave idle (needs partials and
 * locks). */
int iris_gemm_plan_name(const iris_gemm_args* args, char* buf, size_t len);

/* Name of tuning variant `variant` (1-based) of the kernel list used for
 * (ab_dtype, fp32 output?, atomic?); hipErrorInvalidValue past the end. */
int iris_gemm_variant_name(int ab_dtype, int out_is_f32, int atomic, int variant, char* buf, size_t len);

/*
 * One-shot reduce of `world_size` partial-C buffers that live at the same
 * heap offset on every rank: wait for tile_completed[tile] == world_size-1
 * (CAS back to 0, acquire), sum the tile over ranks 0..world_size-1 in fp32,
 * store to c_global.  The consumer half of
 * examples/09_gemm_one_shot_all_reduce/gemm_one_shot_all_reduce.py:220-271
 * as a kernel of its own.  `c` is this rank's partial buffer.
 */
typedef struct iris_reduce_args {
  const void* c;
  void* c_global;
  int32_t* tile_completed;
  const uint64_t* heap_bases;
  uint32_t* status;
  int32_t M, N;
  int64_t stride_cm, stride_cn;
  int64_t stride_cm_global, stride_cn_global;
  int32_t block_m, block_n, group_size_m;
  int32_t num_sms;   /* grid size; 0 = one program per tile */
  int32_t num_xcds;
  int32_t cur_rank, world_size;
  int32_t c_dtype, c_global_dtype;
  int32_t scope;
  int32_t wait_flags; /* 0: skip the flag wait (plain P-way sum) */
  int32_t variant;
  uint64_t spin_timeout_ticks;
  int32_t flag_sem;   /* IRIS_FLAG_SEM_*: RELEASE_ACQUIRE adds an acquire fence after every flag wait */
} iris_reduce_args;

int iris_one_shot_reduce_launch(const iris_reduce_args* args, void* stream);

/*
 * The producer's signal on its own: +1 (release) on tile_completed[tile] of
 * every rank other than cur_rank (include_self != 0: of every rank), for
 * tile in [0, total_tiles).  gemm_one_shot_all_reduce.py:207-218.
 */
int iris_signal_tiles_launch(int32_t* tile_completed, const uint64_t* heap_bases, int32_t total_tiles,
                             int32_t cur_rank, int32_t world_size, int32_t include_self, int32_t scope,
                             void* stream);

/* int32 fill; iris/util.py:107-128 (memset_kernel / memset_tensor). */
int iris_memset_i32_launch(int32_t* ptr, int32_t value, int64_t n_elements, void* stream);

/*
 * The tile schedule exactly as the kernels compute it, for checking it bit
 * for bit: out is int32[total_tiles][4] = (pid_m, pid_n, program, position
 * in the program's tile list) per tile id.  tile_id -> (pid_m, pid_n) is
 * gemm_*:155-160; the program's tile list is gemm_*:133-136,150.
 */
int iris_tile_schedule_launch(int32_t* out, int32_t M, int32_t N, int32_t block_m, int32_t block_n,
                              int32_t group_size_m, int32_t num_sms, int32_t num_xcds, void* stream);
/* The same tile_id -> (pid_m, pid_n) function, compiled for the host. */
void iris_tile_map_host(int32_t tile_id, int32_t M, int32_t N, int32_t block_m, int32_t block_n,
                        int32_t group_size_m, int32_t* pid_m, int32_t* pid_n);

/*
 * The stream-K schedule exactly as the kernels compute it (the same source,
 * compiled for the host), for checking it without a GPU: the items of program
 * `pid` when `total_tiles` tiles of `k_steps` K-steps each are cut into
 * `num_programs` runs.  items is int32[cap][4] = (tile, first K-step, end
 * K-step, parts), parts being the number of programs that share the tile when
 * this program owns it (its run holds the tile's first step) and 0 when it
 * hands its part over; *n_items is the number of items of the run.
 */
int iris_stream_k_schedule_host(int32_t total_tiles, int32_t k_steps, int32_t num_programs, int32_t pid,
                                int32_t* items, int32_t cap, int32_t* n_items);

/*
 * The kernels of the reference's point-to-point microbenchmarks as HIP kernels
 * over include/iris_device.hpp.  Thread i of a grid of ceil(n / block_size)
 * blocks owns element i of `buffer` and `result`, both at the same heap offset
 * on every rank; the launch acts as rank `cur_rank`.
 *   LOAD        result[i] = load(buffer + i) from `peer_rank`          examples/00_load/load_bench.py:20-47
 *   LOCAL_STORE result[i] = 0, the benchmarks' local baseline          examples/00_load/load_bench.py:50-61
 *   STORE       store(buffer + i, i) on `peer_rank`                    examples/01_store/store_bench.py:18-45
 *   ALL_LOAD    result[i] = sum over all ranks of load(buffer + i)     examples/02_all_load/all_load_bench.py:43-87
 *   ALL_STORE   store(buffer + i, i) on every other rank               examples/03_all_store/all_store_bench.py:20-47
 *   ATOMIC_ADD  atomic_add(buffer + i, 1) on `peer_rank`, relaxed, sys examples/04_atomic_add/atomic_add_bench.py:18-40
 *   ATOMIC_XCHG result[i] = atomic_xchg(buffer + i, 1) on `peer_rank`  examples/05_atomic_xchg/atomic_xchg_bench.py:18-43
 * dtype: F32, F16, BF16, I8 (no atomics), I32.  block_size is 1..1024.
 */
#define IRIS_P2P_LOAD 0
#define IRIS_P2P_LOCAL_STORE 1
#define IRIS_P2P_STORE 2
#define IRIS_P2P_ALL_LOAD 3
#define IRIS_P2P_ALL_STORE 4
#define IRIS_P2P_ATOMIC_ADD 5
#define IRIS_P2P_ATOMIC_XCHG 6
int iris_p2p_bench_launch(int32_t op, int32_t dtype, void* buffer, void* result, int64_t n_elements,
                          int32_t cur_rank, int32_t peer_rank, int32_t num_ranks, const uint64_t* heap_bases,
                          int32_t block_size, void* stream);

/* Library version, bumped when a signature in this header changes. */
int iris_amd_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* IRIS_AMD_H_ */
