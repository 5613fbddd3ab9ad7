/*
 * iris_amd_testing.h -- C-ABI of libiris_amd_testing.so: kernels that only the
 * tests and bench.py call.  Not part of the product library (libiris_amd.so,
 * include/iris_amd.h): measurement probes for the matrix cores and the store
 * path, and the unit-test kernels over the device-side remote-access header.
 * Same conventions as iris_amd.h: extern "C", plain pointers and integers, a
 * hipError_t as int, a stream as void*, nothing allocated, nothing synchronised.
 */
#ifndef IRIS_AMD_TESTING_H_
#define IRIS_AMD_TESTING_H_

#include "iris_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Measurement aid; no counterpart in the reference.  `num_groups` workgroups of
 * 8 waves each run `iters` rounds of 16 v_mfma_f32_16x16x32 (ab_dtype: F16 or
 * BF16) per wave on operands read once from `operands` (64 KiB, 16-byte
 * aligned, any bit patterns), with nothing but registers inside the loop:
 * num_groups * 8 * iters * 16 * 16384 FLOP per launch.  `sink` receives one
 * float per thread (num_groups * 512).  Timed by the caller, it gives the rate
 * the matrix cores sustain on such data under the board's power limit.
 */
int iris_mfma_probe_launch(const void* operands, float* sink, int32_t ab_dtype, int32_t iters, int32_t num_groups,
                           void* stream);

/*
 * Measurement aid; no counterpart in the reference.  What a tile's worth of
 * output stores costs next to the matrix cores, by how the stores are spread:
 * each of `num_groups` workgroups of 8 waves runs `tiles` tiles, a tile being
 * 16 K-steps of 64 register-only bf16 MFMAs a wave (a 256 x 256 x 1024 tile's
 * worth) and 16 one-KiB stores a wave (128 KiB a group) to a region of its own
 * in `out` (`out_bytes` >= num_groups * 128 KiB, 16-byte aligned; tile t goes
 * to offset t * num_groups * 128 KiB modulo what fits).  `chunk` stores go out
 * back to back every `chunk` K-steps: 16 = a whole tile at once, 4, 1 = one a
 * K-step, 0 = none.  `write_through`: sc1 stores (else plain); `lockstep`: the
 * waves of a group meet at a barrier after every K-step.  `operands` and
 * `sink` as for iris_mfma_probe_launch.
 */
int iris_store_probe_launch(const void* operands, float* sink, void* out, uint64_t out_bytes, int32_t tiles,
                            int32_t chunk, int32_t write_through, int32_t lockstep, int32_t num_groups, void* stream);

/*
 * Device-side remote access (include/iris_device.hpp, the HIP counterpart of
 * iris/iris.py:317-521) exercised the way the reference's unit tests exercise
 * the Triton functions: one workgroup, lane i < block_size owns element i of
 * `data` / `results` (buffers at the same heap offset on every rank), and every
 * rank 0..num_ranks-1 is the target in turn.
 *   LOAD        results[i]  = sum over ranks of load(data + i)      tests/unittests/test_load.py:8-31
 *   STORE       store(results + i, data[i]) on every rank           tests/unittests/test_store.py:8-30
 *   GET         get(data + i -> results + i), accumulate, store     tests/unittests/test_get.py:8-31
 *   PUT         put(data + i -> results + i) on every rank          tests/unittests/test_put.py:8-26
 *   ATOMIC_ADD  atomic_add(results + i, 1) on every rank            tests/unittests/test_atomic_add.py:8-30
 *   ATOMIC_SUB  atomic_sub(results + i, 1) on every rank            (iris/iris.py:452-473; no reference test)
 *   ATOMIC_CAS  atomic_cas(results, 0 -> num_ranks) on every rank   tests/unittests/test_atomic_cas.py:8-24
 *   ATOMIC_XCHG atomic_xchg(results, num_ranks) on every rank       tests/unittests/test_atomic_xchg.py:8-23
 * sem / scope only matter for the atomics.  block_size is 1..64; int8 has no atomics.
 */
#define IRIS_RMA_LOAD 0
#define IRIS_RMA_STORE 1
#define IRIS_RMA_GET 2
#define IRIS_RMA_PUT 3
#define IRIS_RMA_ATOMIC_ADD 4
#define IRIS_RMA_ATOMIC_SUB 5
#define IRIS_RMA_ATOMIC_CAS 6
#define IRIS_RMA_ATOMIC_XCHG 7
#define IRIS_SEM_RELAXED 0
#define IRIS_SEM_ACQUIRE 1
#define IRIS_SEM_RELEASE 2
#define IRIS_SEM_ACQ_REL 3
int iris_rma_selftest_launch(int32_t op, int32_t dtype, int32_t sem, int32_t scope, const void* data, void* results,
                             const uint64_t* heap_bases, int32_t cur_rank, int32_t num_ranks, int32_t block_size,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* IRIS_AMD_TESTING_H_ */
