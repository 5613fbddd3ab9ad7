// Kernels that exercise the device-side remote-access functions of
// include/iris_device.hpp the way the reference's unit tests exercise the
// Triton ones (tests/unittests/test_{load,store,get,put,atomic_add,atomic_cas,
// atomic_xchg}.py): one workgroup, lane i owns element i, every rank is a
// target in turn.  C-ABI: iris_rma_selftest_launch.
#include <hip/hip_runtime.h>

#include "../../../include/iris_amd_testing.h"
#include "../../../include/iris_device.hpp"

namespace {

using iris::Scope;
using iris::Sem;

template <typename T>
__device__ inline T add(T a, T b) {
  if constexpr (sizeof(T) == 2 && !std::is_integral<T>::value)
    return static_cast<T>(static_cast<float>(a) + static_cast<float>(b));
  else
    return static_cast<T>(a + b);
}
template <typename T>
__device__ inline T from_int(int v) {
  if constexpr (sizeof(T) == 2 && !std::is_integral<T>::value)
    return static_cast<T>(static_cast<float>(v));
  else
    return static_cast<T>(v);
}

// tests/unittests/test_load.py:8-31
template <typename T>
__global__ void load_kernel(const T* data, T* results, const uint64_t* hb, int rank, int num_ranks, int block) {
  const int i = threadIdx.x;
  const bool mask = i < block;
  T acc = from_int<T>(0);
  for (int t = 0; t < num_ranks; ++t) acc = add(acc, iris::load(data + i, rank, t, hb, mask));
  if (mask) results[i] = acc;
}
// tests/unittests/test_store.py:8-30
template <typename T>
__global__ void store_kernel(const T* data, T* results, const uint64_t* hb, int rank, int num_ranks, int block) {
  const int i = threadIdx.x;
  const bool mask = i < block;
  const T value = mask ? data[i] : from_int<T>(0);
  for (int t = 0; t < num_ranks; ++t) iris::store(results + i, value, rank, t, hb, mask);
}
// tests/unittests/test_get.py:8-31
template <typename T>
__global__ void get_kernel(const T* data, T* results, const uint64_t* hb, int rank, int num_ranks, int block) {
  const int i = threadIdx.x;
  const bool mask = i < block;
  T acc = from_int<T>(0);
  for (int t = 0; t < num_ranks; ++t) {
    iris::get(data + i, results + i, rank, t, hb, mask);
    if (mask) acc = add(acc, results[i]);
  }
  if (mask) results[i] = acc;
}
// tests/unittests/test_put.py:8-26
template <typename T>
__global__ void put_kernel(const T* data, T* results, const uint64_t* hb, int rank, int num_ranks, int block) {
  const int i = threadIdx.x;
  const bool mask = i < block;
  for (int t = 0; t < num_ranks; ++t) iris::put(data + i, results + i, rank, t, hb, mask);
}
// tests/unittests/test_atomic_add.py:8-30 (and its mirror image for atomic_sub)
template <typename T, Sem S, Scope C, bool SUB>
__global__ void atomic_add_kernel(const T*, T* results, const uint64_t* hb, int rank, int num_ranks, int block) {
  const int i = threadIdx.x;
  const bool mask = i < block;
  for (int t = 0; t < num_ranks; ++t) {
    if constexpr (SUB)
      iris::atomic_sub<S, C>(results + i, from_int<T>(1), rank, t, hb, mask);
    else
      iris::atomic_add<S, C>(results + i, from_int<T>(1), rank, t, hb, mask);
  }
}
// tests/unittests/test_atomic_cas.py:8-24
template <typename T, Sem S, Scope C>
__global__ void atomic_cas_kernel(const T*, T* results, const uint64_t* hb, int rank, int num_ranks, int) {
  if (threadIdx.x != 0) return;
  for (int t = 0; t < num_ranks; ++t)
    iris::atomic_cas<S, C>(results, from_int<T>(0), from_int<T>(num_ranks), rank, t, hb);
}
// tests/unittests/test_atomic_xchg.py:8-23
template <typename T, Sem S, Scope C>
__global__ void atomic_xchg_kernel(const T*, T* results, const uint64_t* hb, int rank, int num_ranks, int) {
  if (threadIdx.x != 0) return;
  for (int t = 0; t < num_ranks; ++t) iris::atomic_xchg<S, C>(results, from_int<T>(num_ranks), rank, t, hb);
}

template <typename T>
using Kernel = void (*)(const T*, T*, const uint64_t*, int, int, int);

template <typename T, Sem S, Scope C>
Kernel<T> pick_atomic(int op) {
  if constexpr (sizeof(T) == 1) {
    return nullptr;
  } else {
    switch (op) {
      case IRIS_RMA_ATOMIC_ADD: return &atomic_add_kernel<T, S, C, false>;
      case IRIS_RMA_ATOMIC_SUB: return &atomic_add_kernel<T, S, C, true>;
      case IRIS_RMA_ATOMIC_CAS: return &atomic_cas_kernel<T, S, C>;
      case IRIS_RMA_ATOMIC_XCHG: return &atomic_xchg_kernel<T, S, C>;
      default: return nullptr;
    }
  }
}
template <typename T, Sem S>
Kernel<T> pick_scope(int op, int scope) {
  switch (scope) {
    case IRIS_SCOPE_WORKGROUP: return pick_atomic<T, S, Scope::cta>(op);
    case IRIS_SCOPE_AGENT: return pick_atomic<T, S, Scope::gpu>(op);
    case IRIS_SCOPE_SYSTEM: return pick_atomic<T, S, Scope::sys>(op);
    default: return nullptr;
  }
}
template <typename T>
Kernel<T> pick(int op, int sem, int scope) {
  switch (op) {
    case IRIS_RMA_LOAD: return &load_kernel<T>;
    case IRIS_RMA_STORE: return &store_kernel<T>;
    case IRIS_RMA_GET: return &get_kernel<T>;
    case IRIS_RMA_PUT: return &put_kernel<T>;
    default: break;
  }
  switch (sem) {
    case IRIS_SEM_RELAXED: return pick_scope<T, Sem::relaxed>(op, scope);
    case IRIS_SEM_ACQUIRE: return pick_scope<T, Sem::acquire>(op, scope);
    case IRIS_SEM_RELEASE: return pick_scope<T, Sem::release>(op, scope);
    case IRIS_SEM_ACQ_REL: return pick_scope<T, Sem::acq_rel>(op, scope);
    default: return nullptr;
  }
}

template <typename T>
int launch(int op, int sem, int scope, const void* data, void* results, const uint64_t* hb, int rank, int num_ranks,
           int block, hipStream_t stream) {
  Kernel<T> k = pick<T>(op, sem, scope);
  if (!k) return hipErrorInvalidValue;
  hipLaunchKernelGGL(k, dim3(1), dim3(64), 0, stream, static_cast<const T*>(data), static_cast<T*>(results), hb, rank,
                     num_ranks, block);
  return hipGetLastError();
}

}  // namespace

extern "C" int iris_rma_selftest_launch(int32_t op, int32_t dtype, int32_t sem, int32_t scope, const void* data,
                                        void* results, const uint64_t* heap_bases, int32_t cur_rank,
                                        int32_t num_ranks, int32_t block_size, void* stream) {
  if (!results || !heap_bases || num_ranks <= 0 || cur_rank < 0 || cur_rank >= num_ranks || block_size < 1 ||
      block_size > 64)
    return hipErrorInvalidValue;
  if (op <= IRIS_RMA_PUT && !data) return hipErrorInvalidValue;
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case IRIS_DTYPE_F32: return launch<float>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    case IRIS_DTYPE_F16: return launch<_Float16>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    case IRIS_DTYPE_BF16: return launch<__bf16>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    case IRIS_DTYPE_I8: return launch<int8_t>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    case IRIS_DTYPE_I16: return launch<int16_t>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    case IRIS_DTYPE_I32: return launch<int32_t>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    case IRIS_DTYPE_I64: return launch<int64_t>(op, sem, scope, data, results, heap_bases, cur_rank, num_ranks, block_size, st);
    default: return hipErrorInvalidValue;
  }
}
