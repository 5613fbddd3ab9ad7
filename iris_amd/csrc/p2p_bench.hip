// Element-per-thread kernels of the point-to-point microbenchmarks
// (examples/00_load .. 05_atomic_xchg of the reference), written over the
// device-side remote-access functions of include/iris_device.hpp.  Thread i
// of the grid owns element i of the buffers.  C-ABI: iris_p2p_bench_launch.
#include <hip/hip_runtime.h>

#include "../../include/iris_amd.h"
#include "../../include/iris_device.hpp"

namespace {

using iris::Scope;
using iris::Sem;

template <typename T>
__device__ inline T from_index(int64_t v) {
  if constexpr (sizeof(T) == 2 && !std::is_integral<T>::value)
    return static_cast<T>(static_cast<float>(v));
  else
    return static_cast<T>(v);
}
template <typename T>
__device__ inline T add(T a, T b) {
  if constexpr (sizeof(T) == 2 && !std::is_integral<T>::value)
    return static_cast<T>(static_cast<float>(a) + static_cast<float>(b));
  else
    return static_cast<T>(a + b);
}

// examples/00_load/load_bench.py:20-47: read the peer's buffer, keep it here
template <typename T>
__global__ void load_kernel(const T* buffer, T* result, int64_t n, int rank, int peer, const uint64_t* hb) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool mask = i < n;
  const T v = iris::load(buffer + i, rank, peer, hb, mask);
  if (mask) result[i] = v;
}
// the benchmarks' local baseline (load_bench.py:50-61): a plain store of zeros
template <typename T>
__global__ void local_store_kernel(T* result, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) result[i] = from_index<T>(0);
}
// examples/01_store/store_bench.py:18-45: write the element's index into the peer's buffer
template <typename T>
__global__ void store_kernel(T* buffer, int64_t n, int rank, int peer, const uint64_t* hb) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  iris::store(buffer + i, from_index<T>(i), rank, peer, hb, i < n);
}
// examples/02_all_load/all_load_bench.py:43-87: sum of every rank's buffer
template <typename T>
__global__ void all_load_kernel(const T* buffer, T* result, int64_t n, int rank, int num_ranks, const uint64_t* hb) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool mask = i < n;
  T acc = iris::load(buffer + i, rank, 0, hb, mask);
  for (int r = 1; r < num_ranks; ++r) acc = add(acc, iris::load(buffer + i, rank, r, hb, mask));
  if (mask) result[i] = acc;
}
// examples/03_all_store/all_store_bench.py:20-47: the index into every other rank's buffer
template <typename T>
__global__ void all_store_kernel(T* buffer, int64_t n, int rank, int num_ranks, const uint64_t* hb) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int r = 0; r < num_ranks; ++r)
    if (r != rank) iris::store(buffer + i, from_index<T>(i), rank, r, hb, i < n);
}
// examples/04_atomic_add/atomic_add_bench.py:18-40: +1 on the peer, relaxed, system scope
template <typename T>
__global__ void atomic_add_kernel(T* buffer, int64_t n, int rank, int peer, const uint64_t* hb) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  iris::atomic_add<Sem::relaxed, Scope::sys>(buffer + i, from_index<T>(1), rank, peer, hb, i < n);
}
// examples/05_atomic_xchg/atomic_xchg_bench.py:18-43: exchange with 1 on the peer, keep the old value
template <typename T>
__global__ void atomic_xchg_kernel(T* buffer, T* result, int64_t n, int rank, int peer, const uint64_t* hb) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool mask = i < n;
  const T old = iris::atomic_xchg<Sem::relaxed, Scope::sys>(buffer + i, from_index<T>(1), rank, peer, hb, mask);
  if (mask) result[i] = old;
}

template <typename T>
int launch(int op, void* buffer, void* result, int64_t n, int rank, int peer, int num_ranks, const uint64_t* hb,
           int block, hipStream_t s) {
  const dim3 grid((unsigned)((n + block - 1) / block)), blk(block);
  T* b = static_cast<T*>(buffer);
  T* r = static_cast<T*>(result);
  switch (op) {
    case IRIS_P2P_LOAD: hipLaunchKernelGGL(load_kernel<T>, grid, blk, 0, s, b, r, n, rank, peer, hb); break;
    case IRIS_P2P_LOCAL_STORE: hipLaunchKernelGGL(local_store_kernel<T>, grid, blk, 0, s, r, n); break;
    case IRIS_P2P_STORE: hipLaunchKernelGGL(store_kernel<T>, grid, blk, 0, s, b, n, rank, peer, hb); break;
    case IRIS_P2P_ALL_LOAD: hipLaunchKernelGGL(all_load_kernel<T>, grid, blk, 0, s, b, r, n, rank, num_ranks, hb); break;
    case IRIS_P2P_ALL_STORE: hipLaunchKernelGGL(all_store_kernel<T>, grid, blk, 0, s, b, n, rank, num_ranks, hb); break;
    case IRIS_P2P_ATOMIC_ADD:
      if constexpr (sizeof(T) == 1) return hipErrorInvalidValue;
      else hipLaunchKernelGGL(atomic_add_kernel<T>, grid, blk, 0, s, b, n, rank, peer, hb);
      break;
    case IRIS_P2P_ATOMIC_XCHG:
      if constexpr (sizeof(T) == 1) return hipErrorInvalidValue;
      else hipLaunchKernelGGL(atomic_xchg_kernel<T>, grid, blk, 0, s, b, r, n, rank, peer, hb);
      break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

extern "C" int iris_p2p_bench_launch(int32_t op, int32_t dtype, void* buffer, void* result, int64_t n_elements,
                                     int32_t cur_rank, int32_t peer_rank, int32_t num_ranks,
                                     const uint64_t* heap_bases, int32_t block_size, void* stream) {
  if (n_elements < 0 || num_ranks <= 0 || cur_rank < 0 || cur_rank >= num_ranks) return hipErrorInvalidValue;
  if (block_size <= 0 || block_size > 1024) return hipErrorInvalidValue;
  const bool pairwise = op == IRIS_P2P_LOAD || op == IRIS_P2P_STORE || op == IRIS_P2P_ATOMIC_ADD || op == IRIS_P2P_ATOMIC_XCHG;
  if (pairwise && (peer_rank < 0 || peer_rank >= num_ranks)) return hipErrorInvalidValue;
  const bool needs_result = op == IRIS_P2P_LOAD || op == IRIS_P2P_LOCAL_STORE || op == IRIS_P2P_ALL_LOAD || op == IRIS_P2P_ATOMIC_XCHG;
  if (n_elements == 0) return hipSuccess;
  if (n_elements > (int64_t)block_size * 0x7fffffff) return hipErrorInvalidValue;
  if (op != IRIS_P2P_LOCAL_STORE && (!buffer || !heap_bases)) return hipErrorInvalidValue;
  if (needs_result && !result) return hipErrorInvalidValue;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case IRIS_DTYPE_F32: return launch<float>(op, buffer, result, n_elements, cur_rank, peer_rank, num_ranks, heap_bases, block_size, s);
    case IRIS_DTYPE_F16: return launch<_Float16>(op, buffer, result, n_elements, cur_rank, peer_rank, num_ranks, heap_bases, block_size, s);
    case IRIS_DTYPE_BF16: return launch<__bf16>(op, buffer, result, n_elements, cur_rank, peer_rank, num_ranks, heap_bases, block_size, s);
    case IRIS_DTYPE_I8: return launch<int8_t>(op, buffer, result, n_elements, cur_rank, peer_rank, num_ranks, heap_bases, block_size, s);
    case IRIS_DTYPE_I32: return launch<int32_t>(op, buffer, result, n_elements, cur_rank, peer_rank, num_ranks, heap_bases, block_size, s);
    default: return hipErrorInvalidValue;
  }
}
