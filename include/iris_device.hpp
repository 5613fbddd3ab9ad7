// iris_device.hpp -- device-side remote memory access on the symmetric heap,
// for HIP kernels on gfx950.  Header only.
//
// The HIP counterpart of the Triton device functions of ROCm/iris
// (iris/iris.py:317-521): a pointer into the caller's heap is rebased onto
// another rank's heap with the table of heap bases, then loaded, stored or
// updated atomically there.  Every function is per lane: the Triton versions
// act on a block of pointers with a mask, here each thread passes its own
// pointer and its own `mask` bit (a lane whose mask is false does nothing and
// gets T{} back).
//
//   translate    iris/iris.py:317-339      atomic_add   iris/iris.py:428-449
//   load         iris/iris.py:342-359      atomic_sub   iris/iris.py:452-473
//   store        iris/iris.py:362-379      atomic_cas   iris/iris.py:476-497
//   get          iris/iris.py:382-402      atomic_xchg  iris/iris.py:500-521
//   put          iris/iris.py:405-425
//
// `Sem` and `Scope` are the reference's sem= ("acquire", "release",
// "acq_rel"; relaxed is the extra that flag protocols with write-through data
// use) and scope= ("cta", "gpu", "sys") arguments as template parameters.
//
// Element types: 32- and 64-bit integers and float take the hardware atomics;
// 16-bit types (_Float16, __bf16, int16_t) go through a compare-and-swap loop
// on the aligned 32-bit word that holds them.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace iris {

enum class Sem { relaxed, acquire, release, acq_rel };
enum class Scope { cta, gpu, sys };

namespace detail {

template <Sem S>
constexpr int order() {
  return S == Sem::relaxed ? __ATOMIC_RELAXED
         : S == Sem::acquire ? __ATOMIC_ACQUIRE
         : S == Sem::release ? __ATOMIC_RELEASE
                             : __ATOMIC_ACQ_REL;
}
// the failure order of a compare-exchange may not release
template <Sem S>
constexpr int load_order() {
  return (S == Sem::acquire || S == Sem::acq_rel) ? __ATOMIC_ACQUIRE : __ATOMIC_RELAXED;
}
template <Scope C>
constexpr int scope() {
  return C == Scope::cta ? __HIP_MEMORY_SCOPE_WORKGROUP
         : C == Scope::gpu ? __HIP_MEMORY_SCOPE_AGENT
                           : __HIP_MEMORY_SCOPE_SYSTEM;
}

template <typename T>
constexpr bool is_native_atomic =
    (std::is_integral<T>::value && (sizeof(T) == 4 || sizeof(T) == 8)) || std::is_same<T, float>::value;

// Read-modify-write of a 16-bit element by compare-and-swap on its 32-bit
// word.  F maps the old element to the new one; returns the old element.
template <typename T, Sem S, Scope C, typename F>
__device__ inline T rmw16(T* ptr, F f) {
  static_assert(sizeof(T) == 2, "16-bit elements");
  const uintptr_t addr = reinterpret_cast<uintptr_t>(ptr);
  unsigned int* word = reinterpret_cast<unsigned int*>(addr & ~uintptr_t(3));
  const int shift = (addr & 2) ? 16 : 0;
  unsigned int old = __hip_atomic_load(word, __ATOMIC_RELAXED, scope<C>());
  for (;;) {
    const unsigned short cur_bits = static_cast<unsigned short>(old >> shift);
    const T cur = __builtin_bit_cast(T, cur_bits);
    const unsigned short new_bits = __builtin_bit_cast(unsigned short, f(cur));
    const unsigned int repl = (old & ~(0xFFFFu << shift)) | (static_cast<unsigned int>(new_bits) << shift);
    if (__hip_atomic_compare_exchange_strong(word, &old, repl, order<S>(), load_order<S>(), scope<C>()))
      return cur;
  }
}

}  // namespace detail

// `ptr`, an address in rank `cur_rank`'s heap, as the same offset in rank
// `target_rank`'s heap.
template <typename T>
__device__ inline T* translate(T* ptr, int cur_rank, int target_rank, const uint64_t* heap_bases) {
  const uint64_t offset = reinterpret_cast<uint64_t>(ptr) - heap_bases[cur_rank];
  return reinterpret_cast<T*>(heap_bases[target_rank] + offset);
}

// Value at `src`'s place on rank `target_rank`.
template <typename T>
__device__ inline T load(const T* src, int cur_rank, int target_rank, const uint64_t* heap_bases, bool mask = true) {
  if (!mask) return T{};
  return *translate(src, cur_rank, target_rank, heap_bases);
}

// Write `data` to `dst`'s place on rank `target_rank`.
template <typename T>
__device__ inline void store(T* dst, T data, int cur_rank, int target_rank, const uint64_t* heap_bases,
                             bool mask = true) {
  if (mask) *translate(dst, cur_rank, target_rank, heap_bases) = data;
}

// Copy from `src`'s place on rank `target_rank` to the local `dst`.
template <typename T>
__device__ inline void get(const T* src, T* dst, int cur_rank, int target_rank, const uint64_t* heap_bases,
                           bool mask = true) {
  if (mask) *dst = *translate(src, cur_rank, target_rank, heap_bases);
}

// Copy from the local `src` to `dst`'s place on rank `target_rank`.
template <typename T>
__device__ inline void put(const T* src, T* dst, int cur_rank, int target_rank, const uint64_t* heap_bases,
                           bool mask = true) {
  if (mask) *translate(dst, cur_rank, target_rank, heap_bases) = *src;
}

// Atomic add on rank `target_rank`; returns the value before the add.
template <Sem S = Sem::acq_rel, Scope C = Scope::sys, typename T>
__device__ inline T atomic_add(T* ptr, T data, int cur_rank, int target_rank, const uint64_t* heap_bases,
                               bool mask = true) {
  if (!mask) return T{};
  T* p = translate(ptr, cur_rank, target_rank, heap_bases);
  if constexpr (detail::is_native_atomic<T>) {
    return __hip_atomic_fetch_add(p, data, detail::order<S>(), detail::scope<C>());
  } else {
    return detail::rmw16<T, S, C>(p, [data](T cur) { return static_cast<T>(static_cast<float>(cur) + static_cast<float>(data)); });
  }
}

// Atomic subtract on rank `target_rank`; returns the value before.
template <Sem S = Sem::acq_rel, Scope C = Scope::sys, typename T>
__device__ inline T atomic_sub(T* ptr, T data, int cur_rank, int target_rank, const uint64_t* heap_bases,
                               bool mask = true) {
  if (!mask) return T{};
  T* p = translate(ptr, cur_rank, target_rank, heap_bases);
  if constexpr (std::is_integral<T>::value && detail::is_native_atomic<T>) {
    return __hip_atomic_fetch_sub(p, data, detail::order<S>(), detail::scope<C>());
  } else if constexpr (std::is_same<T, float>::value) {
    return __hip_atomic_fetch_add(p, -data, detail::order<S>(), detail::scope<C>());
  } else {
    return detail::rmw16<T, S, C>(p, [data](T cur) { return static_cast<T>(static_cast<float>(cur) - static_cast<float>(data)); });
  }
}

// Compare-and-swap on rank `target_rank`: writes `value` if the element equals
// `compare`; returns the value found.
template <Sem S = Sem::acq_rel, Scope C = Scope::sys, typename T>
__device__ inline T atomic_cas(T* ptr, T compare, T value, int cur_rank, int target_rank,
                               const uint64_t* heap_bases) {
  T* p = translate(ptr, cur_rank, target_rank, heap_bases);
  if constexpr (detail::is_native_atomic<T> && std::is_integral<T>::value) {
    T expected = compare;
    __hip_atomic_compare_exchange_strong(p, &expected, value, detail::order<S>(), detail::load_order<S>(),
                                         detail::scope<C>());
    return expected;
  } else if constexpr (std::is_same<T, float>::value) {
    unsigned int expected = __builtin_bit_cast(unsigned int, compare);
    __hip_atomic_compare_exchange_strong(reinterpret_cast<unsigned int*>(p), &expected,
                                         __builtin_bit_cast(unsigned int, value), detail::order<S>(),
                                         detail::load_order<S>(), detail::scope<C>());
    return __builtin_bit_cast(float, expected);
  } else {
    const unsigned short cmp_bits = __builtin_bit_cast(unsigned short, compare);
    return detail::rmw16<T, S, C>(p, [cmp_bits, value](T cur) {
      return __builtin_bit_cast(unsigned short, cur) == cmp_bits ? value : cur;
    });
  }
}

// Atomic exchange on rank `target_rank`; returns the value before.
template <Sem S = Sem::acq_rel, Scope C = Scope::sys, typename T>
__device__ inline T atomic_xchg(T* ptr, T value, int cur_rank, int target_rank, const uint64_t* heap_bases,
                                bool mask = true) {
  if (!mask) return T{};
  T* p = translate(ptr, cur_rank, target_rank, heap_bases);
  if constexpr (detail::is_native_atomic<T> && std::is_integral<T>::value) {
    return __hip_atomic_exchange(p, value, detail::order<S>(), detail::scope<C>());
  } else if constexpr (std::is_same<T, float>::value) {
    const unsigned int old = __hip_atomic_exchange(reinterpret_cast<unsigned int*>(p),
                                                   __builtin_bit_cast(unsigned int, value), detail::order<S>(),
                                                   detail::scope<C>());
    return __builtin_bit_cast(float, old);
  } else {
    return detail::rmw16<T, S, C>(p, [value](T) { return value; });
  }
}

}  // namespace iris
