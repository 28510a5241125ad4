// Device-side building blocks shared by the kernels of libmi355ccl: geometry constants, the
// 16-byte vector type, element traits (storage type, accumulation type, conversions) and the
// reduction chain.  Header-only, included by exactly one translation unit (mccl_kernels.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "mccl.h"

namespace {

constexpr int kWave = 64;               // one wavefront per workgroup (small / stream shapes)
constexpr int kBlockPersistent = 256;   // 4 wavefronts
constexpr int kUnrollPersistent = 2;    // vectors per lane per input per tile
constexpr int kMaxJobs = 64;            // independent reductions per launch
constexpr int kMaxSegs = 64;            // copy segments per launch
constexpr int kCopyUnroll = 2;          // vectors per lane per chunk
constexpr size_t kCopyChunk = (size_t)kWave * 16 * kCopyUnroll;  // 2 KiB per wavefront

// ------------------------------------------------------------------------------------------
// element types
// ------------------------------------------------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// The same vector behind a pointer that promises no alignment: global loads may be unaligned on
// this target (the hardware splits them), and an aligned address gets the same instruction.
typedef u32x4 u32x4_unaligned __attribute__((aligned(1)));

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

template <int DT>
struct Elem;

template <>
struct Elem<MCCL_BF16> {
  using store_t = uint16_t;
  using acc_t = float;
  static constexpr bool kIsFloat = true;
  static __device__ __forceinline__ acc_t load(store_t h) { return bits_to_f32((uint32_t)h << 16); }
  // round to nearest even; every NaN becomes 0x7FC0
  static __device__ __forceinline__ store_t store(acc_t f) {
    uint32_t u = f32_to_bits(f);
    uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    return (store_t)(((u & 0x7fffffffu) > 0x7f800000u) ? 0x7fc0u : r);
  }
};

template <>
struct Elem<MCCL_F16> {
  using store_t = uint16_t;
  using acc_t = float;
  static constexpr bool kIsFloat = true;
  static __device__ __forceinline__ acc_t load(store_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
  }
  // hardware convert is round-to-nearest-even with gradual underflow; NaN -> 0x7E00
  static __device__ __forceinline__ store_t store(acc_t f) {
    uint16_t r = __builtin_bit_cast(uint16_t, (_Float16)f);
    return (f != f) ? (store_t)0x7e00u : r;
  }
};

template <typename T, typename UT, int CODE>
struct IntElem {
  using store_t = T;
  using acc_t = T;
  using uacc_t = UT;
  static constexpr bool kIsFloat = false;
  static __device__ __forceinline__ acc_t load(store_t v) { return v; }
  static __device__ __forceinline__ store_t store(acc_t v) { return v; }
};
template <> struct Elem<MCCL_U8> : IntElem<uint8_t, uint8_t, MCCL_U8> {};
template <> struct Elem<MCCL_I8> : IntElem<int8_t, uint8_t, MCCL_I8> {};
template <> struct Elem<MCCL_I16> : IntElem<int16_t, uint16_t, MCCL_I16> {};
template <> struct Elem<MCCL_I32> : IntElem<int32_t, uint32_t, MCCL_I32> {};
template <> struct Elem<MCCL_I64> : IntElem<int64_t, uint64_t, MCCL_I64> {};

template <typename T>
struct FloatElem {
  using store_t = T;
  using acc_t = T;
  static constexpr bool kIsFloat = true;
  static __device__ __forceinline__ acc_t load(store_t v) { return v; }
  static __device__ __forceinline__ store_t store(acc_t v) { return v; }
};
template <> struct Elem<MCCL_F32> : FloatElem<float> {};
template <> struct Elem<MCCL_F64> : FloatElem<double> {};

// One 16-byte vector viewed as elements of the storage type.
template <int DT>
constexpr int vec_elems() { return 16 / (int)sizeof(typename Elem<DT>::store_t); }

template <int DT>
union VecU {
  u32x4 v;
  typename Elem<DT>::store_t e[vec_elems<DT>()];
};

// Element e of a vector.  One-byte types go through shifts on the 32-bit lanes: read through the
// union, the compiler re-types the 16-byte load as a byte vector and loses its cache hint on the way.
template <int DT>
__device__ __forceinline__ typename Elem<DT>::store_t vec_get(const VecU<DT>& x, int e) {
  using S = typename Elem<DT>::store_t;
  if constexpr (sizeof(S) == 1) return (S)(uint8_t)(x.v[e >> 2] >> ((e & 3) * 8));
  else return x.e[e];
}

template <int DT>
__device__ __forceinline__ void vec_set(VecU<DT>& x, int e, typename Elem<DT>::store_t val) {
  using S = typename Elem<DT>::store_t;
  if constexpr (sizeof(S) == 1) {  // x starts as zero: or the byte in
    x.v[e >> 2] |= (uint32_t)(uint8_t)val << ((uint32_t)(e & 3) * 8);
  } else {
    x.e[e] = val;
  }
}

// ------------------------------------------------------------------------------------------
// the reduction chain
// ------------------------------------------------------------------------------------------
// First element of the chain.  SUM/AVG start from literal +0 and add rank 0 (so an all -0
// column yields +0, as "result = 0; result = result + buf[r]" does); the other ops start
// from rank 0's value.
template <int DT, int OP>
__device__ __forceinline__ typename Elem<DT>::acc_t chain_first(typename Elem<DT>::acc_t x) {
  using A = typename Elem<DT>::acc_t;
  if constexpr (OP == MCCL_SUM || OP == MCCL_AVG) {
    if constexpr (Elem<DT>::kIsFloat) return (A)0 + x;
    else return x;
  } else {
    return x;
  }
}

template <int DT, int OP>
__device__ __forceinline__ typename Elem<DT>::acc_t chain_next(typename Elem<DT>::acc_t acc,
                                                                typename Elem<DT>::acc_t x) {
  using A = typename Elem<DT>::acc_t;
  if constexpr (Elem<DT>::kIsFloat) {
    if constexpr (OP == MCCL_SUM || OP == MCCL_AVG) return acc + x;
    else if constexpr (OP == MCCL_PROD) return acc * x;
    // MIN / MAX propagate NaN whatever the rank order: a NaN input replaces the accumulator, and
    // no later value replaces a NaN accumulator (both compares are false)
    else if constexpr (OP == MCCL_MIN) return (x < acc || x != x) ? x : acc;
    else return (x > acc || x != x) ? x : acc;
  } else {
    using U = typename Elem<DT>::uacc_t;
    if constexpr (OP == MCCL_SUM) return (A)(U)((U)acc + (U)x);
    else if constexpr (OP == MCCL_PROD) return (A)(U)((U)acc * (U)x);
    else if constexpr (OP == MCCL_MIN) return (x < acc) ? x : acc;
    else return (x > acc) ? x : acc;
  }
}

template <int DT, int OP>
__device__ __forceinline__ typename Elem<DT>::acc_t chain_last(typename Elem<DT>::acc_t acc, int n) {
  using A = typename Elem<DT>::acc_t;
  if constexpr (OP == MCCL_AVG) return acc / (A)n;
  else return acc;
}

}  // namespace
