// Shared device-side definitions: element traits, order keys, bucket geometry.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/approx_topk_hip.h"

namespace atk {

// ---------------------------------------------------------------------------
// Element traits.  Kernels move elements as raw bit patterns (`raw_t`) so that
// outputs are bit-identical to inputs, and compare them through `key_t`, an
// unsigned integer whose order is the selection order:
//   floats: IEEE value order, -0.0 == +0.0, every NaN equal and above +inf;
//   signed integers: value order; unsigned: identity.
// `pad_raw` is the element a padded position holds (the dtype's finite minimum,
// as torch.finfo(dtype).min / torch.iinfo(dtype).min).  `unkey` gives back the
// element of a key where `key_is_exact` says the key names one bit pattern
// only (not a zero, whose sign the key drops, and not a NaN).
// ---------------------------------------------------------------------------
template <int DT> struct Elem;

template <> struct Elem<ATK_F32> {
  using raw_t = uint32_t; using key_t = uint32_t;
  static constexpr int key_bits = 32;
  static constexpr raw_t pad_raw = 0xff7fffffu;
  __host__ __device__ static inline key_t key(raw_t u) {
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0xffffffffu;
    if (u == 0x80000000u) u = 0;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  }
  __host__ __device__ static inline raw_t unkey(key_t k) { return (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k; }
  __host__ __device__ static inline bool key_is_exact(key_t k) { return k != 0x80000000u && k != 0xffffffffu; }
};

template <uint16_t INF, uint16_t PAD> struct Elem16Float {
  using raw_t = uint16_t; using key_t = uint32_t;
  static constexpr int key_bits = 16;
  static constexpr raw_t pad_raw = PAD;
  __host__ __device__ static inline key_t key(raw_t u) {
    if ((u & 0x7fffu) > INF) return 0xffffu;
    if (u == 0x8000u) u = 0;
    return (u & 0x8000u) ? (uint16_t)~u : (uint16_t)(u | 0x8000u);
  }
  __host__ __device__ static inline raw_t unkey(key_t k) { return (k & 0x8000u) ? (raw_t)(k & 0x7fffu) : (raw_t)~k; }
  __host__ __device__ static inline bool key_is_exact(key_t k) { return k != 0x8000u && k != 0xffffu; }
};
template <> struct Elem<ATK_F16> : Elem16Float<0x7c00u, 0xfbffu> {};
template <> struct Elem<ATK_BF16> : Elem16Float<0x7f80u, 0xff7fu> {};

template <> struct Elem<ATK_F64> {
  using raw_t = uint64_t; using key_t = uint64_t;
  static constexpr int key_bits = 64;
  static constexpr raw_t pad_raw = 0xffefffffffffffffull;
  __host__ __device__ static inline key_t key(raw_t u) {
    if ((u & 0x7fffffffffffffffull) > 0x7ff0000000000000ull) return ~0ull;
    if (u == 0x8000000000000000ull) u = 0;
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
  }
  __host__ __device__ static inline raw_t unkey(key_t k) { return (k >> 63) ? (k & 0x7fffffffffffffffull) : ~k; }
  __host__ __device__ static inline bool key_is_exact(key_t k) { return k != 0x8000000000000000ull && k != ~0ull; }
};

template <> struct Elem<ATK_U8> {
  using raw_t = uint8_t; using key_t = uint32_t;
  static constexpr int key_bits = 8;
  static constexpr raw_t pad_raw = 0;
  __host__ __device__ static inline key_t key(raw_t u) { return u; }
  __host__ __device__ static inline raw_t unkey(key_t k) { return (raw_t)k; }
  __host__ __device__ static inline bool key_is_exact(key_t) { return true; }
};
template <> struct Elem<ATK_I8> {
  using raw_t = uint8_t; using key_t = uint32_t;
  static constexpr int key_bits = 8;
  static constexpr raw_t pad_raw = 0x80u;
  __host__ __device__ static inline key_t key(raw_t u) { return (uint8_t)(u ^ 0x80u); }
  __host__ __device__ static inline raw_t unkey(key_t k) { return (raw_t)(k ^ 0x80u); }
  __host__ __device__ static inline bool key_is_exact(key_t) { return true; }
};
template <> struct Elem<ATK_I16> {
  using raw_t = uint16_t; using key_t = uint32_t;
  static constexpr int key_bits = 16;
  static constexpr raw_t pad_raw = 0x8000u;
  __host__ __device__ static inline key_t key(raw_t u) { return (uint16_t)(u ^ 0x8000u); }
  __host__ __device__ static inline raw_t unkey(key_t k) { return (raw_t)(k ^ 0x8000u); }
  __host__ __device__ static inline bool key_is_exact(key_t) { return true; }
};
template <> struct Elem<ATK_I32> {
  using raw_t = uint32_t; using key_t = uint32_t;
  static constexpr int key_bits = 32;
  static constexpr raw_t pad_raw = 0x80000000u;
  __host__ __device__ static inline key_t key(raw_t u) { return u ^ 0x80000000u; }
  __host__ __device__ static inline raw_t unkey(key_t k) { return k ^ 0x80000000u; }
  __host__ __device__ static inline bool key_is_exact(key_t) { return true; }
};
template <> struct Elem<ATK_I64> {
  using raw_t = uint64_t; using key_t = uint64_t;
  static constexpr int key_bits = 64;
  static constexpr raw_t pad_raw = 0x8000000000000000ull;
  __host__ __device__ static inline key_t key(raw_t u) { return u ^ 0x8000000000000000ull; }
  __host__ __device__ static inline raw_t unkey(key_t k) { return k ^ 0x8000000000000000ull; }
  __host__ __device__ static inline bool key_is_exact(key_t) { return true; }
};

// Destination of the result indices: int64 (the operator's contract) or, for
// the compact entry points, int32.  `at` counts indices, not bytes.
struct IndexOut {
  void* base;
  int narrow;  // != 0: int32_t
  __device__ __forceinline__ void put(int64_t at, int64_t index) const {
    if (narrow) static_cast<int32_t*>(base)[at] = (int32_t)index;
    else static_cast<int64_t*>(base)[at] = index;
  }
};

__host__ __device__ constexpr int elem_bytes(int dtype) {
  switch (dtype) {
    case ATK_F32: case ATK_I32: return 4;
    case ATK_F16: case ATK_BF16: case ATK_I16: return 2;
    case ATK_F64: case ATK_I64: return 8;
    case ATK_U8: case ATK_I8: return 1;
  }
  return 0;
}

// The element type code of a traits type.
template <typename E> struct DtypeOf;
template <int DT> struct DtypeOf<Elem<DT>> { static constexpr int value = DT; };

// ---------------------------------------------------------------------------
// Bucket geometry: first position, stride between members and member count of
// bucket c out of b over a row of n elements.  The two padded layouts count
// positions >= n, which hold `pad_raw`.
// ---------------------------------------------------------------------------
struct Bucket { int64_t start, stride, count; };

__host__ __device__ inline Bucket bucket_of(int64_t n, int64_t b, int64_t c, int layout) {
  Bucket g;
  const int64_t base = n / b, r = n - base * b;
  switch (layout) {
    case ATK_INTERLEAVED:
      g.start = c; g.stride = b; g.count = base + (c < r ? 1 : 0); break;
    case ATK_BALANCED:
      g.start = c * base + (c < r ? c : r); g.stride = 1; g.count = base + (c < r ? 1 : 0); break;
    case ATK_CEIL_CHUNK: {
      const int64_t m = (n + b - 1) / b;
      g.start = c * m; g.stride = 1; g.count = m; break;
    }
    default: {  // ATK_INTERLEAVED_PADDED
      const int64_t m = (n + b - 1) / b;
      g.start = c; g.stride = b; g.count = m; break;
    }
  }
  return g;
}

// Run `...` once with `E` naming the Elem<> of a runtime dtype; `on_bad` runs
// for an unknown dtype.
#define ATK_DTYPE_CASE(DT, E, ...) \
  case DT: { using E = ::atk::Elem<DT>; __VA_ARGS__; break; }
#define ATK_DTYPE_SWITCH(dtype, E, on_bad, ...)   \
  switch (dtype) {                                \
    ATK_DTYPE_CASE(ATK_F32, E, __VA_ARGS__)       \
    ATK_DTYPE_CASE(ATK_F16, E, __VA_ARGS__)       \
    ATK_DTYPE_CASE(ATK_BF16, E, __VA_ARGS__)      \
    ATK_DTYPE_CASE(ATK_F64, E, __VA_ARGS__)       \
    ATK_DTYPE_CASE(ATK_U8, E, __VA_ARGS__)        \
    ATK_DTYPE_CASE(ATK_I8, E, __VA_ARGS__)        \
    ATK_DTYPE_CASE(ATK_I16, E, __VA_ARGS__)       \
    ATK_DTYPE_CASE(ATK_I32, E, __VA_ARGS__)       \
    ATK_DTYPE_CASE(ATK_I64, E, __VA_ARGS__)       \
    default: { on_bad; }                          \
  }

}  // namespace atk
