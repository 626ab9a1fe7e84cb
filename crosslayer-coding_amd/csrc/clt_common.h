// Shared device/host helpers for the gfx950 CLT kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/clt_hip.h"

#define CLT_WAVE 64

typedef uint16_t bf16_t;  // raw bfloat16 bits

// ---------------------------------------------------------------- conversions
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) {
  return __uint_as_float(b << 16);
}

// round-to-nearest-even, NaN kept quiet (same rule torch uses for float->bfloat16)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float round_to_bf16(float f) {
  return bf16_bits_to_f32(f32_to_bf16_bits(f));
}

// IEEE half as raw bits, a type of its own so that templates tell it from bf16_t
struct f16_t { uint16_t bits; };

__host__ __device__ static inline float f16_bits_to_f32(uint32_t h) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint16_t b = (uint16_t)h;
  _Float16 v;
  __builtin_memcpy(&v, &b, 2);
  return (float)v;
#else
  const uint32_t sign = (h & 0x8000u) << 16, ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
  uint32_t u;
  if (ex == 0x1Fu) u = sign | 0x7F800000u | (man << 13);
  else if (ex != 0u) u = sign | ((ex + 112u) << 23) | (man << 13);
  else if (man == 0u) u = sign;
  else {
    int e = -1;
    uint32_t m = man;
    do { m <<= 1; ++e; } while ((m & 0x400u) == 0u);
    u = sign | ((uint32_t)(112 - e) << 23) | ((m & 0x3FFu) << 13);
  }
  float f;
  __builtin_memcpy(&f, &u, 4);
  return f;
#endif
}

// round-to-nearest-even (v_cvt_f16_f32 under the default rounding mode), NaN stays NaN
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  const _Float16 v = (_Float16)f;
  uint16_t b;
  __builtin_memcpy(&b, &v, 2);
  return b;
}

// Element traits: T is float, bf16_t (raw bits) or f16_t (raw bits).
//   IS16   16-bit element (eight per 16-byte vector, 16-bit ranking keys)
//   INF16  raw bits of +infinity of a 16-bit type
template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int VEC = 4;       // elements per 16-byte vector
  static constexpr int KEYBITS = 32;  // bits of the ranking key
  __device__ static __forceinline__ float to_f32(float v) { return v; }
  __device__ static __forceinline__ float from_f32(float v) { return v; }
  __device__ static __forceinline__ float round(float v) { return v; }
  __device__ static __forceinline__ uint32_t raw(float v) { return __float_as_uint(v); }
  __device__ static __forceinline__ float from_raw(uint32_t r) { return __uint_as_float(r); }
};
template <> struct Elem<bf16_t> {
  static constexpr int VEC = 8;
  static constexpr int KEYBITS = 16;
  static constexpr uint32_t INF16 = 0x7F80u;
  __device__ static __forceinline__ float to_f32(bf16_t v) { return bf16_bits_to_f32(v); }
  __device__ static __forceinline__ bf16_t from_f32(float v) { return (bf16_t)f32_to_bf16_bits(v); }
  __device__ static __forceinline__ float round(float v) { return round_to_bf16(v); }
  __device__ static __forceinline__ uint32_t raw(bf16_t v) { return v; }
  __device__ static __forceinline__ bf16_t from_raw(uint32_t r) { return (bf16_t)r; }
};

template <> struct Elem<f16_t> {
  static constexpr int VEC = 8;
  static constexpr int KEYBITS = 16;
  static constexpr uint32_t INF16 = 0x7C00u;
  __device__ static __forceinline__ float to_f32(f16_t v) { return f16_bits_to_f32(v.bits); }
  __device__ static __forceinline__ f16_t from_f32(float v) { return f16_t{(uint16_t)f32_to_f16_bits(v)}; }
  __device__ static __forceinline__ float round(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }
  __device__ static __forceinline__ uint32_t raw(f16_t v) { return v.bits; }
  __device__ static __forceinline__ f16_t from_raw(uint32_t r) { return f16_t{(uint16_t)r}; }
};
template <typename T> struct IsHalf { static constexpr bool value = false; };
template <> struct IsHalf<f16_t> { static constexpr bool value = true; };

// Two 16-bit elements of one 32-bit word (low half first) as floats, and back (round to nearest even).
template <typename T> __device__ __forceinline__ void unpack_pair(uint32_t w, float &lo, float &hi) {
  if constexpr (IsHalf<T>::value) {
    lo = f16_bits_to_f32(w & 0xFFFFu);
    hi = f16_bits_to_f32(w >> 16);
  } else {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xFFFF0000u);
  }
}
template <typename T> __device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  if constexpr (IsHalf<T>::value) return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
  else return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}
// raw 16 bits of a float that is a value of the 16-bit type T (exact)
template <typename T> __device__ __forceinline__ uint32_t raw16_of(float v) {
  if constexpr (IsHalf<T>::value) return f32_to_f16_bits(v);
  else return __float_as_uint(v) >> 16;
}
// dtype code -> element size in bytes (0: not a model dtype)
static inline int clt_elem_bytes(int dtype) { return dtype == CLT_F32 ? 4 : (dtype == CLT_BF16 || dtype == CLT_F16) ? 2 : 0; }
static inline bool clt_model_dtype(int dtype) { return dtype == CLT_F32 || dtype == CLT_BF16 || dtype == CLT_F16; }

// ---------------------------------------------------------------- ranking keys
// Order-preserving unsigned key: ascending float order, -0.0 == +0.0, NaN on top.
__device__ __forceinline__ uint32_t rank_key32(float x) {
  uint32_t u = __float_as_uint(x);
  if (x != x) return 0xFFFFFFFFu;
  if (u == 0x80000000u) u = 0u;
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
// Key of width KB (16: for values that are exactly representable in bf16).
template <int KB> __device__ __forceinline__ uint32_t rank_key(float x) {
  return KB == 32 ? rank_key32(x) : (rank_key32(x) >> 16);
}
// Float whose key is `key` (the lowest such float for 16-bit keys).
template <int KB> __device__ __host__ __forceinline__ uint32_t key_to_f32_bits(uint32_t key) {
  uint32_t k32 = KB == 32 ? key : ((key << 16) | ((key & 0x8000u) ? 0u : 0xFFFFu));
  return (k32 & 0x80000000u) ? (k32 & 0x7FFFFFFFu) : ~k32;
}

// The same by element type.  `x` must be a value of T (the key of a 16-bit type is taken from its own bits).
template <typename T> __device__ __forceinline__ uint32_t rank_key_of(float x) {
  if constexpr (IsHalf<T>::value) {
    if (x != x) return 0xFFFFu;
    uint32_t h = f32_to_f16_bits(x);
    if (h == 0x8000u) h = 0u;
    return (h & 0x8000u) ? (~h & 0xFFFFu) : (h | 0x8000u);
  } else {
    return rank_key<Elem<T>::KEYBITS>(x);
  }
}
template <typename T> __device__ __host__ __forceinline__ uint32_t key_value_bits(uint32_t key) {
  if constexpr (IsHalf<T>::value) {
    const uint32_t h = (key & 0x8000u) ? (key & 0x7FFFu) : (~key & 0xFFFFu);
    const float f = f16_bits_to_f32(h);
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    return u;
  } else {
    return key_to_f32_bits<Elem<T>::KEYBITS>(key);
  }
}

// ---------------------------------------------------------------- wave helpers
__device__ __forceinline__ int lane_id() { return threadIdx.x & (CLT_WAVE - 1); }

// number of set bits of `mask` strictly below this lane
__device__ __forceinline__ uint32_t mbcnt64(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

__device__ __forceinline__ uint64_t ballot64(bool p) { return __ballot(p); }

// ---------------------------------------------------------------- packed decoder rows
// Row pitch (elements) of the feature-major decoder slab [n_dec][F][pitch].  A row that is a whole,
// EVEN number of 128-byte cache lines is padded by one line: with an even line pitch the same column part
// of every row falls on a fraction of the 16 L2 channels (pitch 16 lines: on ONE channel), so a kernel
// that gathers one column part per XCD would use only that fraction of its L2; an odd pitch spreads any
// column part over all channels and sets.  Other widths are stored densely.
__host__ __device__ static inline int64_t clt_pitch(int64_t d, int elem_bytes) {
  const int64_t row_bytes = d * elem_bytes;
  if (row_bytes % 128 != 0 || (row_bytes / 128) % 2 != 0) return d;
  return d + 128 / elem_bytes;
}

// ---------------------------------------------------------------- host helpers
static inline int clt_check_launch() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? CLT_OK : CLT_ERR_LAUNCH;
}
static inline bool clt_aligned16(const void *p) { return (((uintptr_t)p) & 15u) == 0; }
static inline int64_t clt_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
