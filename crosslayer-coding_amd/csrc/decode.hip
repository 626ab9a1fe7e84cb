// Sparse cross-layer decode, decoder repacking, densify and decoder norms.
//
// Decode (reference clt/models/decoder.py:176-340): the reference multiplies dense
// [T,F] activations that are >99 % zeros by every decoder.  Here each (token, target)
// pair is one wavefront that walks the survivor rows of the sources s <= t, fetches the
// decoder vector of every active feature (feature-major packing: one contiguous
// d-element run, 16 bytes per lane per load) and accumulates in fp32 registers; the
// output row is written once.
#include <type_traits>
#include "clt_common.h"

namespace {

// Row layout seen by one wavefront: NF full chunks of 64 lanes x 16 bytes, then an optional
// tail chunk - TAIL 1: 64 lanes x 8 bytes (exactly fills the row), TAIL 2: a 16-byte chunk
// in which only the leading lanes are inside the row.
template <typename T> struct WVec;
template <> struct WVec<float> {
  static constexpr int V = 4;   // elements per 16 bytes
  __device__ static __forceinline__ void fma16(float *acc, const uint4 &w, float v) {
    acc[0] = fmaf(v, __uint_as_float(w.x), acc[0]); acc[1] = fmaf(v, __uint_as_float(w.y), acc[1]);
    acc[2] = fmaf(v, __uint_as_float(w.z), acc[2]); acc[3] = fmaf(v, __uint_as_float(w.w), acc[3]);
  }
  __device__ static __forceinline__ void fma8(float *acc, const uint2 &w, float v) {
    acc[0] = fmaf(v, __uint_as_float(w.x), acc[0]); acc[1] = fmaf(v, __uint_as_float(w.y), acc[1]);
  }
};
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

template <> struct WVec<bf16_t> {
  static constexpr int V = 8;
  // Two survivors at once: for each pair of bf16 weights in a 32-bit word, a byte permute puts
  // the same element of both rows side by side and v_dot2c_f32_bf16 multiplies them with the two
  // activation values (bf16 pair `vv`) and accumulates in fp32 - one op per element instead of two.
  // `vp`: the two activation values as raw 16-bit elements, (first | second << 16)
  __device__ static __forceinline__ void dot32(float *acc, uint32_t a, uint32_t b, uint32_t vp) {
    const bf16x2_t vv = __builtin_bit_cast(bf16x2_t, vp);
    const uint32_t lo = __builtin_amdgcn_perm(b, a, 0x05040100u);   // (a.lo16, b.lo16)
    const uint32_t hi = __builtin_amdgcn_perm(b, a, 0x07060302u);   // (a.hi16, b.hi16)
    acc[0] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, lo), vv, acc[0], false);
    acc[1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, hi), vv, acc[1], false);
  }
  __device__ static __forceinline__ void dot16(float *acc, const uint4 &a, const uint4 &b, uint32_t vp) {
    dot32(acc, a.x, b.x, vp); dot32(acc + 2, a.y, b.y, vp); dot32(acc + 4, a.z, b.z, vp); dot32(acc + 6, a.w, b.w, vp);
  }
  __device__ static __forceinline__ void dot8(float *acc, const uint2 &a, const uint2 &b, uint32_t vp) {
    dot32(acc, a.x, b.x, vp); dot32(acc + 2, a.y, b.y, vp);
  }
  __device__ static __forceinline__ void fma32(float *acc, uint32_t u, float v) {
    acc[0] = fmaf(v, __uint_as_float(u << 16), acc[0]);
    acc[1] = fmaf(v, __uint_as_float(u & 0xFFFF0000u), acc[1]);
  }
  __device__ static __forceinline__ void fma16(float *acc, const uint4 &w, float v) {
    fma32(acc, w.x, v); fma32(acc + 2, w.y, v); fma32(acc + 4, w.z, v); fma32(acc + 6, w.w, v);
  }
  __device__ static __forceinline__ void fma8(float *acc, const uint2 &w, float v) {
    fma32(acc, w.x, v); fma32(acc + 2, w.y, v);
  }
};

// IEEE half: the same scheme with v_dot2_f32_f16 (exact products, fp32 accumulation)
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
template <> struct WVec<f16_t> {
  static constexpr int V = 8;
  __device__ static __forceinline__ void dot32(float *acc, uint32_t a, uint32_t b, uint32_t vp) {
    const f16x2_t vv = __builtin_bit_cast(f16x2_t, vp);
    const uint32_t lo = __builtin_amdgcn_perm(b, a, 0x05040100u);
    const uint32_t hi = __builtin_amdgcn_perm(b, a, 0x07060302u);
    acc[0] = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, lo), vv, acc[0], false);
    acc[1] = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, hi), vv, acc[1], false);
  }
  __device__ static __forceinline__ void dot16(float *acc, const uint4 &a, const uint4 &b, uint32_t vp) {
    dot32(acc, a.x, b.x, vp); dot32(acc + 2, a.y, b.y, vp); dot32(acc + 4, a.z, b.z, vp); dot32(acc + 6, a.w, b.w, vp);
  }
  __device__ static __forceinline__ void dot8(float *acc, const uint2 &a, const uint2 &b, uint32_t vp) {
    dot32(acc, a.x, b.x, vp); dot32(acc + 2, a.y, b.y, vp);
  }
  __device__ static __forceinline__ void fma32(float *acc, uint32_t u, float v) {
    float lo, hi;
    unpack_pair<f16_t>(u, lo, hi);
    acc[0] = fmaf(v, lo, acc[0]);
    acc[1] = fmaf(v, hi, acc[1]);
  }
  __device__ static __forceinline__ void fma16(float *acc, const uint4 &w, float v) {
    fma32(acc, w.x, v); fma32(acc + 2, w.y, v); fma32(acc + 4, w.z, v); fma32(acc + 6, w.w, v);
  }
  __device__ static __forceinline__ void fma8(float *acc, const uint2 &w, float v) {
    fma32(acc, w.x, v); fma32(acc + 2, w.y, v);
  }
};

__device__ __forceinline__ int64_t decoder_slot(int tying, int64_t s, int64_t t, int64_t L) {
  if (tying == CLT_TYING_PER_SOURCE) return s;
  if (tying == CLT_TYING_PER_TARGET) return t;
  return s * L - (s * (s - 1)) / 2 + (t - s);
}

static inline int64_t decoder_slot_host(int tying, int64_t s, int64_t t, int64_t L) {
  if (tying == CLT_TYING_PER_SOURCE) return s;
  if (tying == CLT_TYING_PER_TARGET) return t;
  return s * L - (s * (s - 1)) / 2 + (t - s);
}

// UU decoder vectors in flight: the row pieces of one lane plus the (wave-uniform) weights.
template <typename T, int NF, int TAIL, int UU> struct RowBatch {
  uint4 wq[UU][NF > 0 ? NF : 1];
  uint4 wt16[UU];
  uint2 wt8[UU];
  float v[UU];

  // request rows i0 .. i0+UU-1 of the 64 survivors held one per lane in (my_col, my_val)
  __device__ __forceinline__ void load(const T *wbase, int64_t d, int32_t my_col, float my_val, int i0, int n,
                                       int lane, int64_t tail_off, bool tail_on) {
    constexpr int V = WVec<T>::V;
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      const int idx = (i0 + u) < n ? (i0 + u) : (n - 1);   // clamp: a repeated fetch, weight 0
      const int32_t f = __builtin_amdgcn_readlane(my_col, idx);
      const float vv = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(my_val), idx));
      v[u] = (i0 + u) < n ? vv : 0.0f;
      const T *wrow = wbase + (int64_t)f * d;
#pragma unroll
      for (int c = 0; c < NF; ++c) wq[u][c] = *reinterpret_cast<const uint4 *>(wrow + (int64_t)c * 64 * V + (int64_t)lane * V);
      if (TAIL == 1) wt8[u] = *reinterpret_cast<const uint2 *>(wrow + tail_off);
      if (TAIL == 2) wt16[u] = tail_on ? *reinterpret_cast<const uint4 *>(wrow + tail_off) : make_uint4(0, 0, 0, 0);
    }
  }

  __device__ __forceinline__ void consume(float *acc) const {
    constexpr int V = WVec<T>::V;
    if constexpr (sizeof(T) == 2 && (UU % 2) == 0) {
      // bf16: the activation values are exact bf16 numbers, so two of them fit one dot2 operand
#pragma unroll
      for (int u = 0; u < UU; u += 2) {
        const uint32_t vv = raw16_of<T>(v[u]) | (raw16_of<T>(v[u + 1]) << 16);
#pragma unroll
        for (int c = 0; c < NF; ++c) WVec<T>::dot16(acc + c * V, wq[u][c], wq[u + 1][c], vv);
        if (TAIL == 1) WVec<T>::dot8(acc + NF * V, wt8[u], wt8[u + 1], vv);
        if (TAIL == 2) WVec<T>::dot16(acc + NF * V, wt16[u], wt16[u + 1], vv);
      }
    } else {
#pragma unroll
      for (int u = 0; u < UU; ++u) {
#pragma unroll
        for (int c = 0; c < NF; ++c) WVec<T>::fma16(acc + c * V, wq[u][c], v[u]);
        if (TAIL == 1) WVec<T>::fma8(acc + NF * V, wt8[u], v[u]);
        if (TAIL == 2) WVec<T>::fma16(acc + NF * V, wt16[u], v[u]);
      }
    }
  }
};

// Fetch UU decoder vectors (all requests issued before the first multiply) and accumulate.
template <typename T, int NF, int TAIL, int UU>
__device__ __forceinline__ void decode_batch(float *acc, const T *wbase, int64_t d, int32_t my_col, float my_val,
                                             int i0, int n, int lane, int64_t tail_off, bool tail_on) {
  RowBatch<T, NF, TAIL, UU> rb;
  rb.load(wbase, d, my_col, my_val, i0, n, lane, tail_off, tail_on);
  rb.consume(acc);
}

// Up to 64 survivors (one per lane) with two batches in flight: while one batch is multiplied
// the next one is already on its way.
template <typename T, int NF, int TAIL, int UU>
__device__ __forceinline__ void decode_chunk_pipelined(float *acc, const T *wbase, int64_t d, int32_t my_col,
                                                       float my_val, int n, int lane, int64_t tail_off, bool tail_on) {
  RowBatch<T, NF, TAIL, UU> ra, rb;
  ra.load(wbase, d, my_col, my_val, 0, n, lane, tail_off, tail_on);
  for (int i0 = 0; i0 < n; i0 += 2 * UU) {
    if (i0 + UU < n) rb.load(wbase, d, my_col, my_val, i0 + UU, n, lane, tail_off, tail_on);
    ra.consume(acc);
    if (i0 + UU < n) {
      if (i0 + 2 * UU < n) ra.load(wbase, d, my_col, my_val, i0 + 2 * UU, n, lane, tail_off, tail_on);
      rb.consume(acc);
    }
  }
}

// The partial rows are touched once per launch: streaming loads / stores keep them from pushing the
// decoder slice out of the L2.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ldg_stream4(const float *p) {
  const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stg_stream4(float *p, float4 v) {
  f32x4_t q = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(q, reinterpret_cast<f32x4_t *>(p));
}

template <typename T, int NF, int TAIL, bool SLICED> constexpr int decode_min_waves() {
  constexpr int V = 16 / (int)sizeof(T);
  constexpr int nacc = NF * V + (TAIL == 1 ? V / 2 : TAIL == 2 ? V : 0);
  return (SLICED && sizeof(T) == 2 && nacc <= 12) ? 4 : 1;
}

constexpr int SLICED_NTOK = 4;   // tokens per wavefront in the sliced kernel

// One wavefront per (target, token): walks all sources s <= t, accumulates in registers,
// writes the output row once.  Used for small batches.
//
// SLICED (large batches): one launch per source layer `src`; one wavefront per
// (target >= src, token, feature slice).  The feature axis is cut into `ns` slices and block b
// works on slice b % ns.  Workgroups are handed to the XCDs round-robin, so with ns = 8 each
// XCD sees one slice of a decoder matrix (1/8 of its rows); blocks are ordered target-major,
// so at any moment the wavefronts resident on an XCD gather from ONE slice of ONE matrix
// (a few MB, L2-resident) while all tokens stream past - every row is fetched from HBM once
// and then hit ~T*k/F times in L2.  The price is that a (target, token, slice) accumulator
// cannot stay in registers across launches: it lives as an fp32 partial row that each launch
// reads, updates and writes back (skipped when the token has no survivor in the slice).
// k_decode_reduce finally adds the slices in a fixed order and applies bias / skip / rounding.
template <typename T, int NF, int TAIL, int U, bool AFFINE, bool SLICED>
// The sliced variant with up to 12 accumulators per lane (d <= 768 in bf16) needs 129 registers when left
// alone, one more than four wavefronts per SIMD allow; held to 128 it spills nothing and runs 4 % faster.
// Wider rows would spill at that limit and keep the compiler's own choice.
__global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(decode_min_waves<T, NF, TAIL, SLICED>(), 8))) void k_decode(
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col, const T *__restrict__ val,
    const T *__restrict__ wp, const float *__restrict__ bias_sum, const T *__restrict__ foff,
    const T *__restrict__ fscale, const float *__restrict__ skip_add, void *__restrict__ out,
    int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t t_begin, int64_t t_end,
    uint64_t src_mask, int out_f32, const int32_t *__restrict__ sptr, float *__restrict__ partial, int ns,
    int src, int64_t pitch) {
  constexpr int V = WVec<T>::V;
  constexpr int HV = V / 2;                       // elements per 8 bytes
  constexpr int NACC = NF * V + (TAIL == 1 ? HV : TAIL == 2 ? V : 0);
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t tok_per_blk = SLICED ? (int64_t)nwv * SLICED_NTOK : (int64_t)nwv;
  const int64_t blocks_per_t = (Tn + tok_per_blk - 1) / tok_per_blk;
  const int64_t bid = SLICED ? (int64_t)blockIdx.x / ns : (int64_t)blockIdx.x;
  const int slice = SLICED ? (int)(blockIdx.x % ns) : 0;
  // single pass: heaviest targets (most sources) first; sliced: targets in ascending order
  const int64_t t = SLICED ? t_begin + bid / blocks_per_t : t_end - 1 - bid / blocks_per_t;
  const int64_t tok = (bid % blocks_per_t) * nwv + wv;
  if (!SLICED && tok >= Tn) return;
  float acc[NACC];
#pragma unroll
  for (int j = 0; j < NACC; ++j) acc[j] = 0.0f;
  const int64_t tail_off = TAIL == 1 ? (int64_t)NF * 64 * V + (int64_t)lane * HV : (int64_t)NF * 64 * V + (int64_t)lane * V;
  const bool tail_on = TAIL == 1 ? true : (TAIL == 2 ? tail_off < d : false);

  auto gather_rows = [&](int64_t s, int32_t b, int32_t e) {
    const T *wbase = wp + decoder_slot(tying, s, t, L) * F * pitch;
    for (int32_t j0 = b; j0 < e; j0 += 64) {
      const int n = (e - j0) < 64 ? (e - j0) : 64;
      int32_t my_col = 0; float my_val = 0.0f;
      if (lane < n) {
        my_col = col[j0 + lane];
        my_val = Elem<T>::to_f32(val[j0 + lane]);
        if (AFFINE && my_val != 0.0f) {
          if (foff) my_val = Elem<T>::round(my_val + Elem<T>::to_f32(foff[t * F + my_col]));
          if (fscale) my_val = Elem<T>::round(my_val * Elem<T>::to_f32(fscale[t * F + my_col]));
        }
      }
      int i0 = 0;
      for (; i0 + U <= n; i0 += U) decode_batch<T, NF, TAIL, U>(acc, wbase, pitch, my_col, my_val, i0, n, lane, tail_off, tail_on);
      for (; i0 < n; i0 += 2) decode_batch<T, NF, TAIL, 2>(acc, wbase, pitch, my_col, my_val, i0, n, lane, tail_off, tail_on);
    }
  };

  if (SLICED) {
    // this wavefront: tokens tok*NTOK .. +NTOK-1 of source `src`, slice `slice`, target t.
    // Their slice bounds are fetched at once (one lane per token), and the survivor list of the
    // next token is requested before the current token's rows are gathered.
    const int64_t tok0 = tok * SLICED_NTOK;
    if (tok0 >= Tn) return;
    if (src < 0) {
      // All sources in one launch (decoders tied per target: every source <= t gathers from the same
      // matrix W[t], so the slice an XCD works on stays the same while the sources go by): the
      // accumulators stay in registers over the sources and the partial row is written once.
      const T *wb = wp + decoder_slot(tying, 0, t, L) * F * pitch;
      for (int i = 0; i < SLICED_NTOK; ++i) {
        if (tok0 + i >= Tn) break;
#pragma unroll
        for (int j = 0; j < NACC; ++j) acc[j] = 0.0f;
        for (int64_t s = 0; s <= t; ++s) {
          if (!((src_mask >> s) & 1ull)) continue;
          const int64_t r = s * Tn + tok0 + i;
          const int32_t b = sptr[r * (ns + 1) + slice], e = sptr[r * (ns + 1) + slice + 1];
          for (int32_t j0 = b; j0 < e; j0 += 64) {
            const int n = (e - j0) < 64 ? (e - j0) : 64;
            int32_t my_col = 0; float my_val = 0.0f;
            if (lane < n) { my_col = col[j0 + lane]; my_val = Elem<T>::to_f32(val[j0 + lane]); }
            if (AFFINE && my_val != 0.0f) {
              if (foff) my_val = Elem<T>::round(my_val + Elem<T>::to_f32(foff[t * F + my_col]));
              if (fscale) my_val = Elem<T>::round(my_val * Elem<T>::to_f32(fscale[t * F + my_col]));
            }
            decode_chunk_pipelined<T, NF, TAIL, (U > 6 ? 6 : U)>(acc, wb, pitch, my_col, my_val, n, lane, tail_off, tail_on);
          }
        }
        float *prow = partial + (((int64_t)slice * L + t) * Tn + tok0 + i) * d;
#pragma unroll
        for (int c = 0; c < NF; ++c) {
          float *pp = prow + (int64_t)c * 64 * V + (int64_t)lane * V;
#pragma unroll
          for (int j = 0; j < V; j += 4)
            stg_stream4(pp + j, make_float4(acc[c * V + j], acc[c * V + j + 1], acc[c * V + j + 2], acc[c * V + j + 3]));
        }
        if (TAIL == 1) {
#pragma unroll
          for (int j = 0; j < HV; ++j) prow[tail_off + j] = acc[NF * V + j];
        }
        if (TAIL == 2 && tail_on) {
#pragma unroll
          for (int j = 0; j < V; ++j) prow[tail_off + j] = acc[NF * V + j];
        }
      }
      return;
    }
    const uint64_t below = src_mask & ((1ull << src) - 1ull);
    const bool first = below == 0;   // the first source initialises the partial rows
    int32_t mb = 0, me = 0;
    if (lane < SLICED_NTOK && tok0 + lane < Tn) {
      const int64_t r = (int64_t)src * Tn + tok0 + lane;
      mb = sptr[r * (ns + 1) + slice];
      me = sptr[r * (ns + 1) + slice + 1];
    }
    const T *wbase = wp + decoder_slot(tying, src, t, L) * F * pitch;
    int32_t nb = __builtin_amdgcn_readlane(mb, 0), ne = __builtin_amdgcn_readlane(me, 0);
    int32_t nxt_col = 0; T nxt_val = Elem<T>::from_raw(0u);
    if (lane < ne - nb) { nxt_col = col[nb + lane]; nxt_val = val[nb + lane]; }
#pragma unroll
    for (int i = 0; i < SLICED_NTOK; ++i) {
      const int32_t b = nb, e = ne;
      const int32_t cur_col = nxt_col; const T cur_val = nxt_val;
      if (i + 1 < SLICED_NTOK) {
        nb = __builtin_amdgcn_readlane(mb, i + 1); ne = __builtin_amdgcn_readlane(me, i + 1);
        nxt_col = 0; nxt_val = Elem<T>::from_raw(0u);
        if (lane < ne - nb) { nxt_col = col[nb + lane]; nxt_val = val[nb + lane]; }
      }
      if (tok0 + i >= Tn) break;
      if (b == e && !first) continue;
      float *prow = partial + (((int64_t)slice * L + t) * Tn + tok0 + i) * d;
      float old[NACC];
#pragma unroll
      for (int j = 0; j < NACC; ++j) { old[j] = 0.0f; acc[j] = 0.0f; }
      if (!first) {   // requested before the gathers so that its latency hides behind them
#pragma unroll
        for (int c = 0; c < NF; ++c) {
          const float *pp = prow + (int64_t)c * 64 * V + (int64_t)lane * V;
#pragma unroll
          for (int j = 0; j < V; j += 4) {
            float4 q = ldg_stream4(pp + j);
            old[c * V + j] = q.x; old[c * V + j + 1] = q.y; old[c * V + j + 2] = q.z; old[c * V + j + 3] = q.w;
          }
        }
        if (TAIL == 1) {
#pragma unroll
          for (int j = 0; j < HV; ++j) old[NF * V + j] = prow[tail_off + j];
        }
        if (TAIL == 2 && tail_on) {
#pragma unroll
          for (int j = 0; j < V; ++j) old[NF * V + j] = prow[tail_off + j];
        }
      }
      for (int32_t j0 = b; j0 < e; j0 += 64) {
        const int n = (e - j0) < 64 ? (e - j0) : 64;
        int32_t my_col = cur_col; float my_val = Elem<T>::to_f32(cur_val);
        if (j0 > b) {   // more than 64 survivors in this slice: fetch the next 64
          my_col = 0; my_val = 0.0f;
          if (lane < n) { my_col = col[j0 + lane]; my_val = Elem<T>::to_f32(val[j0 + lane]); }
        }
        if (AFFINE && my_val != 0.0f) {
          if (foff) my_val = Elem<T>::round(my_val + Elem<T>::to_f32(foff[t * F + my_col]));
          if (fscale) my_val = Elem<T>::round(my_val * Elem<T>::to_f32(fscale[t * F + my_col]));
        }
        decode_chunk_pipelined<T, NF, TAIL, (U > 6 ? 6 : U)>(acc, wbase, pitch, my_col, my_val, n, lane, tail_off, tail_on);
      }
#pragma unroll
      for (int c = 0; c < NF; ++c) {
        float *pp = prow + (int64_t)c * 64 * V + (int64_t)lane * V;
#pragma unroll
        for (int j = 0; j < V; j += 4)
          stg_stream4(pp + j, make_float4(old[c * V + j] + acc[c * V + j], old[c * V + j + 1] + acc[c * V + j + 1],
                                          old[c * V + j + 2] + acc[c * V + j + 2], old[c * V + j + 3] + acc[c * V + j + 3]));
      }
      if (TAIL == 1) {
#pragma unroll
        for (int j = 0; j < HV; ++j) prow[tail_off + j] = old[NF * V + j] + acc[NF * V + j];
      }
      if (TAIL == 2 && tail_on) {
#pragma unroll
        for (int j = 0; j < V; ++j) prow[tail_off + j] = old[NF * V + j] + acc[NF * V + j];
      }
    }
    return;
  }

  for (int64_t s = 0; s <= t; ++s) {
    if (!((src_mask >> s) & 1ull)) continue;
    const int64_t r = s * Tn + tok;
    gather_rows(s, row_ptr[r], row_ptr[r + 1]);
  }
  // epilogue: bias, skip term, one write of the output row
  auto emit = [&](int64_t o, const float *a, int cnt, bool on) {
    if (!on) return;
    for (int j = 0; j < cnt; ++j) {
      float y = a[j];
      if (bias_sum) y += bias_sum[t * d + o + j];
      if (skip_add) y += skip_add[(t * Tn + tok) * d + o + j];
      if (out_f32) ((float *)out)[(t * Tn + tok) * d + o + j] = y;
      else ((T *)out)[(t * Tn + tok) * d + o + j] = Elem<T>::from_f32(y);
    }
  };
#pragma unroll
  for (int c = 0; c < NF; ++c) emit((int64_t)c * 64 * V + (int64_t)lane * V, acc + c * V, V, true);
  if (TAIL == 1) emit(tail_off, acc + NF * V, HV, true);
  if (TAIL == 2) emit(tail_off, acc + NF * V, V, tail_on);
}

// How the units (slice, column part) of one target are dealt to the 8 XCDs: `full` rounds in which XCD x
// takes unit round * 8 + x over all tokens, then the `rem` units that are left over, with the tokens of each
// split between q XCDs so that all eight stay busy (rem divides 8: one round, q = 8 / rem; otherwise `rem`
// rounds in which all XCDs share one unit, q = 8).  Blocks go to the XCDs round-robin, so block b runs on
// XCD b % 8; within an XCD the blocks are ordered target, round, token block: an XCD finishes one part of
// one decoder matrix before it touches the next.
struct UnitPlan {
  int ns, ncp, full, rem, q;
  int bf, br;            // blocks per XCD in a full round / in a remainder round
  int64_t tpp;           // tokens per XCD in a remainder round
  int bpx;               // blocks per XCD and target
};

static UnitPlan make_unit_plan(int ns, int ncp, int64_t Tn, int tok_per_block) {
  UnitPlan up;
  up.ns = ns; up.ncp = ncp;
  const int units = ns * ncp;
  up.full = units / 8; up.rem = units % 8;
  up.q = up.rem == 0 ? 1 : (8 % up.rem == 0 ? 8 / up.rem : 8);
  const int rem_rounds = up.rem == 0 ? 0 : (8 % up.rem == 0 ? 1 : up.rem);
  up.tpp = clt_ceil_div(Tn, up.q);
  up.bf = (int)clt_ceil_div(Tn, tok_per_block);
  up.br = (int)clt_ceil_div(up.tpp, tok_per_block);
  up.bpx = up.full * up.bf + rem_rounds * up.br;
  return up;
}

// this block's work: target index (relative), unit -> (slice, column part), its token range and its token block
struct UnitWork { int64_t target; int slice, cpart; int64_t tok_begin, tok_end; int tb; };
__device__ __forceinline__ UnitWork unit_work(const UnitPlan &up, int64_t Tn) {
  UnitWork w;
  const int xcd = (int)(blockIdx.x & 7);
  const int64_t i = (int64_t)(blockIdx.x >> 3);
  w.target = i / up.bpx;
  const int j = (int)(i % up.bpx);
  int unit;
  w.tok_begin = 0; w.tok_end = Tn;
  if (j < up.full * up.bf) {
    unit = (j / up.bf) * 8 + xcd; w.tb = j % up.bf;
  } else {
    const int jr = j - up.full * up.bf, rr = jr / up.br;
    w.tb = jr % up.br;
    int tpart;
    if (up.q * up.rem == 8) { unit = up.full * 8 + xcd / up.q; tpart = xcd % up.q; }
    else { unit = up.full * 8 + rr; tpart = xcd; }
    w.tok_begin = (int64_t)tpart * up.tpp;
    w.tok_end = w.tok_begin + up.tpp < Tn ? w.tok_begin + up.tpp : Tn;
  }
  w.cpart = unit % up.ncp; w.slice = unit / up.ncp;
  return w;
}

// ---- quarter-row schedule -------------------------------------------------------------------------
// Large batches, untied or per-source decoders, d a multiple of 256: the feature axis is cut into 2
// slices and the columns into 4 quarters; workgroup b works on part b % 8 = (slice, quarter), so an XCD
// still gathers from one 1/8 of one decoder matrix at a time (F/2 rows x d/4 columns) but a (target,
// token) has 2 partial rows instead of 8: a quarter of the fp32 read-modify-write traffic between source
// launches.  So that a quarter row (384 bytes at d = 768, three whole cache lines) costs no more
// instructions than its share of a whole one, a wavefront fetches FOUR rows per load: each group of
// QLANES = 16 lanes takes one survivor's quarter row, 16 (+8) bytes per lane; every group accumulates
// its own rows and the four groups are added once per token.
constexpr int QLANES = 16;              // lanes per quarter row
constexpr int QROWS = 64 / QLANES;      // rows per load
constexpr int QUARTER_SLICES = 2;       // feature slices; 8 / QUARTER_SLICES column parts
constexpr int QUARTER_PARTS = 8 / QUARTER_SLICES;
template <typename T, int HQ, int HTAIL, int UU, bool PACK> struct PartBatch {
  uint4 wq[UU][HQ > 0 ? HQ : 1];
  uint2 wt8[UU];
  float v[UU];          // !PACK: the activation values
  uint32_t pk[UU];      // PACK: feature index | bf16 value << 16
  // slot QROWS * u + g of the (up to 64) survivors held one per lane goes to lane group g.  Lanes past the
  // end of the list hold feature 0 with value 0: a repeated fetch with weight 0, so nothing is clamped.
  // PACK (bf16, F <= 65536): one cross-lane move per row, and the row offset is a 24-bit multiply-add.
  __device__ __forceinline__ void load(const T *wbase, int64_t d, uint32_t my_pk, int32_t my_col, float my_val, int i0, int n,
                                       int ll, int grp) {
    constexpr int V = WVec<T>::V;
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      const int idx = i0 + QROWS * u + grp;
      if constexpr (PACK) {
        pk[u] = (uint32_t)__builtin_amdgcn_ds_bpermute(idx << 2, (int)my_pk);
        const uint32_t off = __umul24(pk[u] & 0xFFFFu, (uint32_t)d * (uint32_t)sizeof(T)) + (uint32_t)(ll * 16);
        const char *wrow = reinterpret_cast<const char *>(wbase) + off;
#pragma unroll
        for (int c = 0; c < HQ; ++c) wq[u][c] = *reinterpret_cast<const uint4 *>(wrow + c * QLANES * 16);
        if (HTAIL) wt8[u] = *reinterpret_cast<const uint2 *>(wrow + HQ * QLANES * 16 - ll * 8);
      } else {
        const int ci = idx < n ? idx : n - 1;                 // clamp: a repeated fetch, weight 0
        const int32_t f = __shfl(my_col, ci);
        const float vv = __shfl(my_val, ci);
        v[u] = idx < n ? vv : 0.0f;
        const T *wrow = wbase + (int64_t)f * d;
#pragma unroll
        for (int c = 0; c < HQ; ++c) wq[u][c] = *reinterpret_cast<const uint4 *>(wrow + c * QLANES * V + ll * V);
        if (HTAIL) wt8[u] = *reinterpret_cast<const uint2 *>(wrow + HQ * QLANES * V + ll * (V / 2));
      }
    }
  }
  __device__ __forceinline__ uint32_t value_pair(int u) const {
    if constexpr (PACK) return __builtin_amdgcn_perm(pk[u + 1], pk[u], 0x07060302u);   // (value u, value u + 1)
    else return raw16_of<T>(v[u]) | (raw16_of<T>(v[u + 1]) << 16);
  }
  __device__ __forceinline__ void consume(float *acc) const {
    constexpr int V = WVec<T>::V;
    if constexpr (sizeof(T) == 2 && (UU % 2) == 0) {
#pragma unroll
      for (int u = 0; u < UU; u += 2) {
        const uint32_t vv = value_pair(u);
#pragma unroll
        for (int c = 0; c < HQ; ++c) WVec<T>::dot16(acc + c * V, wq[u][c], wq[u + 1][c], vv);
        if (HTAIL) WVec<T>::dot8(acc + HQ * V, wt8[u], wt8[u + 1], vv);
      }
    } else {
#pragma unroll
      for (int u = 0; u < UU; ++u) {
#pragma unroll
        for (int c = 0; c < HQ; ++c) WVec<T>::fma16(acc + c * V, wq[u][c], v[u]);
        if (HTAIL) WVec<T>::fma8(acc + HQ * V, wt8[u], v[u]);
      }
    }
  }
};

constexpr int QUARTER_NTOK = 2;     // tokens per wavefront
// 12 accumulators per lane (d = 768): 72 registers, seven wavefronts per SIMD; wider rows are left alone
template <typename T, int HQ, int HTAIL> constexpr int quarter_min_waves() {
  constexpr int V = 16 / (int)sizeof(T);
  return (sizeof(T) == 2 && HQ * V + (HTAIL ? V / 2 : 0) <= 12) ? 7 : 1;   // fp32 at 7 would spill
}

template <typename T, int HQ, int HTAIL, int UU, bool AFFINE, bool PACK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(quarter_min_waves<T, HQ, HTAIL>(), 8))) void k_decode_quarter(
    const int32_t *__restrict__ col, const T *__restrict__ val, const T *__restrict__ wp, const T *__restrict__ foff,
    const T *__restrict__ fscale, int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t t_begin, uint64_t src_mask,
    const int32_t *__restrict__ sptr, float *__restrict__ partial, int src, int64_t pitch, UnitPlan up) {
  constexpr int V = WVec<T>::V;
  constexpr int NACC = HQ * V + (HTAIL ? V / 2 : 0);      // columns per lane: d / 64
  constexpr int NCP = QUARTER_PARTS;
  const int ns = up.ns;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int ll = lane & (QLANES - 1), grp = lane / QLANES;
  const bool hi = grp != 0;                    // only the first lane group touches the partial row
  const UnitWork uw = unit_work(up, Tn);
  const int slice = uw.slice, cpart = uw.cpart;
  const int64_t t = t_begin + uw.target;
  const int64_t tok_end = uw.tok_end;
  const int64_t tok0 = uw.tok_begin + ((int64_t)uw.tb * nwv + wv) * QUARTER_NTOK;
  if (tok0 >= tok_end) return;
  const uint64_t below = src_mask & ((1ull << src) - 1ull);
  const bool first = below == 0;   // the first source initialises the partial rows
  int32_t mb = 0, me = 0;
  if (lane < QUARTER_NTOK && tok0 + lane < tok_end) {
    const int64_t r = (int64_t)src * Tn + tok0 + lane;
    mb = sptr[r * (ns + 1) + slice];
    me = sptr[r * (ns + 1) + slice + 1];
  }
  const T *wbase = wp + decoder_slot(tying, src, t, L) * F * pitch + (int64_t)cpart * (d / NCP);
  int32_t nb = __builtin_amdgcn_readlane(mb, 0), ne = __builtin_amdgcn_readlane(me, 0);
  int32_t nxt_col = 0; T nxt_val = Elem<T>::from_raw(0u);
  if (lane < ne - nb) { nxt_col = col[nb + lane]; nxt_val = val[nb + lane]; }
#pragma unroll
  for (int i = 0; i < QUARTER_NTOK; ++i) {
    const int32_t b = nb, e = ne;
    const int32_t cur_col = nxt_col; const T cur_val = nxt_val;
    if (i + 1 < QUARTER_NTOK) {
      nb = __builtin_amdgcn_readlane(mb, i + 1); ne = __builtin_amdgcn_readlane(me, i + 1);
      nxt_col = 0; nxt_val = Elem<T>::from_raw(0u);
      if (lane < ne - nb) { nxt_col = col[nb + lane]; nxt_val = val[nb + lane]; }
    }
    if (tok0 + i >= tok_end) break;
    if (b == e && !first) continue;
    // this lane's columns of the partial row (the first lane group writes it): pieces of V, then the tail
    float *prow = partial + (((int64_t)slice * L + t) * Tn + tok0 + i) * d + (int64_t)cpart * (d / NCP);
    float old[NACC], acc[NACC];
#pragma unroll
    for (int j = 0; j < NACC; ++j) { old[j] = 0.0f; acc[j] = 0.0f; }
    for (int32_t j0 = b; j0 < e; j0 += 64) {
      const int n = (e - j0) < 64 ? (e - j0) : 64;
      int32_t my_col = cur_col; float my_val = Elem<T>::to_f32(cur_val);
      if (j0 > b) {   // more than 64 survivors in this slice: fetch the next 64
        my_col = 0; my_val = 0.0f;
        if (lane < n) { my_col = col[j0 + lane]; my_val = Elem<T>::to_f32(val[j0 + lane]); }
      }
      if (AFFINE && my_val != 0.0f) {
        if (foff) my_val = Elem<T>::round(my_val + Elem<T>::to_f32(foff[t * F + my_col]));
        if (fscale) my_val = Elem<T>::round(my_val * Elem<T>::to_f32(fscale[t * F + my_col]));
      }
      // two batches of UU row pairs in flight
      const uint32_t my_pk = PACK ? ((uint32_t)my_col | (raw16_of<T>(my_val) << 16)) : 0u;
      PartBatch<T, HQ, HTAIL, UU, PACK> ra, rb;
      constexpr int R = QROWS;
      ra.load(wbase, pitch, my_pk, my_col, my_val, 0, n, ll, grp);
      for (int i0 = 0; i0 < n; i0 += 2 * R * UU) {
        if (i0 + R * UU < n) rb.load(wbase, pitch, my_pk, my_col, my_val, i0 + R * UU, n, ll, grp);
        ra.consume(acc);
        if (i0 + R * UU < n) {
          if (i0 + 2 * R * UU < n) ra.load(wbase, pitch, my_pk, my_col, my_val, i0 + 2 * R * UU, n, ll, grp);
          rb.consume(acc);
        }
      }
    }
    // The old partial row is asked for only now: held across the gathers it would cost 12 registers and
    // one wavefront per SIMD, and the other wavefronts cover its latency better than an early request.
    if (!first && !hi) {
#pragma unroll
      for (int c = 0; c < HQ; ++c) {
#pragma unroll
        for (int j = 0; j < V; j += 4) {
          const float4 q = ldg_stream4(prow + c * QLANES * V + ll * V + j);
          old[c * V + j] = q.x; old[c * V + j + 1] = q.y; old[c * V + j + 2] = q.z; old[c * V + j + 3] = q.w;
        }
      }
      if (HTAIL) {
        if constexpr (V / 2 == 4) {
          const float4 q = ldg_stream4(prow + HQ * QLANES * V + ll * 4);
          old[HQ * V] = q.x; old[HQ * V + 1] = q.y; old[HQ * V + 2] = q.z; old[HQ * V + 3] = q.w;
        } else {
#pragma unroll
          for (int j = 0; j < V / 2; ++j) old[HQ * V + j] = prow[HQ * QLANES * V + ll * (V / 2) + j];
        }
      }
    }
    // the lane groups hold sums over different survivors: add them, in a fixed order (group 0 ends up
    // with ((g0 + g1) + (g2 + g3)))
#pragma unroll
    for (int j = 0; j < NACC; ++j) {
      const float o16 = __shfl_xor(acc[j], 16);
      acc[j] = (lane & 16) ? o16 + acc[j] : acc[j] + o16;
      const float o32 = __shfl_xor(acc[j], 32);
      acc[j] = (lane & 32) ? o32 + acc[j] : acc[j] + o32;
    }
    if (!hi) {
#pragma unroll
      for (int c = 0; c < HQ; ++c) {
#pragma unroll
        for (int j = 0; j < V; j += 4)
          stg_stream4(prow + c * QLANES * V + ll * V + j,
                      make_float4(old[c * V + j] + acc[c * V + j], old[c * V + j + 1] + acc[c * V + j + 1],
                                  old[c * V + j + 2] + acc[c * V + j + 2], old[c * V + j + 3] + acc[c * V + j + 3]));
      }
      if (HTAIL) {
        if constexpr (V / 2 == 4) {
          stg_stream4(prow + HQ * QLANES * V + ll * 4, make_float4(old[HQ * V] + acc[HQ * V], old[HQ * V + 1] + acc[HQ * V + 1],
                                                               old[HQ * V + 2] + acc[HQ * V + 2], old[HQ * V + 3] + acc[HQ * V + 3]));
        } else {
#pragma unroll
          for (int j = 0; j < V / 2; ++j) prow[HQ * QLANES * V + ll * (V / 2) + j] = old[HQ * V + j] + acc[HQ * V + j];
        }
      }
    }
  }
}

// ---- line schedule ---------------------------------------------------------------------------------
// Large batches, untied or per-source decoders, rows that are whole 128-byte cache lines: the COLUMNS are
// cut into parts of exactly one cache line (64 bf16 / 32 fp32), so the piece of a decoder matrix that an
// XCD gathers from while all tokens stream past is F x 128 bytes (3.0 MiB at F = 24576, inside its 4 MiB
// L2; wider feature axes are cut into `ns` slices to stay there).  The units of work (slice, column part,
// token part) are dealt to the XCDs in rounds - unit u runs on XCD u % 8 in round u / 8 - and the token
// axis is cut into `ntp` parts only to make their number a multiple of 8.  A load instruction fetches the
// line of EIGHT survivors (8 lanes x 16 bytes each); every lane group accumulates its own survivors and a
// butterfly that halves the accumulators at every step (reduce-scatter: 7 shuffles for 8 accumulators)
// leaves each lane with the finished sum of one column.  With ns = 1 a (target, token) has one fp32
// partial row, read and written once per source layer.
constexpr int LINE_UU = 2;                // loads per batch (two batches in flight)
constexpr int64_t LINE_L2_BYTES = 3407872;   // 3.25 MiB: the part of a matrix one XCD works on stays below this

template <typename T, int UU, bool PACK> struct LineBatch {
  uint4 wq[UU];
  float v[UU];          // !PACK: the activation values
  uint32_t pk[UU];      // PACK: feature index | bf16 value << 16
  // entry 8 * u + grp of the (up to 64) survivors held one per lane goes to lane group grp; lanes past the
  // end of the list hold feature 0 with value 0 (a repeated fetch, weight 0)
  __device__ __forceinline__ void load(const T *wbase, int64_t rstride, uint32_t my_pk, int32_t my_col, float my_val, int i0,
                                       int n, int ll, int grp) {
    constexpr int V = WVec<T>::V;
#pragma unroll
    for (int u = 0; u < UU; ++u) {
      const int idx = i0 + 8 * u + grp;
      if constexpr (PACK) {
        pk[u] = (uint32_t)__builtin_amdgcn_ds_bpermute(idx << 2, (int)my_pk);
        const uint32_t off = __umul24(pk[u] & 0xFFFFu, (uint32_t)rstride * (uint32_t)sizeof(T)) + (uint32_t)(ll * 16);
        wq[u] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(wbase) + off);
      } else {
        const int ci = idx < n ? idx : n - 1;
        const int32_t f = __shfl(my_col, ci);
        const float vv = __shfl(my_val, ci);
        v[u] = idx < n ? vv : 0.0f;
        wq[u] = *reinterpret_cast<const uint4 *>(wbase + (int64_t)f * rstride + ll * V);
      }
    }
  }
  __device__ __forceinline__ void consume(float *acc) const {
    if constexpr (sizeof(T) == 2 && (UU % 2) == 0) {
#pragma unroll
      for (int u = 0; u < UU; u += 2) {
        uint32_t vb;
        if constexpr (PACK) vb = __builtin_amdgcn_perm(pk[u + 1], pk[u], 0x07060302u);
        else vb = raw16_of<T>(v[u]) | (raw16_of<T>(v[u + 1]) << 16);
        WVec<T>::dot16(acc, wq[u], wq[u + 1], vb);
      }
    } else {
#pragma unroll
      for (int u = 0; u < UU; ++u) WVec<T>::fma16(acc, wq[u], v[u]);
    }
  }
};

template <typename T, bool AFFINE, bool PACK, int NTOK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(8, 8))) void k_decode_line(
    const int32_t *__restrict__ col, const T *__restrict__ val, const T *__restrict__ wp, const T *__restrict__ foff,
    const T *__restrict__ fscale, int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t t_begin, uint64_t src_mask,
    const int32_t *__restrict__ sptr, float *__restrict__ partial, int src, UnitPlan lp, int64_t pitch) {
  constexpr int V = WVec<T>::V;                     // elements per lane: 16 bytes
  constexpr int LW = 8 * V;                         // columns per part: one 128-byte line
  constexpr int LINE_NTOK = NTOK;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int ll = lane & 7, grp = lane >> 3;
  const int ns = lp.ns;
  const UnitWork uw = unit_work(lp, Tn);
  const int64_t t = t_begin + uw.target;
  const int cpart = uw.cpart, slice = uw.slice;
  const int64_t part_end = uw.tok_end;
  const int64_t tok0 = uw.tok_begin + ((int64_t)uw.tb * nwv + wv) * LINE_NTOK;
  if (tok0 >= part_end) return;
  const uint64_t below = src_mask & ((1ull << src) - 1ull);
  const bool first = below == 0;   // the first source initialises the partial rows
  int32_t mb = 0, me = 0;
  if (lane < LINE_NTOK && tok0 + lane < part_end) {
    const int64_t r = (int64_t)src * Tn + tok0 + lane;
    mb = sptr[r * (ns + 1) + slice];
    me = sptr[r * (ns + 1) + slice + 1];
  }
  const T *wbase = wp + decoder_slot(tying, src, t, L) * F * pitch + (int64_t)cpart * LW;
  int32_t nb = __builtin_amdgcn_readlane(mb, 0), ne = __builtin_amdgcn_readlane(me, 0);
  int32_t nxt_col = 0; T nxt_val = Elem<T>::from_raw(0u);
  if (lane < ne - nb) { nxt_col = col[nb + lane]; nxt_val = val[nb + lane]; }
#pragma unroll
  for (int it = 0; it < LINE_NTOK; ++it) {
    const int32_t b = nb, e = ne;
    const int32_t cur_col = nxt_col; const T cur_val = nxt_val;
    if (it + 1 < LINE_NTOK) {
      nb = __builtin_amdgcn_readlane(mb, it + 1); ne = __builtin_amdgcn_readlane(me, it + 1);
      nxt_col = 0; nxt_val = Elem<T>::from_raw(0u);
      if (lane < ne - nb) { nxt_col = col[nb + lane]; nxt_val = val[nb + lane]; }
    }
    if (tok0 + it >= part_end) break;
    if (b == e && !first) continue;
    float acc[V];
#pragma unroll
    for (int j = 0; j < V; ++j) acc[j] = 0.0f;
    LineBatch<T, LINE_UU, PACK> ra, rb;
    for (int32_t j0 = b; j0 < e; j0 += 64) {
      const int n = (e - j0) < 64 ? (e - j0) : 64;
      int32_t my_col = cur_col; float my_val = Elem<T>::to_f32(cur_val);
      if (j0 > b) {   // more than 64 survivors in this slice: fetch the next 64
        my_col = 0; my_val = 0.0f;
        if (lane < n) { my_col = col[j0 + lane]; my_val = Elem<T>::to_f32(val[j0 + lane]); }
      }
      if (AFFINE && my_val != 0.0f) {
        if (foff) my_val = Elem<T>::round(my_val + Elem<T>::to_f32(foff[t * F + my_col]));
        if (fscale) my_val = Elem<T>::round(my_val * Elem<T>::to_f32(fscale[t * F + my_col]));
      }
      // bf16: feature index (< 65536) and value travel to their lane group in one 32-bit word
      const uint32_t my_pk = PACK ? ((uint32_t)my_col | (raw16_of<T>(my_val) << 16)) : 0u;
      constexpr int R = 8 * LINE_UU;                 // survivors per batch
      ra.load(wbase, pitch, my_pk, my_col, my_val, 0, n, ll, grp);
      for (int i0 = 0; i0 < n; i0 += 2 * R) {
        if (i0 + R < n) rb.load(wbase, pitch, my_pk, my_col, my_val, i0 + R, n, ll, grp);
        ra.consume(acc);
        if (i0 + R < n) {
          if (i0 + 2 * R < n) ra.load(wbase, pitch, my_pk, my_col, my_val, i0 + 2 * R, n, ll, grp);
          rb.consume(acc);
        }
      }
    }
    // reduce-scatter over the eight lane groups (fixed order): every step hands half of the accumulators to
    // the partner group and adds the half that comes back, so a lane ends with the sum of ONE column
    float r; int csel; bool writer = true;
    if constexpr (V == 8) {
      float a4[4], a2[2];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float keep = (grp & 4) ? acc[j + 4] : acc[j], send = (grp & 4) ? acc[j] : acc[j + 4];
        a4[j] = keep + __shfl_xor(send, 32);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float keep = (grp & 2) ? a4[j + 2] : a4[j], send = (grp & 2) ? a4[j] : a4[j + 2];
        a2[j] = keep + __shfl_xor(send, 16);
      }
      const float keep = (grp & 1) ? a2[1] : a2[0], send = (grp & 1) ? a2[0] : a2[1];
      r = keep + __shfl_xor(send, 8);
      csel = ll * 8 + grp;
    } else {
      float a2[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float keep = (grp & 4) ? acc[j + 2] : acc[j], send = (grp & 4) ? acc[j] : acc[j + 2];
        a2[j] = keep + __shfl_xor(send, 32);
      }
      const float keep = (grp & 2) ? a2[1] : a2[0], send = (grp & 2) ? a2[0] : a2[1];
      const float a1 = keep + __shfl_xor(send, 16);
      const float o = __shfl_xor(a1, 8);
      r = (grp & 1) ? o + a1 : a1 + o;             // both lanes of a pair form the same sum
      csel = ll * 4 + ((grp >> 2) & 1) * 2 + ((grp >> 1) & 1);
      writer = (grp & 1) == 0;
    }
    float *pp = partial + (((int64_t)slice * L + t) * Tn + tok0 + it) * d + (int64_t)cpart * LW + csel;
    if (writer) {
      const float old = first ? 0.0f : __builtin_nontemporal_load(pp);
      __builtin_nontemporal_store(old + r, pp);
    }
  }
}

// sptr[r][j] = first survivor of row r whose feature index is >= j * F / ns  (j = 0..ns)
__global__ void k_slice_ptr(const int32_t *row_ptr, const int32_t *col, int64_t R, int64_t F, int ns, int32_t *sptr) {
  const int64_t total = R * (ns + 1);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / (ns + 1);
    const int j = (int)(i - r * (ns + 1));
    const int32_t bound = (int32_t)(((int64_t)j * F) / ns);
    int32_t lo = row_ptr[r], hi = row_ptr[r + 1];
    while (lo < hi) {
      int32_t mid = lo + ((hi - lo) >> 1);
      if (col[mid] < bound) lo = mid + 1; else hi = mid;
    }
    sptr[i] = lo;
  }
}

// out[t][tok][:] = sum over slices (fixed order) + bias + skip, rounded once.  4 elements per thread.
template <typename T>
__global__ void k_decode_reduce(const float *__restrict__ partial, const float *__restrict__ bias_sum,
                                const float *__restrict__ skip_add, void *__restrict__ out, int64_t Tn, int64_t d,
                                int64_t L, int64_t t_begin, int64_t t_end, int ns, int out_f32, uint64_t src_mask) {
  const int64_t per_t = Tn * d, span = (t_end - t_begin) * per_t, slice_stride = L * per_t;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < span; i += (int64_t)gridDim.x * blockDim.x * 4) {
    const int64_t g = t_begin * per_t + i;          // index into [L][T][d]
    const int64_t t = g / per_t, o = g % d;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    if (src_mask & ((2ull << t) - 1ull)) {            // some source <= t wrote partial rows
      a = *reinterpret_cast<const float4 *>(partial + g);
      for (int sl = 1; sl < ns; ++sl) {
        float4 b = *reinterpret_cast<const float4 *>(partial + sl * slice_stride + g);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
      }
    }
    if (bias_sum) { a.x += bias_sum[t * d + o]; a.y += bias_sum[t * d + o + 1]; a.z += bias_sum[t * d + o + 2]; a.w += bias_sum[t * d + o + 3]; }
    if (skip_add) { float4 k = *reinterpret_cast<const float4 *>(skip_add + g); a.x += k.x; a.y += k.y; a.z += k.z; a.w += k.w; }
    if (out_f32) *reinterpret_cast<float4 *>((float *)out + g) = a;
    else if (sizeof(T) == 4) *reinterpret_cast<float4 *>((float *)out + g) = a;
    else {
      uint2 o2;
      o2.x = pack_pair<T>(a.x, a.y);
      o2.y = pack_pair<T>(a.z, a.w);
      *reinterpret_cast<uint2 *>((bf16_t *)out + g) = o2;
    }
  }
}

// Any d (no alignment assumption): lanes stride over the output row one element at a time.
template <typename T>
__global__ __launch_bounds__(256) void k_decode_generic(
    const int32_t *row_ptr, const int32_t *col, const T *val, const T *wp, const float *bias_sum,
    const T *foff, const T *fscale, const float *skip_add, void *out, int64_t Tn, int64_t d,
    int64_t F, int64_t L, int tying, int64_t t_begin, int64_t t_end, uint64_t src_mask, int out_f32, int64_t pitch) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t blocks_per_t = (Tn + nwv - 1) / nwv;
  const int64_t t = t_end - 1 - (int64_t)blockIdx.x / blocks_per_t;
  const int64_t tok = ((int64_t)blockIdx.x % blocks_per_t) * nwv + wv;
  if (tok >= Tn) return;
  for (int64_t o0 = 0; o0 < d; o0 += 64) {
    const int64_t o = o0 + lane;
    float acc = 0.0f;
    for (int64_t s = 0; s <= t; ++s) {
      if (!((src_mask >> s) & 1ull)) continue;
      const int64_t r = s * Tn + tok;
      const T *wbase = wp + decoder_slot(tying, s, t, L) * F * pitch;
      for (int32_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
        const int32_t f = col[j];
        float v = Elem<T>::to_f32(val[j]);
        if (v != 0.0f) {
          if (foff) v = Elem<T>::round(v + Elem<T>::to_f32(foff[t * F + f]));
          if (fscale) v = Elem<T>::round(v * Elem<T>::to_f32(fscale[t * F + f]));
        }
        if (o < d) acc = fmaf(v, Elem<T>::to_f32(wbase[(int64_t)f * pitch + o]), acc);
      }
    }
    if (o < d) {
      if (bias_sum) acc += bias_sum[t * d + o];
      if (skip_add) acc += skip_add[(t * Tn + tok) * d + o];
      if (out_f32) ((float *)out)[(t * Tn + tok) * d + o] = acc;
      else ((T *)out)[(t * Tn + tok) * d + o] = Elem<T>::from_f32(acc);
    }
  }
}

// [d][F] -> [F][d] through a 64x64 LDS tile (coalesced on both sides).
template <typename T>
__global__ __launch_bounds__(256) void k_pack(const T *src, T *dst, int64_t d, int64_t F,
                                              int64_t in_stride, int64_t out_stride, int64_t pitch) {
  __shared__ T tile[64][65];
  const T *s = src + (int64_t)blockIdx.z * in_stride;
  T *o = dst + (int64_t)blockIdx.z * out_stride;
  const int64_t f0 = (int64_t)blockIdx.x * 64, d0 = (int64_t)blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    int64_t dd = d0 + i, ff = f0 + tx;
    if (dd < d && ff < F) tile[i][tx] = s[dd * F + ff];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    int64_t ff = f0 + i, dd = d0 + tx;
    if (ff < F && dd < d) o[ff * pitch + dd] = tile[tx][i];
  }
}

// The same for the matrices whose flag is set, addressed through a table of parameter pointers: FP_PACK_BLOCKS
// workgroups per matrix walk its 64 x 64 tiles; a matrix whose flag is clear costs its workgroups one load.
constexpr int FP_PACK_BLOCKS = 64;
template <typename T>
__global__ __launch_bounds__(256) void k_pack_if(T *const *w_refs, T *dst, int64_t d, int64_t F, int64_t pitch,
                                                 const int32_t *changed) {
  __shared__ T tile[64][65];
  const int z = blockIdx.y;
  if (changed[z] == 0) return;
  const T *s = w_refs[z];
  T *o = dst + (int64_t)z * F * pitch;
  const int64_t tf = (F + 63) / 64, td = (d + 63) / 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int64_t tile_i = blockIdx.x; tile_i < tf * td; tile_i += gridDim.x) {
    const int64_t f0 = (tile_i % tf) * 64, d0 = (tile_i / tf) * 64;
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
      int64_t dd = d0 + i, ff = f0 + tx;
      if (dd < d && ff < F) tile[i][tx] = s[dd * F + ff];
    }
    __syncthreads();
    for (int i = ty; i < 64; i += 4) {
      int64_t ff = f0 + i, dd = d0 + tx;
      if (ff < F && dd < d) o[ff * pitch + dd] = tile[tx][i];
    }
  }
}

// Fingerprint of every decoder parameter [d][F]: a sum (order-free, so the workgroups of a matrix add to it with
// atomics) of mixed 32-bit words from sampled runs of 64 words.  A matrix of up to FP_CHUNKS runs is taken whole.
// A larger one gives one run per row, on a diagonal: row r gives run (61 r + r / runs_per_row) mod runs_per_row, so
// every row is looked at and every column in d / runs_per_row rows - a write to a whole row, a whole column or the
// whole matrix cannot be missed, and the sample is d x 256 bytes (0.5 % of a 768 x 24576 matrix).  Rows that are not
// a whole number of words fall back to FP_CHUNKS evenly spread runs.
// FP_BLOCKS workgroups per matrix (a CU keeps only ~64 line requests in flight, so a matrix's rows are spread over
// several CUs).  state holds one 128-byte line per matrix - FP_BLOCKS partial sums, the stored fingerprint and an
// arrival counter - so that the workgroups of different matrices never meet on a cache line; the last workgroup of
// a matrix to arrive adds the partial sums, compares, stores and leaves the counter at zero.
constexpr int FP_BLOCKS = 8;
constexpr int FP_STATE_WORDS = 16;
constexpr int FP_CHUNKS = 4096;
__device__ __forceinline__ unsigned long long fp_mix(uint32_t word, uint32_t index) {
  unsigned long long h = ((unsigned long long)word << 32) | (unsigned long long)(index * 0x9E3779B1u + 0x7F4A7C15u);
  h ^= h >> 29; h *= 0xBF58476D1CE4E5B9ull; h ^= h >> 32; h *= 0x94D049BB133111EBull; h ^= h >> 29;
  return h;
}
__global__ __launch_bounds__(256) void k_fingerprint(const uint32_t *const *w_refs, int64_t words, int64_t rows,
                                                     int64_t words_per_row, unsigned long long *state,
                                                     int32_t *changed, int store_only) {
  __shared__ unsigned long long red[4];
  const int z = blockIdx.y, lane = lane_id(), wv = threadIdx.x >> 6;
  const uint32_t *w = w_refs[z];
  const int64_t n_chunks = (words + 63) / 64;
  const int64_t rpr = words_per_row > 0 ? (words_per_row + 63) / 64 : 0;      // runs per row
  const bool whole = n_chunks <= FP_CHUNKS, diagonal = !whole && rpr > 0;
  const int64_t take = whole ? n_chunks : diagonal ? rows : FP_CHUNKS;
  unsigned long long h = 0;
  // eight runs per wavefront in flight: the kernel is a handful of independent loads per lane, all latency
  constexpr int FP_UNROLL = 8;
  const int64_t step = (int64_t)FP_BLOCKS * 4;
  for (int64_t j0 = (int64_t)blockIdx.x * 4 + wv; j0 < take; j0 += step * FP_UNROLL) {
    uint32_t v[FP_UNROLL];
    int64_t at[FP_UNROLL];
#pragma unroll
    for (int u = 0; u < FP_UNROLL; ++u) {
      const int64_t j = j0 + u * step;
      int64_t i = -1;
      if (j < take) {
        if (whole) i = j * 64 + lane;
        else if (diagonal) {
          const uint32_t r32 = (uint32_t)rpr, j32 = (uint32_t)j;        // rows and runs per row are far below 2^31
          const int64_t in_row = (int64_t)((j32 * 61u + j32 / r32) % r32) * 64 + lane;
          i = in_row < words_per_row ? j * words_per_row + in_row : -1;
        } else i = (int64_t)(((unsigned long long)j * (unsigned long long)n_chunks) / (unsigned long long)take) * 64 + lane;
        if (i >= words) i = -1;
      }
      at[u] = i;
      v[u] = i >= 0 ? w[i] : 0u;
    }
#pragma unroll
    for (int u = 0; u < FP_UNROLL; ++u)
      if (at[u] >= 0) h += fp_mix(v[u], (uint32_t)at[u]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) h += __shfl_xor(h, o);
  if (lane == 0) red[wv] = h;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long *line = state + (int64_t)z * FP_STATE_WORDS;
    __hip_atomic_store(line + blockIdx.x, red[0] + red[1] + red[2] + red[3], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __threadfence();
    if (atomicAdd(line + FP_BLOCKS + 1, 1ull) == (unsigned long long)(FP_BLOCKS - 1)) {
      __threadfence();
      unsigned long long now = 0;
      for (int i = 0; i < FP_BLOCKS; ++i) now += __hip_atomic_load(line + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      changed[z] = (!store_only && now != line[FP_BLOCKS]) ? 1 : 0;
      line[FP_BLOCKS] = now;
      line[FP_BLOCKS + 1] = 0ull;
    }
  }
}

// out[t][c] = sum of the biases of the decoders that run for target t, sources in ascending order, fp32
template <typename T>
__global__ __launch_bounds__(256) void k_bias_sum(const T *const *b_refs, int64_t d, int64_t L, int tying, uint64_t src_mask,
                                                  float *out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= L * d) return;
  const int64_t t = i / d, c = i - t * d;
  float acc = 0.0f;
  if (tying == CLT_TYING_PER_TARGET) {
    acc = Elem<T>::to_f32(b_refs[t][c]);
  } else {
    for (int64_t s = 0; s <= t; ++s)
      if ((src_mask >> s) & 1ull) acc += Elem<T>::to_f32(b_refs[decoder_slot(tying, s, t, L)][c]);
  }
  out[i] = acc;
}

// [F][pitch] -> [d][F], the way back: decoder z of the slab into the parameter whose address is w_refs[z].
template <typename T>
__global__ __launch_bounds__(256) void k_unpack(const T *src, T *const *w_refs, int64_t d, int64_t F, int64_t pitch) {
  __shared__ T tile[64][65];
  const T *s = src + (int64_t)blockIdx.z * F * pitch;
  T *o = w_refs[blockIdx.z];
  const int64_t f0 = (int64_t)blockIdx.x * 64, d0 = (int64_t)blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    int64_t ff = f0 + i, dd = d0 + tx;
    if (ff < F && dd < d) tile[i][tx] = s[ff * pitch + dd];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    int64_t dd = d0 + i, ff = f0 + tx;
    if (dd < d && ff < F) o[dd * F + ff] = tile[tx][i];
  }
}

// the same with 4 consecutive elements per access on both sides (d % 4 == 0, F % 4 == 0, 16-byte aligned parameters)
template <typename T>
__global__ __launch_bounds__(256) void k_unpack_vec(const T *__restrict__ src, T *const *__restrict__ w_refs, int64_t d, int64_t F,
                                                    int64_t pitch) {
  __shared__ T tile[64][68];
  const T *s = src + (int64_t)blockIdx.z * F * pitch;
  T *o = w_refs[blockIdx.z];
  const int64_t f0 = (int64_t)blockIdx.x * 64, d0 = (int64_t)blockIdx.y * 64;
  const int q = threadIdx.x & 15, r = threadIdx.x >> 4;
  typedef typename std::conditional<sizeof(T) == 2, uint2, uint4>::type quad_t;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int fl = r + 16 * i;
    const int64_t f = f0 + fl, dd = d0 + q * 4;
    if (f < F && dd < d) *reinterpret_cast<quad_t *>(&tile[fl][q * 4]) = *reinterpret_cast<const quad_t *>(s + f * pitch + dd);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int dl = r + 16 * i;
    const int64_t dd = d0 + dl, f = f0 + q * 4;
    if (dd < d && f < F) {
      T t4[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) t4[k] = tile[q * 4 + k][dl];
      *reinterpret_cast<quad_t *>(o + dd * F + f) = *reinterpret_cast<const quad_t *>(t4);
    }
  }
}

template <typename T, typename OT>
__global__ void k_densify_scatter(const int32_t *row_ptr, const int32_t *col, const T *val, OT *out,
                                  int64_t Tn, int64_t F, int64_t L, int64_t out_layer_stride) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t R = L * Tn;
  for (int64_t r = (int64_t)blockIdx.x * nwv + wv; r < R; r += (int64_t)gridDim.x * nwv) {
    const int64_t l = r / Tn, t = r - l * Tn;
    OT *orow = out + l * out_layer_stride + t * F;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) {
      if constexpr (std::is_same<T, OT>::value) orow[col[j]] = val[j];
      else orow[col[j]] = (OT)Elem<T>::to_f32(val[j]);
    }
  }
}

template <typename OT>
__global__ void k_zero_rows(OT *out, int64_t Tn, int64_t F, int64_t L, int64_t out_layer_stride) {
  const int64_t per_layer = Tn * F;
  const int64_t total = per_layer * L;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t l = i / per_layer;
    out[l * out_layer_stride + (i - l * per_layer)] = (OT)0;
  }
}

// norms[s][f]: one wavefront per (s, f), summing over the decoders fed by s.
template <typename T>
__global__ __launch_bounds__(256) void k_norms(const T *wp, T *norms, int64_t d, int64_t F, int64_t L, int tying, int64_t pitch) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t total = L * F;
  for (int64_t i = (int64_t)blockIdx.x * nwv + wv; i < total; i += (int64_t)gridDim.x * nwv) {
    const int64_t s = i / F, f = i - s * F;
    float acc = 0.0f;
    const int64_t t0 = s, t1 = tying == CLT_TYING_PER_SOURCE ? s + 1 : L;
    for (int64_t t = t0; t < t1; ++t) {
      const T *row = wp + (decoder_slot(tying, s, t, L) * F + f) * pitch;
      float part = 0.0f;
      for (int64_t o = lane; o < d; o += 64) { float w = Elem<T>::to_f32(row[o]); part = fmaf(w, w, part); }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
      // the reference squares a norm that was rounded to the model dtype (decoder.py:452)
      float nrm = Elem<T>::round(sqrtf(part));
      acc += Elem<T>::round(nrm * nrm);
    }
    if (lane == 0) norms[i] = Elem<T>::from_f32(sqrtf(acc));
  }
}

// acc[tok][f] = round(acc[tok][f] + v') over the survivors (f, v) of one layer: the running sum of
// activations that decoders tied per target consume (reference clt/models/decoder.py:208-246), every
// addition rounded to the model dtype as the reference's `summed_activation += activation_tensor` is.
// One wavefront per token row; a row's columns are distinct, so no two lanes touch one element.
template <typename T>
__global__ __launch_bounds__(256) void k_accumulate_dense(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col,
                                                          const T *__restrict__ val, const T *__restrict__ foff,
                                                          const T *__restrict__ fscale, T *__restrict__ acc, int64_t Tn,
                                                          int64_t F, int64_t layer, int init) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  for (int64_t tok = (int64_t)blockIdx.x * nwv + wv; tok < Tn; tok += (int64_t)gridDim.x * nwv) {
    const int64_t r = layer * Tn + tok;
    T *arow = acc + tok * F;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) {
      const int32_t f = col[j];
      float v = Elem<T>::to_f32(val[j]);
      if (v != 0.0f) {   // the affine terms apply to the selected (non-zero) entries only
        if (foff) v = Elem<T>::round(v + Elem<T>::to_f32(foff[f]));
        if (fscale) v = Elem<T>::round(v * Elem<T>::to_f32(fscale[f]));
      }
      const float old = init ? 0.0f : Elem<T>::to_f32(arow[f]);
      arow[f] = Elem<T>::from_f32(old + v);
    }
  }
}

constexpr int DEC_SLICES = 8;  // one feature slice per XCD of an MI355X

static size_t decode_ws_bytes(int64_t Tn, int64_t d, int64_t L) {
  size_t part = ((size_t)DEC_SLICES * L * Tn * d * 4 + 255) & ~(size_t)255;
  size_t sp = ((size_t)L * Tn * (DEC_SLICES + 1) * 4 + 255) & ~(size_t)255;
  return part + sp;
}

// feature slices of the line schedule: F x 128 bytes per slice must stay inside an L2
static int line_slices(int64_t F) { return (int)clt_ceil_div(F * 128, LINE_L2_BYTES); }
// The quarter schedule keeps F / QUARTER_SLICES rows x a quarter of the columns per XCD: it is taken while
// that stays near one 4 MiB L2 (measured: 4.7 MiB at F = 24576, d = 768 bf16 is still 2 % ahead of the line
// schedule, 8.4 MiB at F = 32768, d = 1024 is 25 % behind it)
constexpr int64_t QUARTER_L2_BYTES = 5 << 20;
static bool quarter_fits(int64_t F, int64_t d, int elem_bytes) {
  return (F / QUARTER_SLICES) * (d / QUARTER_PARTS) * elem_bytes <= QUARTER_L2_BYTES;
}

static bool quarter_shape_ok(int64_t d, int elem_bytes) {
  const int V = 16 / elem_bytes;
  const int per_lane = (int)(d / 64), hq = per_lane / V;
  const bool htail = (per_lane % V) != 0;
  if (elem_bytes == 2) return (hq == 1) || (hq == 2 && !htail) || (hq == 4 && !htail);
  return (hq == 2 || hq == 3 || hq == 4) && !htail;
}

// Which schedule launch_decode takes; `ws_ok`: a workspace of decode_ws_bytes(), 256-byte aligned;
// `wp_ok`: the packed decoders are 16-byte aligned.
static int plan_route(int64_t d, int64_t F, int tying, int elem_bytes, bool ws_ok, bool wp_ok) {
  const int V = 16 / elem_bytes;
  const int64_t chunk = 64 * V, nf = d / chunk, rem = d % chunk;
  const bool can_slice = ws_ok && (d % 4 == 0) && F >= 64 * DEC_SLICES;
  const bool fast = (d % V == 0) && wp_ok && nf <= 4 && (nf > 0 || rem > 0);
  if (fast && can_slice && tying != CLT_TYING_PER_TARGET && d % 256 == 0 && F >= 64 * QUARTER_SLICES &&
      quarter_shape_ok(d, elem_bytes) && quarter_fits(F, d, elem_bytes))
    return CLT_ROUTE_QUARTER;
  // the line schedule takes any width that is a whole number of cache lines
  if (can_slice && wp_ok && tying != CLT_TYING_PER_TARGET && (d * elem_bytes) % 128 == 0 && line_slices(F) <= DEC_SLICES)
    return CLT_ROUTE_LINE;
  if (!fast) return CLT_ROUTE_GENERIC;
  if (!can_slice) return CLT_ROUTE_SINGLE;
  return tying == CLT_TYING_PER_TARGET ? CLT_ROUTE_SLICED_ALL_SOURCES : CLT_ROUTE_SLICED;
}

template <typename T>
static int launch_decode(const int32_t *row_ptr, const int32_t *col, const void *val, const void *wp,
                         const float *bias_sum, const void *foff, const void *fscale, const float *skip_add,
                         void *out, int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t t_begin,
                         int64_t t_end, uint64_t src_mask, int out_f32, void *workspace, size_t workspace_bytes,
                         hipStream_t stream) {
  constexpr int V = WVec<T>::V;
  const int nwv = 4;
  const int64_t pitch = clt_pitch(d, (int)sizeof(T));
  const int64_t blocks_per_t = clt_ceil_div(Tn, nwv);
  const bool can_slice = workspace && workspace_bytes >= decode_ws_bytes(Tn, d, L) && (d % 4 == 0) &&
                         F >= 64 * DEC_SLICES && ((((uintptr_t)workspace) & 255u) == 0);
  const int ns = can_slice ? DEC_SLICES : 1;
  int32_t *sptr = nullptr; float *partial = nullptr;
  if (can_slice) {
    partial = (float *)workspace;
    sptr = (int32_t *)((char *)workspace + (((size_t)DEC_SLICES * L * Tn * d * 4 + 255) & ~(size_t)255));
  }
  int64_t nblk = blocks_per_t * (t_end - t_begin);
  if (nblk <= 0) return CLT_OK;
  if (nblk > 2147483647LL) return CLT_ERR_RANGE;
  const bool affine = foff || fscale;
  const int64_t chunk = 64 * V;
  const int64_t nf = d / chunk, rem = d % chunk;
  const bool fast = (d % V == 0) && clt_aligned16(wp) && nf <= 4 && (nf > 0 || rem > 0);
  const int route = plan_route(d, F, tying, (int)sizeof(T), can_slice, clt_aligned16(wp));
  if (can_slice && !fast && route != CLT_ROUTE_LINE)
    return launch_decode<T>(row_ptr, col, val, wp, bias_sum, foff, fscale, skip_add, out, Tn, d, F,
                            L, tying, t_begin, t_end, src_mask, out_f32, nullptr, 0, stream);
#define CLT_DEC_ARGS(FO, FS)                                                                                    \
  row_ptr, col, (const T *)val, (const T *)wp, bias_sum, FO, FS, skip_add, out, Tn, d, F, L, tying, tb,         \
      t_end, src_mask, out_f32, sptr, partial, ns, src, pitch
#define CLT_DEC(NFN, TL, UN)                                                                                    \
  do {                                                                                                          \
    if (affine && can_slice)                                                                                    \
      k_decode<T, NFN, TL, UN, true, true><<<(unsigned)nblk, 256, 0, stream>>>(CLT_DEC_ARGS((const T *)foff, (const T *)fscale)); \
    else if (affine)                                                                                            \
      k_decode<T, NFN, TL, UN, true, false><<<(unsigned)nblk, 256, 0, stream>>>(CLT_DEC_ARGS((const T *)foff, (const T *)fscale)); \
    else if (can_slice)                                                                                         \
      k_decode<T, NFN, TL, UN, false, true><<<(unsigned)nblk, 256, 0, stream>>>(CLT_DEC_ARGS(nullptr, nullptr)); \
    else                                                                                                        \
      k_decode<T, NFN, TL, UN, false, false><<<(unsigned)nblk, 256, 0, stream>>>(CLT_DEC_ARGS(nullptr, nullptr)); \
  } while (0)
#define CLT_DEC_TAIL(NFN, UN)                              \
  do {                                                     \
    if (rem == 0) CLT_DEC(NFN, 0, UN);                     \
    else if (rem * 2 == chunk) CLT_DEC(NFN, 1, UN);        \
    else CLT_DEC(NFN, 2, UN);                              \
  } while (0)
  // quarter-row schedule: 2 feature slices x 4 column quarters (see k_decode_quarter)
  bool quartered = false; int quarter_ns = QUARTER_SLICES;
  if (route == CLT_ROUTE_LINE) {
    constexpr int ntok = 2;                               // tokens per wavefront
    const UnitPlan lp = make_unit_plan(line_slices(F), (int)(d * (int64_t)sizeof(T) / 128), Tn, nwv * ntok);
    // one 32-bit word per survivor and 32-bit row offsets: feature index below 2^16, matrix below 4 GiB
    const bool pack = sizeof(T) == 2 && F <= 65536 && F * pitch * (int64_t)sizeof(T) < (1ll << 32);
    k_slice_ptr<<<1024, 256, 0, stream>>>(row_ptr, col, L * Tn, F, lp.ns, sptr);
    for (int src = 0; src < (int)t_end; ++src) {
      if (!((src_mask >> src) & 1ull)) continue;
      const int64_t tb = src > t_begin ? src : t_begin;
      const int64_t lb = 8 * (int64_t)lp.bpx * (t_end - tb);
      if (lb <= 0) continue;
      if (lb > 2147483647LL) return CLT_ERR_RANGE;
#define CLT_DECL(AF, PK, NT)                                                                                          \
  k_decode_line<T, AF, PK, NT><<<(unsigned)lb, 256, 0, stream>>>(col, (const T *)val, (const T *)wp, (const T *)foff, \
      (const T *)fscale, Tn, d, F, L, tying, tb, src_mask, sptr, partial, src, lp, pitch)
#define CLT_DECL2(AF, PK) CLT_DECL(AF, PK, ntok)
      if (affine) { if (pack) CLT_DECL2(true, true); else CLT_DECL2(true, false); }
      else { if (pack) CLT_DECL2(false, true); else CLT_DECL2(false, false); }
#undef CLT_DECL2
#undef CLT_DECL
    }
    k_decode_reduce<T><<<2048, 256, 0, stream>>>(partial, bias_sum, skip_add, out, Tn, d, L, t_begin, t_end, lp.ns, out_f32, src_mask);
    return clt_check_launch();
  }
  if (route == CLT_ROUTE_QUARTER) {
    const int per_lane = (int)(d / 64);                    // columns per lane
    const int hq = per_lane / V, htail = (per_lane % V) != 0;
    // feature slices: F / qs rows x a quarter of the columns per XCD at a time, about one L2
    const int qs = QUARTER_SLICES;
    const UnitPlan up = make_unit_plan(qs, QUARTER_PARTS, Tn, nwv * QUARTER_NTOK);
    // one 32-bit word per survivor and 32-bit row offsets: feature index below 2^16, matrix below 4 GiB
    const bool qpack = sizeof(T) == 2 && F <= 65536 && F * pitch * (int64_t)sizeof(T) < (1ll << 32);
#define CLT_DECQ(HQN, HTN, UN)                                                                                       \
  do {                                                                                                               \
    k_slice_ptr<<<1024, 256, 0, stream>>>(row_ptr, col, L * Tn, F, qs, sptr);                                        \
    for (int src = 0; src < (int)t_end; ++src) {                                                                     \
      if (!((src_mask >> src) & 1ull)) continue;                                                                     \
      const int64_t tb = src > t_begin ? src : t_begin;                                                              \
      const int64_t qb = 8 * (int64_t)up.bpx * (t_end - tb);                                                         \
      if (qb <= 0) continue;                                                                                         \
      if (qb > 2147483647LL) return CLT_ERR_RANGE;                                                                   \
      if (affine) k_decode_quarter<T, HQN, HTN, UN, true, false><<<(unsigned)qb, 256, 0, stream>>>(col, (const T *)val, (const T *)wp, \
          (const T *)foff, (const T *)fscale, Tn, d, F, L, tying, tb, src_mask, sptr, partial, src, pitch, up);      \
      else if (qpack) k_decode_quarter<T, HQN, HTN, UN, false, sizeof(T) == 2><<<(unsigned)qb, 256, 0, stream>>>(col, (const T *)val, (const T *)wp, \
          nullptr, nullptr, Tn, d, F, L, tying, tb, src_mask, sptr, partial, src, pitch, up);                        \
      else k_decode_quarter<T, HQN, HTN, UN, false, false><<<(unsigned)qb, 256, 0, stream>>>(col, (const T *)val, (const T *)wp, \
          nullptr, nullptr, Tn, d, F, L, tying, tb, src_mask, sptr, partial, src, pitch, up);                        \
    }                                                                                                                \
    quartered = true; quarter_ns = qs;                                                                               \
  } while (0)
    if constexpr (sizeof(T) == 2) {
      if (hq == 1 && !htail) CLT_DECQ(1, 0, 2);
      else if (hq == 1 && htail) CLT_DECQ(1, 1, 2);
      else if (hq == 2 && !htail) CLT_DECQ(2, 0, 2);
      else if (hq == 4 && !htail) CLT_DECQ(4, 0, 2);
    } else {
      if (hq == 2 && !htail) CLT_DECQ(2, 0, 2);
      else if (hq == 3 && !htail) CLT_DECQ(3, 0, 2);
      else if (hq == 4 && !htail) CLT_DECQ(4, 0, 2);
    }
#undef CLT_DECQ
  }
  if (quartered) {
    k_decode_reduce<T><<<2048, 256, 0, stream>>>(partial, bias_sum, skip_add, out, Tn, d, L, t_begin, t_end, quarter_ns, out_f32, src_mask);
    return clt_check_launch();
  }
  if (can_slice) k_slice_ptr<<<1024, 256, 0, stream>>>(row_ptr, col, L * Tn, F, ns, sptr);
  if (fast) {
    // sliced: one launch per source layer, targets max(src, t_begin) .. t_end-1
    // decoders tied per target: one launch, sources walked inside the wavefront (src = -1)
    const bool all_src = can_slice && tying == CLT_TYING_PER_TARGET;
    const int n_launch = all_src ? 1 : (can_slice ? (int)t_end : 1);
    for (int src0 = 0; src0 < n_launch; ++src0) {
      const int src = all_src ? -1 : src0;
      int64_t tb = t_begin;
      if (all_src) {
        nblk = clt_ceil_div(Tn, nwv * SLICED_NTOK) * (t_end - tb) * ns;
        if (nblk > 2147483647LL) return CLT_ERR_RANGE;
      } else if (can_slice) {
        if (!((src_mask >> src) & 1ull)) continue;
        if (src > tb) tb = src;
        nblk = clt_ceil_div(Tn, nwv * SLICED_NTOK) * (t_end - tb) * ns;
        if (nblk <= 0) continue;
        if (nblk > 2147483647LL) return CLT_ERR_RANGE;
      }
      if (nf == 0) CLT_DEC(0, 2, 8);
      else if (nf == 1) CLT_DEC_TAIL(1, 8);
      else if (nf == 2) CLT_DEC_TAIL(2, 6);
      else if (nf == 3) CLT_DEC_TAIL(3, 4);
      else if (rem == 0) CLT_DEC(4, 0, 4);
      else CLT_DEC(4, 2, 2);
    }
  } else {
    const int64_t tb = t_begin; const int src = 0; (void)tb; (void)src;
    k_decode_generic<T><<<(unsigned)nblk, 256, 0, stream>>>(row_ptr, col, (const T *)val, (const T *)wp, bias_sum,
        (const T *)foff, (const T *)fscale, skip_add, out, Tn, d, F, L, tying, t_begin, t_end, src_mask, out_f32, pitch);
  }
#undef CLT_DEC_TAIL
#undef CLT_DEC
#undef CLT_DEC_ARGS
  if (can_slice)
    k_decode_reduce<T><<<2048, 256, 0, stream>>>(partial, bias_sum, skip_add, out, Tn, d, L, t_begin, t_end, ns, out_f32, src_mask);
  return clt_check_launch();
}

}  // namespace

extern "C" size_t clt_decode_workspace_bytes(int64_t T, int64_t d, int64_t F, int64_t L) {
  (void)F;
  if (T <= 0 || d <= 0 || L <= 0) return 256;
  return decode_ws_bytes(T, d, L);
}

extern "C" int clt_decode_sparse(const int32_t *row_ptr, const int32_t *col, const void *val, const void *w_packed,
                                 const float *bias_sum, const void *feat_offset, const void *feat_scale,
                                 const float *skip_add, void *out, int64_t T, int64_t d, int64_t F, int64_t L,
                                 int tying, int64_t t_begin, int64_t t_end, uint64_t src_mask, int dtype,
                                 int out_f32, void *workspace, size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || d <= 0 || F <= 0 || L <= 0 || L > 64) return CLT_ERR_ARG;
  if (t_begin < 0 || t_end > L || t_begin > t_end) return CLT_ERR_ARG;
  if (tying < 0 || tying > 2) return CLT_ERR_ARG;
  if (T == 0 || t_begin == t_end) return CLT_OK;
  if (!row_ptr || !w_packed || !out) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16)
    return launch_decode<bf16_t>(row_ptr, col, val, w_packed, bias_sum, feat_offset, feat_scale, skip_add, out, T, d, F, L, tying, t_begin, t_end, src_mask, out_f32, workspace, workspace_bytes, s);
  if (dtype == CLT_F16)
    return launch_decode<f16_t>(row_ptr, col, val, w_packed, bias_sum, feat_offset, feat_scale, skip_add, out, T, d, F, L, tying, t_begin, t_end, src_mask, out_f32, workspace, workspace_bytes, s);
  return launch_decode<float>(row_ptr, col, val, w_packed, bias_sum, feat_offset, feat_scale, skip_add, out, T, d, F, L, tying, t_begin, t_end, src_mask, out_f32, workspace, workspace_bytes, s);
}

extern "C" int clt_pack_decoder(const void *w_ref, void *w_packed, int64_t d, int64_t F, int64_t n_dec,
                                int64_t in_stride, int64_t out_stride, int dtype, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || n_dec < 0 || n_dec > 65535) return CLT_ERR_ARG;
  if (n_dec == 0) return CLT_OK;
  if (!w_ref || !w_packed) return CLT_ERR_ARG;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)clt_ceil_div(d, 64), (unsigned)n_dec);
  if (clt_ceil_div(d, 64) > 65535) return CLT_ERR_RANGE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype != CLT_F32) k_pack<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)w_ref, (bf16_t *)w_packed, d, F, in_stride, out_stride, clt_pitch(d, 2));
  else k_pack<float><<<grid, 256, 0, s>>>((const float *)w_ref, (float *)w_packed, d, F, in_stride, out_stride, clt_pitch(d, 4));
  return clt_check_launch();
}

extern "C" int clt_decoder_fingerprint(void *const *w_refs_dev, int64_t n_dec, int64_t d, int64_t F, int dtype,
                                       uint64_t *state, int32_t *changed, int store_only, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || n_dec < 0 || n_dec > 65535) return CLT_ERR_ARG;
  if (n_dec == 0) return CLT_OK;
  if (!w_refs_dev || !state || !changed) return CLT_ERR_ARG;
  const int64_t words = d * F * clt_elem_bytes(dtype) / 4;     // a last odd 16-bit element is not looked at
  if (words <= 0) return CLT_ERR_ARG;
  const int64_t row_bytes = F * clt_elem_bytes(dtype);
  if ((((uintptr_t)state) & 127u) != 0) return CLT_ERR_ALIGN;
  k_fingerprint<<<dim3(FP_BLOCKS, (unsigned)n_dec), 256, 0, (hipStream_t)stream>>>(
      (const uint32_t *const *)w_refs_dev, words, d, row_bytes % 4 == 0 ? row_bytes / 4 : 0,
      (unsigned long long *)state, changed, store_only);
  return clt_check_launch();
}

extern "C" int clt_pack_decoders_if(void *const *w_refs_dev, void *w_packed, int64_t n_dec, int64_t d, int64_t F,
                                    int dtype, const int32_t *changed, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || n_dec < 0 || n_dec > 65535) return CLT_ERR_ARG;
  if (n_dec == 0) return CLT_OK;
  if (!w_refs_dev || !w_packed || !changed) return CLT_ERR_ARG;
  const dim3 grid(FP_PACK_BLOCKS, (unsigned)n_dec);
  hipStream_t s = (hipStream_t)stream;
  if (dtype != CLT_F32) k_pack_if<bf16_t><<<grid, 256, 0, s>>>((bf16_t *const *)w_refs_dev, (bf16_t *)w_packed, d, F, clt_pitch(d, 2), changed);
  else k_pack_if<float><<<grid, 256, 0, s>>>((float *const *)w_refs_dev, (float *)w_packed, d, F, clt_pitch(d, 4), changed);
  return clt_check_launch();
}

extern "C" int clt_bias_sum(void *const *b_refs_dev, int64_t n_dec, int64_t d, int64_t L, int tying, uint64_t src_mask,
                            int dtype, float *out, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (d <= 0 || L <= 0 || L > 64 || tying < 0 || tying > 2 || !b_refs_dev || !out) return CLT_ERR_ARG;
  if (n_dec != (tying == CLT_TYING_NONE ? L * (L + 1) / 2 : L)) return CLT_ERR_ARG;
  const unsigned nb = (unsigned)clt_ceil_div(L * d, 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_bias_sum<bf16_t><<<nb, 256, 0, s>>>((const bf16_t *const *)b_refs_dev, d, L, tying, src_mask, out);
  else if (dtype == CLT_F16) k_bias_sum<f16_t><<<nb, 256, 0, s>>>((const f16_t *const *)b_refs_dev, d, L, tying, src_mask, out);
  else k_bias_sum<float><<<nb, 256, 0, s>>>((const float *const *)b_refs_dev, d, L, tying, src_mask, out);
  return clt_check_launch();
}

extern "C" int clt_unpack_decoders(const void *w_packed, void *const *w_refs_dev, void *const *w_refs_host, int64_t n_dec,
                                   int64_t d, int64_t F, int dtype, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || n_dec < 0 || n_dec > 65535) return CLT_ERR_ARG;
  if (n_dec == 0) return CLT_OK;
  if (!w_packed || !w_refs_dev) return CLT_ERR_ARG;
  if (clt_ceil_div(d, 64) > 65535) return CLT_ERR_RANGE;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)clt_ceil_div(d, 64), (unsigned)n_dec);
  hipStream_t s = (hipStream_t)stream;
  // w_refs_host (optional): the same addresses on the host, to see whether the 4-element kernel may be used
  bool vec = w_refs_host != nullptr && d % 4 == 0 && F % 4 == 0;
  for (int64_t i = 0; vec && i < n_dec; ++i) vec = clt_aligned16(w_refs_host[i]);
  if (vec) {
    if (dtype != CLT_F32) k_unpack_vec<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)w_packed, (bf16_t *const *)w_refs_dev, d, F, clt_pitch(d, 2));
    else k_unpack_vec<float><<<grid, 256, 0, s>>>((const float *)w_packed, (float *const *)w_refs_dev, d, F, clt_pitch(d, 4));
  } else {
    if (dtype != CLT_F32) k_unpack<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)w_packed, (bf16_t *const *)w_refs_dev, d, F, clt_pitch(d, 2));
    else k_unpack<float><<<grid, 256, 0, s>>>((const float *)w_packed, (float *const *)w_refs_dev, d, F, clt_pitch(d, 4));
  }
  return clt_check_launch();
}

extern "C" int clt_densify(const int32_t *row_ptr, const int32_t *col, const void *val, void *out, int64_t T,
                           int64_t F, int64_t L, int64_t out_layer_stride, int dtype, int out_f32, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0) return CLT_ERR_ARG;
  if (T == 0 || F == 0) return CLT_OK;
  if (!row_ptr || !out) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int nb = 256 * 8;
  if (dtype == CLT_F32 || out_f32) k_zero_rows<float><<<nb, 256, 0, s>>>((float *)out, T, F, L, out_layer_stride);
  else k_zero_rows<bf16_t><<<nb, 256, 0, s>>>((bf16_t *)out, T, F, L, out_layer_stride);
  if (dtype == CLT_F32) k_densify_scatter<float, float><<<nb, 256, 0, s>>>(row_ptr, col, (const float *)val, (float *)out, T, F, L, out_layer_stride);
  else if (out_f32 && dtype == CLT_F16) k_densify_scatter<f16_t, float><<<nb, 256, 0, s>>>(row_ptr, col, (const f16_t *)val, (float *)out, T, F, L, out_layer_stride);
  else if (out_f32) k_densify_scatter<bf16_t, float><<<nb, 256, 0, s>>>(row_ptr, col, (const bf16_t *)val, (float *)out, T, F, L, out_layer_stride);
  else k_densify_scatter<bf16_t, bf16_t><<<nb, 256, 0, s>>>(row_ptr, col, (const bf16_t *)val, (bf16_t *)out, T, F, L, out_layer_stride);
  return clt_check_launch();
}

extern "C" int clt_decoder_norms(const void *w_packed, void *norms, int64_t d, int64_t F, int64_t L, int tying,
                                 int dtype, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || L <= 0 || tying < 0 || tying > 2 || !w_packed || !norms) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_norms<bf16_t><<<256 * 8, 256, 0, s>>>((const bf16_t *)w_packed, (bf16_t *)norms, d, F, L, tying, clt_pitch(d, 2));
  else if (dtype == CLT_F16) k_norms<f16_t><<<256 * 8, 256, 0, s>>>((const f16_t *)w_packed, (f16_t *)norms, d, F, L, tying, clt_pitch(d, 2));
  else k_norms<float><<<256 * 8, 256, 0, s>>>((const float *)w_packed, (float *)norms, d, F, L, tying, clt_pitch(d, 4));
  return clt_check_launch();
}

extern "C" int clt_decode_route(int64_t T, int64_t d, int64_t F, int64_t L, int tying, int dtype,
                                size_t workspace_bytes) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || d <= 0 || F <= 0 || L <= 0 || L > 64 || tying < 0 || tying > 2) return CLT_ERR_ARG;
  return plan_route(d, F, tying, clt_elem_bytes(dtype), workspace_bytes >= decode_ws_bytes(T, d, L), true);
}

extern "C" int64_t clt_decoder_pitch(int64_t d, int dtype) {
  if (d <= 0 || !clt_model_dtype(dtype)) return -1;
  return clt_pitch(d, clt_elem_bytes(dtype));
}

extern "C" int64_t clt_decoder_slab_elems(int64_t d, int64_t F, int64_t L, int tying, int dtype) {
  if (d <= 0 || F <= 0 || L <= 0 || tying < 0 || tying > 2 || !clt_model_dtype(dtype)) return -1;
  const int64_t pitch = clt_pitch(d, clt_elem_bytes(dtype));
  const int64_t n_dec = tying == CLT_TYING_NONE ? L * (L + 1) / 2 : L;
  // the last element any schedule can touch: row F-1 of slot n_dec-1, formed like the kernels form it
  const int64_t last = decoder_slot_host(tying, L - 1, L - 1, L) * F * pitch + (F - 1) * pitch + (d - 1);
  return last + 1 == n_dec * F * pitch - (pitch - d) ? n_dec * F * pitch : -1;
}

extern "C" int clt_accumulate_dense(const int32_t *row_ptr, const int32_t *col, const void *val,
                                    const void *feat_offset, const void *feat_scale, void *acc, int64_t T,
                                    int64_t F, int64_t layer, int init, int dtype, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F <= 0 || (layer < 0 && !init)) return CLT_ERR_ARG;
  if (T == 0) return CLT_OK;
  if (!acc || (layer >= 0 && !row_ptr)) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const unsigned nb = (unsigned)(clt_ceil_div(T, 4) < 8192 ? clt_ceil_div(T, 4) : 8192);
  if (init) {
    if (dtype != CLT_F32) k_zero_rows<bf16_t><<<2048, 256, 0, s>>>((bf16_t *)acc, T, F, 1, T * F);
    else k_zero_rows<float><<<2048, 256, 0, s>>>((float *)acc, T, F, 1, T * F);
  }
  if (layer < 0) return clt_check_launch();   // clear only
  if (dtype == CLT_BF16)
    k_accumulate_dense<bf16_t><<<nb, 256, 0, s>>>(row_ptr, col, (const bf16_t *)val, (const bf16_t *)feat_offset,
                                                 (const bf16_t *)feat_scale, (bf16_t *)acc, T, F, layer, init);
  else if (dtype == CLT_F16)
    k_accumulate_dense<f16_t><<<nb, 256, 0, s>>>(row_ptr, col, (const f16_t *)val, (const f16_t *)feat_offset,
                                                 (const f16_t *)feat_scale, (f16_t *)acc, T, F, layer, init);
  else
    k_accumulate_dense<float><<<nb, 256, 0, s>>>(row_ptr, col, (const float *)val, (const float *)feat_offset,
                                                (const float *)feat_scale, (float *)acc, T, F, layer, init);
  return clt_check_launch();
}
