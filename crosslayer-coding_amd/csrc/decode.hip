// Sparse cross-layer decode, decoder repacking, densify and decoder norms.
//
// Decode (reference clt/models/decoder.py:176-340): the reference multiplies dense
// [T,F] activations that are >99 % zeros by every decoder.  Here each (token, target)
// pair is one wavefront that walks the survivor rows of the sources s <= t, fetches the
// decoder vector of every active feature (feature-major packing: one contiguous
// d-element run, 16 bytes per lane per load) and accumulates in fp32 registers; the
// output row is written once.
#include "clt_common.h"

namespace {

template <typename T> struct WVec;
template <> struct WVec<float> {
  static constexpr int V = 4;
  __device__ static __forceinline__ void fma(float (&acc)[4], const float *p, float v) {
    float4 w = *reinterpret_cast<const float4 *>(p);
    acc[0] = fmaf(v, w.x, acc[0]); acc[1] = fmaf(v, w.y, acc[1]);
    acc[2] = fmaf(v, w.z, acc[2]); acc[3] = fmaf(v, w.w, acc[3]);
  }
};
template <> struct WVec<bf16_t> {
  static constexpr int V = 8;
  __device__ static __forceinline__ void fma(float (&acc)[8], const bf16_t *p, float v) {
    uint4 w = *reinterpret_cast<const uint4 *>(p);
    uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[2 * j] = fmaf(v, __uint_as_float(u[j] << 16), acc[2 * j]);
      acc[2 * j + 1] = fmaf(v, __uint_as_float(u[j] & 0xFFFF0000u), acc[2 * j + 1]);
    }
  }
};

__device__ __forceinline__ int64_t decoder_slot(int tying, int64_t s, int64_t t, int64_t L) {
  if (tying == CLT_TYING_PER_SOURCE) return s;
  if (tying == CLT_TYING_PER_TARGET) return t;
  return s * L - (s * (s - 1)) / 2 + (t - s);
}

// One wavefront per (target, token).  CH = number of 64-lane x V-element chunks that cover d.
template <typename T, int CH, bool AFFINE>
__global__ __launch_bounds__(256) void k_decode(
    const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col, const T *__restrict__ val,
    const T *__restrict__ wp, const float *__restrict__ bias_sum, const T *__restrict__ foff,
    const T *__restrict__ fscale, const float *__restrict__ skip_add, void *__restrict__ out,
    int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t t_begin, int64_t t_end,
    uint64_t src_mask, int out_f32) {
  constexpr int V = WVec<T>::V;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t blocks_per_t = (Tn + nwv - 1) / nwv;
  // heaviest targets (most sources) first
  const int64_t t = t_end - 1 - (int64_t)blockIdx.x / blocks_per_t;
  const int64_t tok = ((int64_t)blockIdx.x % blocks_per_t) * nwv + wv;
  if (tok >= Tn) return;
  float acc[CH][V];
#pragma unroll
  for (int c = 0; c < CH; ++c)
#pragma unroll
    for (int j = 0; j < V; ++j) acc[c][j] = 0.0f;
  bool lane_on[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) lane_on[c] = (int64_t)(c * 64 + lane) * V < d;

  for (int64_t s = 0; s <= t; ++s) {
    if (!((src_mask >> s) & 1ull)) continue;
    const int64_t r = s * Tn + tok;
    const int32_t b = row_ptr[r], e = row_ptr[r + 1];
    const T *wbase = wp + decoder_slot(tying, s, t, L) * F * d + (int64_t)lane * V;
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
#pragma unroll 4
      for (int i = 0; i < n; ++i) {
        const int32_t f = __builtin_amdgcn_readlane(my_col, i);
        const float v = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(my_val), i));
        const T *wrow = wbase + (int64_t)f * d;
#pragma unroll
        for (int c = 0; c < CH; ++c)
          if (lane_on[c]) WVec<T>::fma(acc[c], wrow + c * 64 * V, v);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    if (!lane_on[c]) continue;
    const int64_t o = (int64_t)(c * 64 + lane) * V;
    float y[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
      y[j] = acc[c][j];
      if (bias_sum) y[j] += bias_sum[t * d + o + j];
      if (skip_add) y[j] += skip_add[(t * Tn + tok) * d + o + j];
    }
    if (out_f32) {
      float *po = (float *)out + (t * Tn + tok) * d + o;
#pragma unroll
      for (int j = 0; j < V; ++j) po[j] = y[j];
    } else {
      T *po = (T *)out + (t * Tn + tok) * d + o;
#pragma unroll
      for (int j = 0; j < V; ++j) po[j] = Elem<T>::from_f32(y[j]);
    }
  }
}

// Any d (no alignment assumption): lanes stride over the output row one element at a time.
template <typename T>
__global__ __launch_bounds__(256) void k_decode_generic(
    const int32_t *row_ptr, const int32_t *col, const T *val, const T *wp, const float *bias_sum,
    const T *foff, const T *fscale, const float *skip_add, void *out, int64_t Tn, int64_t d,
    int64_t F, int64_t L, int tying, int64_t t_begin, int64_t t_end, uint64_t src_mask, int out_f32) {
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
      const T *wbase = wp + decoder_slot(tying, s, t, L) * F * d;
      for (int32_t j = row_ptr[r]; j < row_ptr[r + 1]; ++j) {
        const int32_t f = col[j];
        float v = Elem<T>::to_f32(val[j]);
        if (v != 0.0f) {
          if (foff) v = Elem<T>::round(v + Elem<T>::to_f32(foff[t * F + f]));
          if (fscale) v = Elem<T>::round(v * Elem<T>::to_f32(fscale[t * F + f]));
        }
        if (o < d) acc = fmaf(v, Elem<T>::to_f32(wbase[(int64_t)f * d + o]), acc);
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
                                              int64_t in_stride, int64_t out_stride) {
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
    if (ff < F && dd < d) o[ff * d + dd] = tile[tx][i];
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
      float v = Elem<T>::to_f32(val[j]);
      orow[col[j]] = sizeof(OT) == 4 ? (OT)v : (OT)val[j];
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
__global__ __launch_bounds__(256) void k_norms(const T *wp, T *norms, int64_t d, int64_t F, int64_t L, int tying) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t total = L * F;
  for (int64_t i = (int64_t)blockIdx.x * nwv + wv; i < total; i += (int64_t)gridDim.x * nwv) {
    const int64_t s = i / F, f = i - s * F;
    float acc = 0.0f;
    const int64_t t0 = s, t1 = tying == CLT_TYING_PER_SOURCE ? s + 1 : L;
    for (int64_t t = t0; t < t1; ++t) {
      const T *row = wp + (decoder_slot(tying, s, t, L) * F + f) * d;
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

template <typename T>
static int launch_decode(const int32_t *row_ptr, const int32_t *col, const void *val, const void *wp,
                         const float *bias_sum, const void *foff, const void *fscale, const float *skip_add,
                         void *out, int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t t_begin,
                         int64_t t_end, uint64_t src_mask, int out_f32, hipStream_t stream) {
  constexpr int V = WVec<T>::V;
  const int nwv = 4;
  const int64_t blocks_per_t = clt_ceil_div(Tn, nwv);
  const int64_t nblk = blocks_per_t * (t_end - t_begin);
  if (nblk <= 0) return CLT_OK;
  if (nblk > 2147483647LL) return CLT_ERR_RANGE;
  const bool affine = foff || fscale;
  const bool fast = (d % V == 0) && clt_aligned16(wp) && d <= 64 * V * 8;
#define CLT_DEC(CHN)                                                                                          \
  do {                                                                                                        \
    if (affine)                                                                                               \
      k_decode<T, CHN, true><<<(unsigned)nblk, 256, 0, stream>>>(row_ptr, col, (const T *)val, (const T *)wp, \
          bias_sum, (const T *)foff, (const T *)fscale, skip_add, out, Tn, d, F, L, tying, t_begin, t_end,     \
          src_mask, out_f32);                                                                                 \
    else                                                                                                      \
      k_decode<T, CHN, false><<<(unsigned)nblk, 256, 0, stream>>>(row_ptr, col, (const T *)val, (const T *)wp,\
          bias_sum, nullptr, nullptr, skip_add, out, Tn, d, F, L, tying, t_begin, t_end, src_mask, out_f32);  \
  } while (0)
  if (fast) {
    const int64_t ch = clt_ceil_div(d, 64 * V);
    if (ch <= 1) CLT_DEC(1);
    else if (ch == 2) CLT_DEC(2);
    else if (ch == 3) CLT_DEC(3);
    else if (ch == 4) CLT_DEC(4);
    else if (ch <= 6) CLT_DEC(6);
    else CLT_DEC(8);
  } else {
    k_decode_generic<T><<<(unsigned)nblk, 256, 0, stream>>>(row_ptr, col, (const T *)val, (const T *)wp, bias_sum,
        (const T *)foff, (const T *)fscale, skip_add, out, Tn, d, F, L, tying, t_begin, t_end, src_mask, out_f32);
  }
#undef CLT_DEC
  return clt_check_launch();
}

}  // namespace

extern "C" int clt_decode_sparse(const int32_t *row_ptr, const int32_t *col, const void *val, const void *w_packed,
                                 const float *bias_sum, const void *feat_offset, const void *feat_scale,
                                 const float *skip_add, void *out, int64_t T, int64_t d, int64_t F, int64_t L,
                                 int tying, int64_t t_begin, int64_t t_end, uint64_t src_mask, int dtype,
                                 int out_f32, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T < 0 || d <= 0 || F <= 0 || L <= 0 || L > 64) return CLT_ERR_ARG;
  if (t_begin < 0 || t_end > L || t_begin > t_end) return CLT_ERR_ARG;
  if (tying < 0 || tying > 2) return CLT_ERR_ARG;
  if (T == 0 || t_begin == t_end) return CLT_OK;
  if (!row_ptr || !w_packed || !out) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16)
    return launch_decode<bf16_t>(row_ptr, col, val, w_packed, bias_sum, feat_offset, feat_scale, skip_add, out, T, d, F, L, tying, t_begin, t_end, src_mask, out_f32, s);
  return launch_decode<float>(row_ptr, col, val, w_packed, bias_sum, feat_offset, feat_scale, skip_add, out, T, d, F, L, tying, t_begin, t_end, src_mask, out_f32, s);
}

extern "C" int clt_pack_decoder(const void *w_ref, void *w_packed, int64_t d, int64_t F, int64_t n_dec,
                                int64_t in_stride, int64_t out_stride, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || n_dec < 0 || n_dec > 65535) return CLT_ERR_ARG;
  if (n_dec == 0) return CLT_OK;
  if (!w_ref || !w_packed) return CLT_ERR_ARG;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)clt_ceil_div(d, 64), (unsigned)n_dec);
  if (clt_ceil_div(d, 64) > 65535) return CLT_ERR_RANGE;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_pack<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)w_ref, (bf16_t *)w_packed, d, F, in_stride, out_stride);
  else k_pack<float><<<grid, 256, 0, s>>>((const float *)w_ref, (float *)w_packed, d, F, in_stride, out_stride);
  return clt_check_launch();
}

extern "C" int clt_densify(const int32_t *row_ptr, const int32_t *col, const void *val, void *out, int64_t T,
                           int64_t F, int64_t L, int64_t out_layer_stride, int dtype, int out_f32, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0) return CLT_ERR_ARG;
  if (T == 0 || F == 0) return CLT_OK;
  if (!row_ptr || !out) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int nb = 256 * 8;
  if (dtype == CLT_F32 || out_f32) k_zero_rows<float><<<nb, 256, 0, s>>>((float *)out, T, F, L, out_layer_stride);
  else k_zero_rows<bf16_t><<<nb, 256, 0, s>>>((bf16_t *)out, T, F, L, out_layer_stride);
  if (dtype == CLT_F32) k_densify_scatter<float, float><<<nb, 256, 0, s>>>(row_ptr, col, (const float *)val, (float *)out, T, F, L, out_layer_stride);
  else if (out_f32) k_densify_scatter<bf16_t, float><<<nb, 256, 0, s>>>(row_ptr, col, (const bf16_t *)val, (float *)out, T, F, L, out_layer_stride);
  else k_densify_scatter<bf16_t, bf16_t><<<nb, 256, 0, s>>>(row_ptr, col, (const bf16_t *)val, (bf16_t *)out, T, F, L, out_layer_stride);
  return clt_check_launch();
}

extern "C" int clt_decoder_norms(const void *w_packed, void *norms, int64_t d, int64_t F, int64_t L, int tying,
                                 int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || L <= 0 || tying < 0 || tying > 2 || !w_packed || !norms) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_norms<bf16_t><<<256 * 8, 256, 0, s>>>((const bf16_t *)w_packed, (bf16_t *)norms, d, F, L, tying);
  else k_norms<float><<<256 * 8, 256, 0, s>>>((const float *)w_packed, (float *)norms, d, F, L, tying);
  return clt_check_launch();
}
