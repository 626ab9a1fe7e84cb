// Backward pass of the forward path for the MSE reconstruction loss (reference
// clt/training/losses.py:45-92 through torch autograd: F.linear backward, the straight-through
// gate of BatchTopK, clt/models/activations.py:66-96).  Everything stays sparse:
//
//   loss / g      g[t] = 2 (rec[t] - target[t]) / (T d), per-layer mean squared error
//   values        d val[j] = sum over targets t >= s of  g[t][token] . W[s->t][feature]   for every
//                 survivor j = (s, token, feature): the gradient that reaches the encoder through
//                 the straight-through gate (zero for everything that was not selected)
//   feature lists the survivor list regrouped by (layer, feature): which tokens fired it
//   decoder dW    dW[s->t][feature][:] = sum over its tokens of  val * g[t][token][:]
//   encoder dW    dW_enc[s][feature][:] = sum over its tokens of  dval * x[s][token][:],
//                 db_enc[s][feature] = sum of dval
//   decoder db    db[t][:] = sum over tokens of g[t][token][:]
//
// Row vectors are spread over a wavefront in groups of four elements: lane l holds elements
// c * 256 + 4 l .. + 3 of chunk c (NC4 chunks cover d <= 4096; d % 4 == 0).
#include <type_traits>
#include "adam.h"

namespace {

constexpr int BW_THREADS = 256;

__device__ __forceinline__ int64_t bw_decoder_slot(int tying, int64_t s, int64_t t, int64_t L) {
  if (tying == CLT_TYING_PER_SOURCE) return s;
  if (tying == CLT_TYING_PER_TARGET) return t;
  return s * L - (s * (s - 1)) / 2 + (t - s);
}

template <typename T> __device__ __forceinline__ float4 load4(const T *p);
template <> __device__ __forceinline__ float4 load4<float>(const float *p) { return *reinterpret_cast<const float4 *>(p); }
template <> __device__ __forceinline__ float4 load4<bf16_t>(const bf16_t *p) {
  const uint2 u = *reinterpret_cast<const uint2 *>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xFFFF0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xFFFF0000u));
}

// 16 raw bytes of a row (EV = 8 bf16 or 4 fp32 elements) and their float values
template <typename T> struct Piece;
template <> struct Piece<float> {
  static constexpr int EV = 4;
  __device__ static __forceinline__ void unpack(const uint4 &w, float (&x)[4]) {
    x[0] = __uint_as_float(w.x); x[1] = __uint_as_float(w.y); x[2] = __uint_as_float(w.z); x[3] = __uint_as_float(w.w);
  }
};
template <> struct Piece<bf16_t> {
  static constexpr int EV = 8;
  __device__ static __forceinline__ void unpack(const uint4 &w, float (&x)[8]) {
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) { x[2 * j] = __uint_as_float(u[j] << 16); x[2 * j + 1] = __uint_as_float(u[j] & 0xFFFF0000u); }
  }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// ---- loss and its gradient -------------------------------------------------------------------
// loss_acc[l] += sum of squared differences (double); g[l][t][:] = d loss / d rec.
// The reference measures the loss on de-normalised tensors (clt/training/losses.py:70-86): with
// CLT_DENORM_MEAN_STD both sides become x * std + mean, with CLT_DENORM_SCALE x / scale, every step rounded
// to the model dtype as its tensor arithmetic is; the chain rule then puts a factor std (or 1 / scale) on
// the gradient: g = 2 (rec' - target') / (T d) * std.
template <typename T> __device__ __forceinline__ float bw_denorm(float x, int mode, float mean, float stdv, float scale) {
  if (mode == CLT_DENORM_MEAN_STD) return Elem<T>::round(Elem<T>::round(x * stdv) + mean);
  if (mode == CLT_DENORM_SCALE) return Elem<T>::round(x / scale);
  return x;
}

template <typename T>
__global__ __launch_bounds__(BW_THREADS) void k_mse_grad(const T *rec, const T *target, int64_t per_layer, int64_t d, float scale,
                                                          int mode, const T *mean, const T *stdv, float dscale,
                                                          float *g, T *g_model, double *loss_acc) {
  __shared__ double red[BW_THREADS / 64];
  const int l = blockIdx.y;
  const T *r = rec + (int64_t)l * per_layer, *y = target + (int64_t)l * per_layer;
  float *gl = g + (int64_t)l * per_layer;
  T *gm = g_model ? g_model + (int64_t)l * per_layer : nullptr;
  double acc = 0.0;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < per_layer; i += (int64_t)gridDim.x * blockDim.x * 4) {
    const float4 a = load4<T>(r + i), b = load4<T>(y + i);
    const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
    float dv[4], gv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (mode == CLT_DENORM_NONE) {
        dv[k] = av[k] - bv[k];
        gv[k] = scale * dv[k];
      } else {
        const int64_t c = (i + k) % d;
        const float mu = mode == CLT_DENORM_MEAN_STD ? Elem<T>::to_f32(mean[(int64_t)l * d + c]) : 0.0f;
        const float sd = mode == CLT_DENORM_MEAN_STD ? Elem<T>::to_f32(stdv[(int64_t)l * d + c]) : 1.0f;
        dv[k] = bw_denorm<T>(av[k], mode, mu, sd, dscale) - bw_denorm<T>(bv[k], mode, mu, sd, dscale);
        gv[k] = scale * dv[k] * (mode == CLT_DENORM_MEAN_STD ? sd : 1.0f / dscale);
      }
    }
    *reinterpret_cast<float4 *>(gl + i) = make_float4(gv[0], gv[1], gv[2], gv[3]);
    if (gm) { gm[i] = Elem<T>::from_f32(gv[0]); gm[i + 1] = Elem<T>::from_f32(gv[1]);
              gm[i + 2] = Elem<T>::from_f32(gv[2]); gm[i + 3] = Elem<T>::from_f32(gv[3]); }
    acc += (double)dv[0] * dv[0] + (double)dv[1] * dv[1] + (double)dv[2] * dv[2] + (double)dv[3] * dv[3];
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double s = 0.0;
    for (int i = 0; i < BW_THREADS / 64; ++i) s += red[i];
    atomicAdd(&loss_acc[l], s);
  }
}

__global__ void k_loss_finish(const double *loss_acc, int L, double inv_count, float *loss) {
  const int l = blockIdx.x * blockDim.x + threadIdx.x;
  if (l < L) loss[l] = (float)(loss_acc[l] * inv_count);
}

__global__ void k_zero_u32(uint32_t *p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0u;
}

__global__ void k_zero_f64(double *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.0;
}

// ---- column sums over tokens (decoder bias gradients), deterministic two-stage --------------------
constexpr int CS_SPLIT = 32;
__global__ __launch_bounds__(BW_THREADS) void k_colsum_partial(const float *g, int64_t Tn, int64_t d, float *part) {
  const int l = blockIdx.y, sp = blockIdx.z;
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= d) return;
  const int64_t per = (Tn + CS_SPLIT - 1) / CS_SPLIT, t0 = sp * per, t1 = t0 + per < Tn ? t0 + per : Tn;
  float acc = 0.0f;
  for (int64_t t = t0; t < t1; ++t) acc += g[((int64_t)l * Tn + t) * d + c];
  part[((int64_t)sp * gridDim.y + l) * d + c] = acc;
}
__global__ __launch_bounds__(BW_THREADS) void k_colsum_finish(const float *part, int64_t d, int L, float *out) {
  const int l = blockIdx.y;
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= d) return;
  float acc = 0.0f;
  for (int sp = 0; sp < CS_SPLIT; ++sp) acc += part[((int64_t)sp * L + l) * d + c];
  out[(int64_t)l * d + c] = acc;
}

// ---- gradient with respect to the survivor values ---------------------------------------------------
// sptr[r][j] = first survivor of row r whose feature index is >= j * F / ns  (j = 0..ns)
__global__ void k_bw_slice_ptr(const int32_t *row_ptr, const int32_t *col, int64_t R, int64_t F, int ns, int32_t *sptr) {
  const int64_t total = R * (ns + 1);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / (ns + 1);
    const int j = (int)(i - r * (ns + 1));
    const int32_t bound = (int32_t)(((int64_t)j * F) / ns);
    int32_t lo = row_ptr[r], hi = row_ptr[r + 1];
    while (lo < hi) {
      const int32_t mid = lo + ((hi - lo) >> 1);
      if (col[mid] < bound) lo = mid + 1; else hi = mid;
    }
    sptr[i] = lo;
  }
}

constexpr int BWV_XCDS = 8;    // feature slices = XCDs; workgroup b runs on XCD b % 8
constexpr int BWV_NTOK = 4;    // tokens per wavefront
constexpr int BWV_NU = 8;      // survivors whose decoder vectors are in flight together

// Sum of p[u] over the wavefront for BWV_NU values at once: three exchange steps that halve the
// values a lane keeps, then three steps on the one value left.  Afterwards lane l holds the
// total of value ((l >> 5) & 1) * 4 + ((l >> 4) & 1) * 2 + ((l >> 3) & 1).
__device__ __forceinline__ float wave_sum8(const float (&p)[BWV_NU], int lane) {
  float q4[4], q2[2], q1;
  const bool hi32 = lane & 32, hi16 = lane & 16, hi8 = lane & 8;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float keep = hi32 ? p[4 + i] : p[i], give = hi32 ? p[i] : p[4 + i];
    q4[i] = keep + __shfl_xor(give, 32);
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float keep = hi16 ? q4[2 + i] : q4[i], give = hi16 ? q4[i] : q4[2 + i];
    q2[i] = keep + __shfl_xor(give, 16);
  }
  {
    const float keep = hi8 ? q2[1] : q2[0], give = hi8 ? q2[0] : q2[1];
    q1 = keep + __shfl_xor(give, 8);
  }
  q1 += __shfl_xor(q1, 4);
  q1 += __shfl_xor(q1, 2);
  q1 += __shfl_xor(q1, 1);
  return q1;
}

// The same for four values: lane l ends up with the total of value ((l >> 5) & 1) * 2 + ((l >> 4) & 1).
__device__ __forceinline__ float wave_sum4(const float (&p)[4], int lane) {
  float q2[2], q1;
  const bool hi32 = lane & 32, hi16 = lane & 16;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const float keep = hi32 ? p[2 + i] : p[i], give = hi32 ? p[i] : p[2 + i];
    q2[i] = keep + __shfl_xor(give, 32);
  }
  {
    const float keep = hi16 ? q2[1] : q2[0], give = hi16 ? q2[0] : q2[1];
    q1 = keep + __shfl_xor(give, 16);
  }
  q1 += __shfl_xor(q1, 8);
  q1 += __shfl_xor(q1, 4);
  q1 += __shfl_xor(q1, 2);
  q1 += __shfl_xor(q1, 1);
  return q1;
}

// ... and for two: lane l ends up with the total of value (l >> 5) & 1.
__device__ __forceinline__ float wave_sum2(const float (&p)[2], int lane) {
  const bool hi32 = lane & 32;
  const float keep = hi32 ? p[1] : p[0], give = hi32 ? p[0] : p[1];
  float q1 = keep + __shfl_xor(give, 32);
  q1 += __shfl_xor(q1, 16);
  q1 += __shfl_xor(q1, 8);
  q1 += __shfl_xor(q1, 4);
  q1 += __shfl_xor(q1, 2);
  q1 += __shfl_xor(q1, 1);
  return q1;
}

// One wavefront per (source s, target t >= s, feature slice, BWV_NTOK tokens): like the forward
// gather, block b works on slice b % 8 and blocks are ordered (s, t)-pair-major, so an XCD gathers
// from one slice of one decoder matrix at a time.  part[t][j] = g[t][token] . W[s->t][feature of j].
// A row is read in 16-byte pieces (lane l: elements c * 64 EV + l EV ..., NCH pieces); the raw pieces
// of up to BWV_NU rows are in flight together, and BWV_NU dot products are reduced across the
// wavefront at once.
// T8: d = (NCH - 1) * 64 EV + 32 EV (768 in bf16): the last piece of a lane is 8 bytes wide and all 64 lanes
// take one, instead of a 16-byte piece that only the first 32 lanes have - no idle lanes in the loads and
// in the multiply-adds of the last piece.
template <typename T, int NCH, bool T8>
__global__ __launch_bounds__(BW_THREADS) void k_bwd_values_sliced(
    const int32_t *__restrict__ sptr, const int32_t *__restrict__ col, const T *__restrict__ wp,
    const float *__restrict__ g, int64_t Tn, int64_t d, int64_t F, int64_t L, int tying, int64_t nnz,
    float *__restrict__ part) {
  constexpr int EV = Piece<T>::EV;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int slice = (int)(blockIdx.x % BWV_XCDS);
  const int64_t bid = (int64_t)blockIdx.x / BWV_XCDS;
  const int64_t groups = (Tn + (int64_t)nwv * BWV_NTOK - 1) / ((int64_t)nwv * BWV_NTOK);
  const int64_t pair = bid / groups;
  const int64_t tok0 = ((bid - pair * groups) * nwv + wv) * BWV_NTOK;
  // pair -> (s, t): pairs are numbered like the untied decoder slots
  int64_t s = 0, rem = pair;
  while (rem >= L - s) { rem -= L - s; ++s; }
  const int64_t t = s + rem;
  const int64_t pitch = clt_pitch(d, (int)sizeof(T));
  const T *wbase = wp + bw_decoder_slot(tying, s, t, L) * F * pitch;
  float *pt = part + t * nnz;
  constexpr int NFULL = T8 ? NCH - 1 : NCH, HV = EV / 2;
  const int64_t tail_at = (int64_t)NFULL * 64 * EV + lane * HV;
  bool on[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) on[c] = (int64_t)c * 64 * EV + lane * EV < d;
  for (int i = 0; i < BWV_NTOK; ++i) {
    const int64_t tok = tok0 + i;
    if (tok >= Tn) break;
    const int64_t r = s * Tn + tok;
    const int32_t b = sptr[r * (BWV_XCDS + 1) + slice], e = sptr[r * (BWV_XCDS + 1) + slice + 1];
    if (b == e) continue;
    float gv[NCH][EV];
    if constexpr (T8) {
      const float4 v = *reinterpret_cast<const float4 *>(g + (t * Tn + tok) * d + tail_at);
      gv[NFULL][0] = v.x; gv[NFULL][1] = v.y; gv[NFULL][2] = v.z; gv[NFULL][3] = v.w;
    }
#pragma unroll
    for (int c = 0; c < NFULL; ++c)
#pragma unroll
      for (int q = 0; q < EV; q += 4) {
        const float4 v = on[c] ? *reinterpret_cast<const float4 *>(g + (t * Tn + tok) * d + (int64_t)c * 64 * EV + lane * EV + q)
                               : make_float4(0.f, 0.f, 0.f, 0.f);
        gv[c][q] = v.x; gv[c][q + 1] = v.y; gv[c][q + 2] = v.z; gv[c][q + 3] = v.w;
      }
    for (int32_t j0 = b; j0 < e; j0 += 64) {
      const int n = (e - j0) < 64 ? (e - j0) : 64;
      const int32_t my_col = lane < n ? col[j0 + lane] : 0;
      // dot products reduced together.  Narrow rows (d <= 1024 in bf16) run best with four: 79 registers, six
      // wavefronts per SIMD (eight: 105 registers, four wavefronts, 10 % slower; two: 6 % slower than four)
      constexpr int NUV = NCH <= 2 ? 4 : BWV_NU;
      constexpr int LB = NCH <= 2 ? NUV : NCH <= 4 ? BWV_NU / 2 : BWV_NU / 4;     // rows fetched together
      for (int i0 = 0; i0 < n; i0 += NUV) {
        float p[NUV];
#pragma unroll
        for (int h = 0; h < NUV; h += LB) {
          uint4 w[LB][NCH];
          uint2 wt[LB];
#pragma unroll
          for (int u = 0; u < LB; ++u) {
            const int idx = i0 + h + u < n ? i0 + h + u : n - 1;
            const T *wrow = wbase + (int64_t)__builtin_amdgcn_readlane(my_col, idx) * pitch;
#pragma unroll
            for (int c = 0; c < NFULL; ++c)
              w[u][c] = on[c] ? *reinterpret_cast<const uint4 *>(wrow + (int64_t)c * 64 * EV + lane * EV) : make_uint4(0, 0, 0, 0);
            if constexpr (T8) wt[u] = *reinterpret_cast<const uint2 *>(wrow + tail_at);
          }
#pragma unroll
          for (int u = 0; u < LB; ++u) {
            float a = 0.0f;
#pragma unroll
            for (int c = 0; c < NFULL; ++c) {
              float x[EV];
              Piece<T>::unpack(w[u][c], x);
#pragma unroll
              for (int q = 0; q < EV; ++q) a = fmaf(x[q], gv[c][q], a);
            }
            if constexpr (T8 && sizeof(T) == 2) {
              a = fmaf(__uint_as_float(wt[u].x << 16), gv[NFULL][0], a);
              a = fmaf(__uint_as_float(wt[u].x & 0xFFFF0000u), gv[NFULL][1], a);
              a = fmaf(__uint_as_float(wt[u].y << 16), gv[NFULL][2], a);
              a = fmaf(__uint_as_float(wt[u].y & 0xFFFF0000u), gv[NFULL][3], a);
            }
            p[h + u] = a;
          }
        }
        if constexpr (NUV == 8) {
          const float tot = wave_sum8(p, lane);
          const int u = ((lane >> 5) & 1) * 4 + ((lane >> 4) & 1) * 2 + ((lane >> 3) & 1);
          if ((lane & 7) == 0 && i0 + u < n) pt[j0 + i0 + u] = tot;
        } else if constexpr (NUV == 4) {
          const float tot = wave_sum4(p, lane);
          const int u = ((lane >> 5) & 1) * 2 + ((lane >> 4) & 1);
          if ((lane & 15) == 0 && i0 + u < n) pt[j0 + i0 + u] = tot;
        } else {
          const float tot = wave_sum2(p, lane);
          const int u = (lane >> 5) & 1;
          if ((lane & 31) == 0 && i0 + u < n) pt[j0 + i0 + u] = tot;
        }
      }
    }
  }
}

// dval[j] = sum over the targets t >= s of part[t][j], in target order; one wavefront per row.
// With a feature scale (tied decoders, decoder.py:228-285) target t saw the activation times
// fscale[t][feature] (non-zero activations only), so its share of the gradient carries that factor.
template <typename T>
__global__ __launch_bounds__(BW_THREADS) void k_bwd_values_sum(const int32_t *row_ptr, const float *part, int64_t Tn,
                                                                int64_t L, int64_t nnz, uint64_t src_mask, float *dval,
                                                                const int32_t *col, const T *val, const T *fscale, int64_t F) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t R = L * Tn;
  for (int64_t r = (int64_t)blockIdx.x * nwv + wv; r < R; r += (int64_t)gridDim.x * nwv) {
    const int64_t s = r / Tn;
    const bool on = (src_mask >> s) & 1ull;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) {
      float acc = 0.0f;
      if (on && fscale) {
        const int64_t f = col[j];
        const bool nz = Elem<T>::to_f32(val[j]) != 0.0f;
        for (int64_t t = s; t < L; ++t) acc += part[t * nnz + j] * (nz ? Elem<T>::to_f32(fscale[t * F + f]) : 1.0f);
      } else if (on) {
        // four loads in flight; the additions keep the target order
        int64_t t = s;
        for (; t + 4 <= L; t += 4) {
          const float p0 = part[t * nnz + j], p1 = part[(t + 1) * nnz + j], p2 = part[(t + 2) * nnz + j], p3 = part[(t + 3) * nnz + j];
          acc += p0; acc += p1; acc += p2; acc += p3;
        }
        for (; t < L; ++t) acc += part[t * nnz + j];
      }
      dval[j] = acc;
    }
  }
}

// Gradients of the per-target feature offset / scale of tied decoders (decoder.py:228-245, 268-285).  Target t
// sees a' = (a + off[t][f]) * scale[t][f] for the non-zero activations a of feature f in the sources s <= t; with
// h = d loss / d a' (= part[t][j], the dot product of the loss gradient with the decoder row):
//   d off[t][f]   = scale[t][f] * sum h          d scale[t][f] = sum h * (a + off[t][f])
// One wavefront per (target, feature) walks the token-ordered lists of (s, f), s <= t: fixed summation order.
template <typename T>
__global__ __launch_bounds__(BW_THREADS) void k_affine_grad(const int32_t *__restrict__ ptr, const int32_t *__restrict__ lsrc,
                                                             const T *__restrict__ val, const float *__restrict__ part,
                                                             const T *__restrict__ foff, const T *__restrict__ fscale,
                                                             int64_t F, int64_t L, int64_t nnz, uint64_t src_mask,
                                                             float *__restrict__ doff, float *__restrict__ dscale) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t total = L * F;
  for (int64_t w = (int64_t)blockIdx.x * nwv + wv; w < total; w += (int64_t)gridDim.x * nwv) {
    const int64_t t = w / F, f = w - t * F;
    const float off = foff ? Elem<T>::to_f32(foff[w]) : 0.0f, sc = fscale ? Elem<T>::to_f32(fscale[w]) : 1.0f;
    float a_sum = 0.0f, b_sum = 0.0f;
    for (int64_t s = 0; s <= t; ++s) {
      if (!((src_mask >> s) & 1ull)) continue;
      const int32_t b = ptr[s * F + f], e = ptr[s * F + f + 1];
      for (int32_t i = b + lane; i < e; i += 64) {
        const int32_t j = lsrc[i];
        const float a = Elem<T>::to_f32(val[j]);
        if (a != 0.0f) {
          const float h = part[t * nnz + j];
          a_sum += h;
          b_sum += h * (foff ? Elem<T>::round(a + off) : a);
        }
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { a_sum += __shfl_xor(a_sum, o); b_sum += __shfl_xor(b_sum, o); }
    if (lane == 0) {
      if (doff) doff[w] = sc * a_sum;
      if (dscale) dscale[w] = b_sum;
    }
  }
}

// Skip-connection weight gradient (decoder.py:297-338: rec += x @ W_skip.T): out[i][j] (+)= sum over tokens of
// g[tok][i] * x[tok][j].  A block owns a 64 x 64 tile of the [d, d] result and walks all tokens, 16 at a time
// through LDS; a thread owns a 4 x 4 piece.  Tokens in order: the same bits every run.
constexpr int SK_TOK = 16;
template <typename T>
__global__ __launch_bounds__(256) void k_skip_grad(const float *__restrict__ g, const T *__restrict__ x, float *__restrict__ out,
                                                   int64_t Tn, int64_t d, int accumulate) {
  __shared__ float gs[SK_TOK][64], xs[SK_TOK][64];
  const int i0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
  const int ti = (threadIdx.x >> 4) * 4, tj = (threadIdx.x & 15) * 4;
  float acc[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) acc[a][b] = 0.0f;
  for (int64_t t0 = 0; t0 < Tn; t0 += SK_TOK) {
    for (int e = threadIdx.x; e < SK_TOK * 64; e += 256) {
      const int tt = e >> 6, c = e & 63;
      const int64_t tok = t0 + tt;
      gs[tt][c] = (tok < Tn && i0 + c < d) ? g[tok * d + i0 + c] : 0.0f;
      xs[tt][c] = (tok < Tn && j0 + c < d) ? Elem<T>::to_f32(x[tok * d + j0 + c]) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < SK_TOK; ++tt) {
      float gv[4], xv[4];
#pragma unroll
      for (int a = 0; a < 4; ++a) { gv[a] = gs[tt][ti + a]; xv[a] = xs[tt][tj + a]; }
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = fmaf(gv[a], xv[b], acc[a][b]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int64_t i = i0 + ti + a, j = j0 + tj + b;
      if (i < d && j < d) out[i * d + j] = accumulate ? out[i * d + j] + acc[a][b] : acc[a][b];
    }
}

// ---- feature lists: the survivor list regrouped by (layer, feature) ----------------------------------
__global__ __launch_bounds__(BW_THREADS) void k_csc_count(const int32_t *row_ptr, const int32_t *col, int64_t Tn, int64_t F,
                                                           int64_t L, uint32_t *cnt) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t R = L * Tn;
  for (int64_t r = (int64_t)blockIdx.x * nwv + wv; r < R; r += (int64_t)gridDim.x * nwv) {
    const int64_t l = r / Tn;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) atomicAdd(&cnt[l * F + col[j]], 1u);
  }
}

// ptr = exclusive scan of cnt (n entries), ptr[n] = total; cnt is reset to zero (it serves as the
// fill cursor next).  Three steps over chunks of CSC_CHUNK counters: chunk sums, a scan of the
// sums in one block, and the scan inside every chunk from its offset; all accesses coalesced.
constexpr int CSC_CHUNK = 4096;
__global__ __launch_bounds__(BW_THREADS) void k_csc_chunk_sum(const uint32_t *cnt, int64_t n, unsigned long long *sums) {
  __shared__ unsigned long long red[BW_THREADS / 64];
  const int64_t base = (int64_t)blockIdx.x * CSC_CHUNK;
  unsigned long long s = 0;
  for (int i = threadIdx.x; i < CSC_CHUNK; i += BW_THREADS)
    if (base + i < n) s += cnt[base + i];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    unsigned long long t = 0;
    for (int i = 0; i < BW_THREADS / 64; ++i) t += red[i];
    sums[blockIdx.x] = t;
  }
}
// one block: sums -> exclusive offsets in place; ptr[n] = total
__global__ __launch_bounds__(BW_THREADS) void k_csc_chunk_offsets(unsigned long long *sums, int64_t nchunk, int32_t *ptr, int64_t n) {
  __shared__ unsigned long long wsum[BW_THREADS / 64];
  __shared__ unsigned long long carry_s;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (threadIdx.x == 0) carry_s = 0;
  __syncthreads();
  for (int64_t b0 = 0; b0 < nchunk; b0 += BW_THREADS) {
    const int64_t i = b0 + threadIdx.x;
    const unsigned long long v = i < nchunk ? sums[i] : 0;
    unsigned long long inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const unsigned long long y = __shfl_up(inc, o);
      if (lane >= o) inc += y;
    }
    if (lane == 63) wsum[wv] = inc;
    __syncthreads();
    unsigned long long before = carry_s, total = 0;
    for (int k = 0; k < BW_THREADS / 64; ++k) { if (k < wv) before += wsum[k]; total += wsum[k]; }
    if (i < nchunk) sums[i] = before + inc - v;
    __syncthreads();
    if (threadIdx.x == 0) carry_s += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) ptr[n] = (int32_t)carry_s;
}
__global__ __launch_bounds__(BW_THREADS) void k_csc_chunk_scan(uint32_t *cnt, int64_t n, const unsigned long long *offsets,
                                                                int32_t *ptr) {
  __shared__ uint32_t wsum[BW_THREADS / 64];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t base = (int64_t)blockIdx.x * CSC_CHUNK;
  unsigned long long carry = offsets[blockIdx.x];
  for (int it = 0; it < CSC_CHUNK / BW_THREADS; ++it) {
    const int64_t i = base + (int64_t)it * BW_THREADS + threadIdx.x;
    const uint32_t v = i < n ? cnt[i] : 0u;
    uint32_t inc = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const uint32_t y = __shfl_up(inc, o);
      if (lane >= o) inc += y;
    }
    if (lane == 63) wsum[wv] = inc;
    __syncthreads();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int k = 0; k < BW_THREADS / 64; ++k) { if (k < wv) before += wsum[k]; total += wsum[k]; }
    if (i < n) { ptr[i] = (int32_t)(carry + before + inc - v); cnt[i] = 0u; }
    carry += total;
    __syncthreads();
  }
}

__global__ __launch_bounds__(BW_THREADS) void k_csc_fill(const int32_t *row_ptr, const int32_t *col, int64_t Tn, int64_t F,
                                                          int64_t L, const int32_t *ptr, uint32_t *cursor, int32_t *tok_out,
                                                          int32_t *src_out) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t R = L * Tn;
  for (int64_t r = (int64_t)blockIdx.x * nwv + wv; r < R; r += (int64_t)gridDim.x * nwv) {
    const int64_t l = r / Tn, tok = r - l * Tn;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) {
      const int64_t key = l * F + col[j];
      const uint32_t pos = atomicAdd(&cursor[key], 1u);
      tok_out[ptr[key] + pos] = (int32_t)tok;
      src_out[ptr[key] + pos] = j;
    }
  }
}

// Every list is put in token order (the fill order depends on scheduling), so that the sums over a list
// always run in the same order and the weight gradients are the same bits from run to run.
//   up to 64 entries: one entry per lane, rank = number of smaller tokens;
//   longer lists: the tokens of a list are distinct, so the list is a set of tokens: the wavefront marks them in
//   a bitmap in LDS (T bits), takes prefix popcounts over its words, and then walks the WORDS, not the entries:
//   the i-th set bit is the i-th token.  The position of the survivor in col / val is looked up again in its row
//   (the columns of a row ascend), so nothing is read from the arrays that are being rewritten.
// LDS per wavefront: 2 * ceil(T / 32) words (dynamic shared memory, bm_words = ceil(T / 32)).
__global__ __launch_bounds__(BW_THREADS) void k_csc_order(const int32_t *ptr, int64_t nlist, int32_t *tok, int32_t *src,
                                                           const int32_t *row_ptr, const int32_t *col, int64_t Tn, int64_t F,
                                                           int bm_words) {
  extern __shared__ uint32_t order_lds[];
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  uint32_t *bm = order_lds + (size_t)wv * 2 * bm_words, *pfx = bm + bm_words;
  for (int64_t q = (int64_t)blockIdx.x * nwv + wv; q < nlist; q += (int64_t)gridDim.x * nwv) {
    const int32_t b = ptr[q], n = ptr[q + 1] - b;
    if (n < 2) continue;
    if (n <= 64) {
      const int32_t mt = lane < n ? tok[b + lane] : 0x7FFFFFFF, ms = lane < n ? src[b + lane] : 0;
      int rank = 0;
      for (int i = 0; i < n; ++i) rank += __builtin_amdgcn_readlane(mt, i) < mt ? 1 : 0;   // tokens of one list are distinct
      if (lane < n) { tok[b + rank] = mt; src[b + rank] = ms; }
      continue;
    }
    const int64_t l = q / F, f = q - l * F;
    for (int w = lane; w < bm_words; w += 64) bm[w] = 0u;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    for (int32_t i = lane; i < n; i += 64) {
      const int32_t tk = tok[b + i];
      atomicOr(&bm[tk >> 5], 1u << (tk & 31));
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    // exclusive prefix popcounts over the words, 64 words at a time
    uint32_t carry = 0;
    for (int w0 = 0; w0 < bm_words; w0 += 64) {
      const int w = w0 + lane;
      const uint32_t c = w < bm_words ? (uint32_t)__popc(bm[w]) : 0u;
      uint32_t inc = c;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const uint32_t y = __shfl_up(inc, o);
        if (lane >= o) inc += y;
      }
      if (w < bm_words) pfx[w] = carry + inc - c;
      carry += __shfl(inc, 63);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    for (int w = lane; w < bm_words; w += 64) {
      uint32_t bits = bm[w];
      int32_t pos = b + (int32_t)pfx[w];
      while (bits) {
        const int32_t tk = w * 32 + (__ffs(bits) - 1);
        bits &= bits - 1u;
        // the survivor (layer l, token tk, feature f): its place in the row's ascending columns
        const int64_t r = l * Tn + tk;
        int32_t lo = row_ptr[r], hi = row_ptr[r + 1];
        while (lo < hi) {
          const int32_t mid = lo + ((hi - lo) >> 1);
          if (col[mid] < (int32_t)f) lo = mid + 1; else hi = mid;
        }
        tok[pos] = tk; src[pos] = lo;
        ++pos;
      }
    }
  }
}

// ---- the same lists without device-scope atomics and without the sort -----------------------------------
// The tokens of a layer are cut into NB blocks; workgroup (layer, block) keeps one counter per feature in LDS.
//   k_fl_count: histogram of the block's entries (LDS atomics: only counts, the order does not matter);
//   k_fl_total: list length = sum over the blocks (the counts become running sums over the blocks), then the
//               chunked scan above gives list_ptr;
//   k_fl_fill:  LDS counter f starts where the block's part of list (layer, f) starts (list_ptr plus the entries
//               in earlier blocks) and the block's tokens are taken ONE AFTER THE OTHER: the columns of a
//               row are distinct, so within one token no two threads touch the same counter and a plain read /
//               increment gives every entry its place -- in token order by construction.
// Needs F counters of LDS (F <= 35 K); longer feature axes take the atomic route above.
constexpr int FL_THREADS = 512, FL_MAX_BLOCKS = 64, FL_MIN_BLOCK_TOKENS = 64, FL_MIN_CAP = 1024, FL_MAX_CAP = 16384;
constexpr int64_t FL_LDS_MAX = 150 * 1024;
__global__ __launch_bounds__(FL_THREADS) void k_fl_count(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col,
                                                          int64_t Tn, int64_t F, int TB, int NB, uint16_t *__restrict__ counts,
                                                          int64_t n) {
  extern __shared__ uint32_t fl_lds[];
  const int64_t l = blockIdx.x / NB, b = blockIdx.x % NB;
  for (int64_t f = threadIdx.x; f < F; f += FL_THREADS) fl_lds[f] = 0u;
  __syncthreads();
  const int64_t t0 = b * TB, t1 = t0 + TB < Tn ? t0 + TB : Tn;
  if (t0 < t1) {
    const int32_t e0 = row_ptr[l * Tn + t0], e1 = row_ptr[l * Tn + t1];
    for (int32_t j0 = e0 + (int32_t)threadIdx.x; j0 < e1; j0 += 8 * FL_THREADS) {
      int32_t c[8];       // eight loads in flight per thread
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = j0 + u * FL_THREADS < e1 ? col[j0 + u * FL_THREADS] : -1;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (c[u] >= 0) atomicAdd(&fl_lds[c[u]], 1u);
    }
  }
  __syncthreads();
  uint16_t *out = counts + b * n + l * F;
  for (int64_t f = threadIdx.x; f < F; f += FL_THREADS) out[f] = (uint16_t)fl_lds[f];    // <= TB <= 1024
}
// counts[b][q] -> number of entries of list q in the blocks before b (at most T <= 65535), cnt[q] = list length
__global__ __launch_bounds__(BW_THREADS) void k_fl_total(uint16_t *counts, int NB, int64_t n, uint32_t *__restrict__ cnt) {
  for (int64_t q = (int64_t)blockIdx.x * BW_THREADS + threadIdx.x; q < n; q += (int64_t)gridDim.x * BW_THREADS) {
    uint32_t a = 0;
    for (int b0 = 0; b0 < NB; b0 += 16) {
      uint16_t c[16];       // sixteen independent loads, then the stores over them
#pragma unroll
      for (int u = 0; u < 16; ++u) c[u] = b0 + u < NB ? counts[(int64_t)(b0 + u) * n + q] : (uint16_t)0;
#pragma unroll
      for (int u = 0; u < 16; ++u)
        if (b0 + u < NB) { counts[(int64_t)(b0 + u) * n + q] = (uint16_t)a; a += c[u]; }
    }
    cnt[q] = a;
  }
}
__global__ __launch_bounds__(FL_THREADS) void k_fl_fill(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col,
                                                         int64_t Tn, int64_t F, int TB, int NB,
                                                         const uint16_t *__restrict__ counts, int64_t n,
                                                         const int32_t *__restrict__ ptr, int32_t *__restrict__ tok_out,
                                                         int32_t *__restrict__ src_out, int cap) {
  extern __shared__ uint32_t fl_lds[];
  uint32_t *pos = fl_lds;
  uint32_t *buf = fl_lds + F;                               // cap staged entries: column index, then place
  uint16_t *tk = reinterpret_cast<uint16_t *>(buf + cap);   // their tokens, counted from the batch's first
  int32_t *rp = reinterpret_cast<int32_t *>(buf + cap + cap / 2);   // the block's row pointers, TB + 1 of them
  const int64_t l = blockIdx.x / NB, b = blockIdx.x % NB;
  const int64_t t0 = b * TB, t1 = t0 + TB < Tn ? t0 + TB : Tn;
  if (t0 >= t1) return;
  const int ntok = (int)(t1 - t0), tid = (int)threadIdx.x;
  for (int64_t f0 = tid; f0 < F; f0 += 8 * FL_THREADS) {
    uint32_t base[8];     // start of the list + its entries in earlier blocks; eight pairs of loads in flight
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t f = f0 + u * FL_THREADS, q = l * F + f;
      base[u] = f < F ? (uint32_t)ptr[q] + counts[b * n + q] : 0u;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (f0 + u * FL_THREADS < F) pos[f0 + u * FL_THREADS] = base[u];
  }
  for (int i = tid; i <= ntok; i += FL_THREADS) rp[i] = row_ptr[l * Tn + t0 + i];
  __syncthreads();
  // Batches of whole tokens whose entries fit the staging buffer (a row longer than the buffer goes in pieces).
  //   A: the batch's column indices come into LDS (one wait for memory per batch);
  //   B: token after token, every entry swaps its column index for its place in the output -- LDS traffic
  //      only, with a barrier that waits for LDS alone between two tokens;
  //   C: the entries are scattered to their places (no order to keep any more).
  auto lds_barrier = [] {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  int tb = 0;
  while (tb < ntok) {
    const int32_t eb = rp[tb];
    int te = tb + 1;
    while (te < ntok && rp[te + 1] - eb <= cap) ++te;
    int32_t ee = rp[te];
    const bool cut = ee - eb > cap;      // one row longer than the buffer: its first cap entries now
    if (cut) ee = eb + cap;
    const int nb_e = ee - eb;
    for (int i0 = tid; i0 < nb_e; i0 += 8 * FL_THREADS) {
      uint32_t c[8];      // eight loads in flight per thread
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = i0 + u * FL_THREADS < nb_e ? (uint32_t)col[eb + i0 + u * FL_THREADS] : 0u;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (i0 + u * FL_THREADS < nb_e) buf[i0 + u * FL_THREADS] = c[u];
    }
    __syncthreads();
    for (int t = tb; t < te; ++t) {
      const int a0 = rp[t] - eb, a1 = (rp[t + 1] < ee ? rp[t + 1] : ee) - eb;
      for (int i = a0 + tid; i < a1; i += FL_THREADS) {
        const uint32_t f = buf[i], p = pos[f];
        pos[f] = p + 1u;
        buf[i] = p;
        tk[i] = (uint16_t)(t - tb);
      }
      lds_barrier();      // the next token may meet the same features
    }
    for (int i = tid; i < nb_e; i += FL_THREADS) {
      const uint32_t p = buf[i];
      tok_out[p] = (int32_t)(t0 + tb + tk[i]);
      src_out[p] = eb + i;
    }
    __syncthreads();      // buf, tk and rp[tb] are free again
    if (cut) {
      if (tid == 0) rp[tb] = ee;
      __syncthreads();
    } else {
      tb = te;
    }
  }
}

// ---- weight gradients: one wavefront per output row ---------------------------------------------------
// out_row[:] = sum over the list of (layer, feature) of coef[entry] * src[token][:]
//   DECODER: wavefront (s, f, t >= s): coef = survivor value, src = g[t] (model dtype copy),
//            out = dW[slot(s,t)][f]
//   encoder: wavefront (s, f):         coef = dval, src = x[s], out = dW_enc[s][f], rowsum = db_enc[s][f]
// Rows are read in raw 16-byte pieces, up to FO_NU rows in flight.
// (Cutting the columns in two over XCD pairs, so that each XCD gathers from half a [T, d] matrix that
// fits its L2, was measured and dropped: with four rows in flight per wavefront whole rows are 8 % faster.)
constexpr int FO_NU = 8;
// T8: as in k_bwd_values_sliced, the last piece of a lane is 8 bytes wide and every lane has one.
// ADAM (untied decoders only): the row is not written; it is the gradient of an Adam step applied on the
// spot to the moments [n_dec][F][d] and to the feature-major working copy [n_dec][F][pitch] of the decoder.
struct AdamInPlace {
  float *m, *v;      // moments, dense like the gradient would be
  void *w_packed;    // the decoders' working copy
  int64_t pitch;
  AdamCoef c;
};
template <typename T, typename CoefT, int NCH, bool DECODER, bool T8 = false, bool ADAM = false>
__global__ __launch_bounds__(BW_THREADS) void k_feature_outer(
    const int32_t *__restrict__ ptr, const int32_t *__restrict__ ltok, const int32_t *__restrict__ lsrc,
    const CoefT *__restrict__ coef, const T *__restrict__ src, float *__restrict__ out, float *__restrict__ rowsum,
    int64_t Tn, int64_t d, int64_t F, int64_t L, int64_t target, int tying, const T *__restrict__ foff = nullptr,
    const T *__restrict__ fscale = nullptr, AdamInPlace ad = AdamInPlace()) {
  static_assert(!ADAM || DECODER, "the in-place step is for decoder rows");
  constexpr int EV = Piece<T>::EV;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  // One launch per layer of the gathered matrix, so that every wavefront of a launch gathers from the
  // same [T, d] matrix: DECODER launch `target` covers the (source <= target, feature) pairs and reads
  // g[target]; the encoder launch `target` covers the features of that layer and reads x[target].
  // Tied decoders: one matrix per source collects its targets over the launches (the launch
  // target == source writes the row, later launches add to it: launches must run in ascending
  // target order on one stream); one matrix per target sums the lists of all sources <= target
  // inside the wavefront.
  const bool per_target = DECODER && tying == CLT_TYING_PER_TARGET;
  const int64_t total = (DECODER && !per_target) ? (target + 1) * F : F;
  const int64_t vblock = (int64_t)blockIdx.x, nvblock = (int64_t)gridDim.x;
  const int64_t my_pieces = d / EV;
  constexpr int NFULL = T8 ? NCH - 1 : NCH, HV = EV / 2;
  const int64_t tail_at = (int64_t)NFULL * 64 * EV + lane * HV;
  bool on[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) on[c] = (int64_t)c * 64 + lane < my_pieces;
  for (int64_t w = vblock * nwv + wv; w < total; w += nvblock * nwv) {
    const int64_t s = (DECODER && !per_target) ? w / F : target, f = (DECODER && !per_target) ? w - s * F : w, t = target;
    const T *sbase = src + (DECODER ? t : s) * Tn * d;
    float acc[NCH][EV];
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
      for (int k = 0; k < EV; ++k) acc[c][k] = 0.0f;
    float csum = 0.0f;
    // ADAM: the row's moments and parameters are asked for now (streaming: they pass through once and must
    // not push the gathered rows out of the L2) and arrive while the row's gradient is being summed
    typedef float bw_f4 __attribute__((ext_vector_type(4)));
    typedef uint32_t bw_u2 __attribute__((ext_vector_type(2)));
    typedef uint32_t bw_u4 __attribute__((ext_vector_type(4)));
    constexpr int NG = ADAM ? NFULL * (EV / 4) + (T8 ? 1 : 0) : 1;
    bw_f4 am[NG], av[NG];
    typename std::conditional<sizeof(T) == 2, bw_u2, bw_u4>::type aw[NG];
    float *mrow = nullptr, *vrow = nullptr;
    T *wrow = nullptr;
    if constexpr (ADAM) {
      const int64_t rowi = bw_decoder_slot(tying, s, t, L) * F + f;
      mrow = ad.m + rowi * d; vrow = ad.v + rowi * d;
      wrow = reinterpret_cast<T *>(ad.w_packed) + rowi * ad.pitch;
      auto ask4 = [&](int gi, int64_t at) {
        am[gi] = __builtin_nontemporal_load(reinterpret_cast<const bw_f4 *>(mrow + at));
        av[gi] = __builtin_nontemporal_load(reinterpret_cast<const bw_f4 *>(vrow + at));
        aw[gi] = __builtin_nontemporal_load(reinterpret_cast<const decltype(aw[0] + aw[0]) *>(wrow + at));
      };
      int gi = 0;
      if constexpr (T8) ask4(gi++, tail_at);
#pragma unroll
      for (int c = 0; c < NFULL; ++c)
#pragma unroll
        for (int k = 0; k < EV; k += 4) {
          if (on[c]) ask4(gi, (int64_t)c * 64 * EV + lane * EV + k);
          ++gi;
        }
    }
    for (int64_t ls = per_target ? 0 : s; ls <= s; ++ls) {
    const int64_t q = ls * F + f;
    const int32_t b = ptr[q], e = ptr[q + 1];
    for (int32_t i0 = b; i0 < e; i0 += 64) {
      const int n = (e - i0) < 64 ? (e - i0) : 64;
      int32_t mt = 0; float mc = 0.0f;
      if (lane < n) { mt = ltok[i0 + lane]; mc = Elem<CoefT>::to_f32(coef[lsrc[i0 + lane]]); }
      if (DECODER && (foff || fscale) && mc != 0.0f) {
        // the target's feature offset / scale: what this decoder was multiplied with (decoder.py:228-245)
        if (foff) mc = Elem<T>::round(mc + Elem<T>::to_f32(foff[t * F + f]));
        if (fscale) mc = Elem<T>::round(mc * Elem<T>::to_f32(fscale[t * F + f]));
      }
      // rows in flight.  Narrow rows (d <= 1024 in bf16) run best with four: 55 registers, eight wavefronts per
      // SIMD (eight in flight, six wavefronts: 11 % slower); wide rows keep about 16 pieces per lane
      constexpr int NU = NCH <= 4 ? FO_NU / 2 : FO_NU / 4;
      for (int i = 0; i < n; i += NU) {
        uint4 v[NU][NCH];
        uint2 vt[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u) {
          const int idx = i + u < n ? i + u : n - 1;
          const T *row = sbase + (int64_t)__builtin_amdgcn_readlane(mt, idx) * d;
#pragma unroll
          for (int c = 0; c < NFULL; ++c)
            v[u][c] = on[c] ? *reinterpret_cast<const uint4 *>(row + (int64_t)c * 64 * EV + lane * EV) : make_uint4(0, 0, 0, 0);
          if constexpr (T8) vt[u] = *reinterpret_cast<const uint2 *>(row + tail_at);
        }
#pragma unroll
        for (int u = 0; u < NU; ++u) {
          const int idx = i + u < n ? i + u : n - 1;
          const float cf = i + u < n ? __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(mc), idx)) : 0.0f;
          csum += cf;
#pragma unroll
          for (int c = 0; c < NFULL; ++c) {
            float x[EV];
            Piece<T>::unpack(v[u][c], x);
#pragma unroll
            for (int k = 0; k < EV; ++k) acc[c][k] = fmaf(cf, x[k], acc[c][k]);
          }
          if constexpr (T8 && sizeof(T) == 2) {
            acc[NFULL][0] = fmaf(cf, __uint_as_float(vt[u].x << 16), acc[NFULL][0]);
            acc[NFULL][1] = fmaf(cf, __uint_as_float(vt[u].x & 0xFFFF0000u), acc[NFULL][1]);
            acc[NFULL][2] = fmaf(cf, __uint_as_float(vt[u].y << 16), acc[NFULL][2]);
            acc[NFULL][3] = fmaf(cf, __uint_as_float(vt[u].y & 0xFFFF0000u), acc[NFULL][3]);
          }
        }
      }
    }
    }
    const int64_t q = s * F + f;
    if constexpr (ADAM) {
      // groups of four elements, as they were asked for ahead of the gather
      auto step4 = [&](int gi, int64_t at, const float *gk) {
        float mm[4] = {am[gi].x, am[gi].y, am[gi].z, am[gi].w}, vv[4] = {av[gi].x, av[gi].y, av[gi].z, av[gi].w}, pp[4];
        if constexpr (sizeof(T) == 2) {
          pp[0] = __uint_as_float(aw[gi].x << 16); pp[1] = __uint_as_float(aw[gi].x & 0xFFFF0000u);
          pp[2] = __uint_as_float(aw[gi].y << 16); pp[3] = __uint_as_float(aw[gi].y & 0xFFFF0000u);
        } else {
          pp[0] = __uint_as_float(aw[gi].x); pp[1] = __uint_as_float(aw[gi].y);
          pp[2] = __uint_as_float(aw[gi].z); pp[3] = __uint_as_float(aw[gi].w);
        }
        T np[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) np[k] = Elem<T>::from_f32(adam_update(pp[k], gk[k], mm[k], vv[k], ad.c));
        bw_f4 mo = {mm[0], mm[1], mm[2], mm[3]}, vo = {vv[0], vv[1], vv[2], vv[3]};
        __builtin_nontemporal_store(mo, reinterpret_cast<bw_f4 *>(mrow + at));
        __builtin_nontemporal_store(vo, reinterpret_cast<bw_f4 *>(vrow + at));
        if constexpr (sizeof(T) == 2) {
          bw_u2 wo = {(uint32_t)Elem<T>::raw(np[0]) | ((uint32_t)Elem<T>::raw(np[1]) << 16),
                      (uint32_t)Elem<T>::raw(np[2]) | ((uint32_t)Elem<T>::raw(np[3]) << 16)};
          __builtin_nontemporal_store(wo, reinterpret_cast<bw_u2 *>(wrow + at));
        } else {
          bw_f4 wo = {(float)np[0], (float)np[1], (float)np[2], (float)np[3]};
          __builtin_nontemporal_store(wo, reinterpret_cast<bw_f4 *>(wrow + at));
        }
      };
      int gi = 0;
      if constexpr (T8) step4(gi++, tail_at, acc[NFULL]);
#pragma unroll
      for (int c = 0; c < NFULL; ++c)
#pragma unroll
        for (int k = 0; k < EV; k += 4) {
          if (on[c]) step4(gi, (int64_t)c * 64 * EV + lane * EV + k, &acc[c][k]);
          ++gi;
        }
      continue;
    }
    float *orow = out + (DECODER ? (bw_decoder_slot(tying, s, t, L) * F + f) : q) * d;
    const bool add = DECODER && tying == CLT_TYING_PER_SOURCE && t > s;
    if constexpr (T8) {
      float4 *dst = reinterpret_cast<float4 *>(orow + tail_at);
      float4 r = make_float4(acc[NFULL][0], acc[NFULL][1], acc[NFULL][2], acc[NFULL][3]);
      if (add) { const float4 o = *dst; r.x += o.x; r.y += o.y; r.z += o.z; r.w += o.w; }
      *dst = r;
    }
#pragma unroll
    for (int c = 0; c < NFULL; ++c)
      if (on[c]) {
#pragma unroll
        for (int k = 0; k < EV; k += 4) {
          float4 *dst = reinterpret_cast<float4 *>(orow + (int64_t)c * 64 * EV + lane * EV + k);
          float4 r = make_float4(acc[c][k], acc[c][k + 1], acc[c][k + 2], acc[c][k + 3]);
          if (add) { const float4 o = *dst; r.x += o.x; r.y += o.y; r.z += o.z; r.w += o.w; }
          *dst = r;
        }
      }
    if (!DECODER && rowsum && lane == 0) rowsum[q] = csum;
  }
}


// Grid for the grid-stride weight-gradient kernels: exactly the workgroups that are resident at once,
// so that all wavefronts walk the (source, target, feature) order together and the XCDs gather from
// one layer of the source matrix at a time.  (With more workgroups than fit, the early ones run
// through every layer before the late ones start and nothing stays in the L2.)
template <typename K>
static unsigned bw_resident_blocks(K kernel) {
  int dev = 0, cus = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, BW_THREADS, 0) != hipSuccess || cus <= 0 || per_cu <= 0) {
    (void)hipGetLastError();
    return 256 * 4;
  }
  unsigned nb = (unsigned)cus * (unsigned)per_cu;
  return nb < 8 ? 8 : nb & ~7u;   // a multiple of the 8 XCDs
}

// ---- JumpReLU threshold gradient (reference clt/models/activations.py:196-199) -------------------
//   grad_theta[f] = sum over tokens of grad_out * (-x / bandwidth)  where |x - theta[f]| <= bandwidth / 2
// on dense [T, F] pre-activations x and dense d loss / d activation, every step rounded to the
// model dtype as the reference's tensor arithmetic is; the sum itself is fp32, rows in a fixed order.
constexpr int TG_SPLIT = 128;   // row slices per column: enough wavefronts in flight to cover the memory latency
template <typename T>
__global__ __launch_bounds__(BW_THREADS) void k_theta_grad_partial(const T *__restrict__ pre, const T *__restrict__ dact,
                                                                    const T *__restrict__ theta, int64_t Tn, int64_t F,
                                                                    float bw, float *__restrict__ part) {
  const int64_t f = (int64_t)blockIdx.x * BW_THREADS + threadIdx.x;
  if (f >= F) return;
  const int64_t rows = (Tn + TG_SPLIT - 1) / TG_SPLIT, r0 = (int64_t)blockIdx.y * rows, r1 = r0 + rows < Tn ? r0 + rows : Tn;
  // (the reference compares with the scalar bandwidth / 2 in the tensors' dtype: the scalar is rounded to it)
  const float th = Elem<T>::to_f32(theta[f]), half = Elem<T>::round(0.5f * bw);
  float acc = 0.0f;
  for (int64_t r = r0; r < r1; ++r) {
    const float x = Elem<T>::to_f32(pre[r * F + f]);
    if (fabsf(Elem<T>::round(x - th)) <= half) {
      const float g = Elem<T>::to_f32(dact[r * F + f]);
      acc += Elem<T>::round(g * Elem<T>::round(-x / bw));
    }
  }
  part[(int64_t)blockIdx.y * F + f] = acc;
}
// The same sums with 16 bytes of a row per thread (8 bf16 / 4 fp32 columns) and four rows of both operands asked
// for at a time: each column is still summed by one thread, over the same rows in the same order.  POW2: the
// bandwidth is a power of two, so -x / bandwidth is the exact product with its reciprocal.
template <typename T, bool POW2>
__global__ __launch_bounds__(BW_THREADS) void k_theta_grad_partial_vec(const T *__restrict__ pre, const T *__restrict__ dact,
                                                                        const T *__restrict__ theta, int64_t Tn, int64_t F,
                                                                        float bw, float inv_bw, float *__restrict__ part) {
  constexpr int V = 16 / (int)sizeof(T), NR = 4;
  const int64_t f0 = ((int64_t)blockIdx.x * BW_THREADS + threadIdx.x) * V;
  if (f0 >= F) return;
  const int64_t rows = (Tn + TG_SPLIT - 1) / TG_SPLIT, r0 = (int64_t)blockIdx.y * rows, r1 = r0 + rows < Tn ? r0 + rows : Tn;
  auto unpack = [](const uint4 &v, float (&x)[V]) {
    if constexpr (sizeof(T) == 2) {
      const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) { x[2 * k] = __uint_as_float(w4[k] << 16); x[2 * k + 1] = __uint_as_float(w4[k] & 0xFFFF0000u); }
    } else {
      x[0] = __uint_as_float(v.x); x[1] = __uint_as_float(v.y); x[2] = __uint_as_float(v.z); x[3] = __uint_as_float(v.w);
    }
  };
  float th[V], acc[V];
  unpack(*reinterpret_cast<const uint4 *>(theta + f0), th);
#pragma unroll
  for (int j = 0; j < V; ++j) acc[j] = 0.0f;
  const float half = Elem<T>::round(0.5f * bw);    // the scalar of the comparison, in the tensors' dtype as torch has it
  for (int64_t r = r0; r < r1; r += NR) {
    uint4 xv[NR], gv[NR];
#pragma unroll
    for (int u = 0; u < NR; ++u) {      // (past the slice: its last row again, not used)
      const int64_t rr = r + u < r1 ? r + u : r1 - 1;
      xv[u] = *reinterpret_cast<const uint4 *>(pre + rr * F + f0);
      gv[u] = *reinterpret_cast<const uint4 *>(dact + rr * F + f0);
    }
#pragma unroll
    for (int u = 0; u < NR; ++u) {
      if (r + u >= r1) break;
      float x[V], g[V];
      unpack(xv[u], x);
      unpack(gv[u], g);
#pragma unroll
      for (int j = 0; j < V; ++j)
        if (fabsf(Elem<T>::round(x[j] - th[j])) <= half)
          acc[j] += Elem<T>::round(g[j] * Elem<T>::round(POW2 ? -x[j] * inv_bw : -x[j] / bw));
    }
  }
#pragma unroll
  for (int j = 0; j < V; ++j) part[(int64_t)blockIdx.y * F + f0 + j] = acc[j];
}
__global__ void k_theta_grad_finish(const float *part, int64_t F, float *out) {
  for (int64_t f = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; f < F; f += (int64_t)gridDim.x * blockDim.x) {
    float a = 0.0f;
    for (int z = 0; z < TG_SPLIT; ++z) a += part[(int64_t)z * F + f];
    out[f] = a;
  }
}

// dense[tok][col[j]] = src[j] (rounded to the model dtype) for the survivors j of one layer's rows
template <typename T>
__global__ __launch_bounds__(BW_THREADS) void k_scatter_layer(const int32_t *row_ptr, const int32_t *col, const float *src,
                                                               int64_t layer, int64_t Tn, int64_t F, T *dense) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    const int64_t r = layer * Tn + t;
    T *row = dense + t * F;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) row[col[j]] = Elem<T>::from_f32(src[j]);
  }
}

// rows of up to 4096 elements: 8 16-byte pieces per lane in bf16, up to 16 in fp32
static bool bw_shape_ok(int64_t d, int dtype) { return d > 0 && d % (dtype == CLT_BF16 ? 8 : 4) == 0 && d <= 4096; }

}  // namespace

extern "C" size_t clt_mse_workspace_bytes(int64_t T, int64_t d, int64_t L) {
  (void)T;
  if (d <= 0 || L <= 0) return 256;
  return (((size_t)L * 8 + 255) & ~(size_t)255) + (size_t)CS_SPLIT * (size_t)L * (size_t)d * 4;
}

extern "C" int clt_mse_loss_grad(const void *rec, const void *target, int64_t T, int64_t d, int64_t L, int dtype,
                                 int denorm_mode, const void *mean, const void *stdv, double denorm_scale,
                                 float *loss_per_layer, float *g, void *g_model, float *bias_grad, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || d <= 0 || L <= 0 || L > 65535 || !rec || !target || !loss_per_layer || !g || !workspace) return CLT_ERR_ARG;
  if (denorm_mode < CLT_DENORM_NONE || denorm_mode > CLT_DENORM_SCALE) return CLT_ERR_ARG;
  if (denorm_mode == CLT_DENORM_MEAN_STD && (!mean || !stdv)) return CLT_ERR_ARG;
  if (denorm_mode == CLT_DENORM_SCALE && !(denorm_scale != 0.0)) return CLT_ERR_ARG;
  if ((T * d) % 4 != 0) return CLT_ERR_ARG;
  if (workspace_bytes < clt_mse_workspace_bytes(T, d, L)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  double *acc = (double *)workspace;
  float *part = (float *)((char *)workspace + (((size_t)L * 8 + 255) & ~(size_t)255));
  k_zero_f64<<<(unsigned)clt_ceil_div(L, 256), 256, 0, s>>>(acc, (int)L);
  const int64_t per_layer = T * d;
  const float scale = (float)(2.0 / (double)per_layer);
  dim3 grid(512, (unsigned)L);
  if (dtype == CLT_BF16) k_mse_grad<bf16_t><<<grid, BW_THREADS, 0, s>>>((const bf16_t *)rec, (const bf16_t *)target, per_layer, d, scale, denorm_mode, (const bf16_t *)mean, (const bf16_t *)stdv, (float)denorm_scale, g, (bf16_t *)g_model, acc);
  else k_mse_grad<float><<<grid, BW_THREADS, 0, s>>>((const float *)rec, (const float *)target, per_layer, d, scale, denorm_mode, (const float *)mean, (const float *)stdv, (float)denorm_scale, g, (float *)g_model, acc);
  k_loss_finish<<<(unsigned)clt_ceil_div(L, 256), 256, 0, s>>>(acc, (int)L, 1.0 / (double)per_layer, loss_per_layer);
  if (bias_grad) {
    k_colsum_partial<<<dim3((unsigned)clt_ceil_div(d, BW_THREADS), (unsigned)L, CS_SPLIT), BW_THREADS, 0, s>>>(g, T, d, part);
    k_colsum_finish<<<dim3((unsigned)clt_ceil_div(d, BW_THREADS), (unsigned)L), BW_THREADS, 0, s>>>(part, d, (int)L, bias_grad);
  }
  return clt_check_launch();
}

extern "C" size_t clt_decode_backward_workspace_bytes(int64_t T, int64_t L, int64_t nnz) {
  if (T <= 0 || L <= 0 || nnz < 0) return 256;
  return (((size_t)L * (size_t)T * (BWV_XCDS + 1) * 4 + 255) & ~(size_t)255) + (size_t)L * (size_t)(nnz > 0 ? nnz : 1) * 4;
}

extern "C" int clt_decode_backward_values(const int32_t *row_ptr, const int32_t *col, const void *val, const void *w_packed,
                                          const void *feat_scale, const float *g, int64_t T, int64_t d, int64_t F, int64_t L,
                                          int tying, uint64_t src_mask, int64_t nnz, int dtype, float *dval, void *workspace,
                                          size_t workspace_bytes, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 64 || tying < 0 || tying > 2 || nnz < 0) return CLT_ERR_ARG;
  if (!row_ptr || !w_packed || !g || !dval || !workspace) return CLT_ERR_ARG;
  if (!bw_shape_ok(d, dtype)) return CLT_ERR_RANGE;
  if (nnz == 0) return CLT_OK;
  if (workspace_bytes < clt_decode_backward_workspace_bytes(T, L, nnz)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  int32_t *sptr = (int32_t *)workspace;
  float *part = (float *)((char *)workspace + (((size_t)L * (size_t)T * (BWV_XCDS + 1) * 4 + 255) & ~(size_t)255));
  k_bw_slice_ptr<<<1024, 256, 0, s>>>(row_ptr, col, L * T, F, BWV_XCDS, sptr);
  const int nc4 = (int)clt_ceil_div(d, dtype == CLT_BF16 ? 512 : 256);   // 16-byte pieces per lane
  const int64_t npair = L * (L + 1) / 2;
  const int64_t nblk = npair * clt_ceil_div(T, (BW_THREADS / 64) * BWV_NTOK) * BWV_XCDS;
  if (nblk > 2147483647LL) return CLT_ERR_RANGE;
#define CLT_BWV(TT, N) k_bwd_values_sliced<TT, N, false><<<(unsigned)nblk, BW_THREADS, 0, s>>>(sptr, col, (const TT *)w_packed, g, T, d, F, L, tying, nnz, part)
#define CLT_BWV_N(TT)                                                                       \
  do {                                                                                      \
    switch (nc4) {                                                                          \
      case 1: CLT_BWV(TT, 1); break; case 2: CLT_BWV(TT, 2); break; case 3: CLT_BWV(TT, 3); break; \
      case 4: CLT_BWV(TT, 4); break; case 5: CLT_BWV(TT, 5); break; case 6: CLT_BWV(TT, 6); break; \
      case 7: CLT_BWV(TT, 7); break; default: CLT_BWV(TT, 8); break;                        \
    }                                                                                       \
  } while (0)
  if (dtype == CLT_BF16 && d == 768)
    k_bwd_values_sliced<bf16_t, 2, true><<<(unsigned)nblk, BW_THREADS, 0, s>>>(sptr, col, (const bf16_t *)w_packed, g, T, d, F, L, tying, nnz, part);
  else if (dtype == CLT_BF16) CLT_BWV_N(bf16_t);
  else if (nc4 <= 8) CLT_BWV_N(float);
  else if (nc4 <= 10) CLT_BWV(float, 10);      // fp32 rows beyond 2048 elements: a piece count that covers them
  else if (nc4 <= 12) CLT_BWV(float, 12);
  else if (nc4 <= 14) CLT_BWV(float, 14);
  else CLT_BWV(float, 16);
#undef CLT_BWV_N
#undef CLT_BWV
  if (feat_scale && !val) return CLT_ERR_ARG;
  if (dtype == CLT_BF16)
    k_bwd_values_sum<bf16_t><<<256 * 8, BW_THREADS, 0, s>>>(row_ptr, part, T, L, nnz, src_mask, dval, col, (const bf16_t *)val,
                                                            (const bf16_t *)feat_scale, F);
  else
    k_bwd_values_sum<float><<<256 * 8, BW_THREADS, 0, s>>>(row_ptr, part, T, L, nnz, src_mask, dval, col, (const float *)val,
                                                           (const float *)feat_scale, F);
  return clt_check_launch();
}

extern "C" int clt_feature_affine_grad(const int32_t *list_ptr, const int32_t *list_src, const void *val,
                                       const void *feat_offset, const void *feat_scale, int64_t T, int64_t F, int64_t L,
                                       uint64_t src_mask, int64_t nnz, int dtype, float *d_offset, float *d_scale,
                                       const void *workspace, size_t workspace_bytes, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 64 || nnz < 0 || !list_ptr || !list_src || !val || !workspace) return CLT_ERR_ARG;
  if (!d_offset && !d_scale) return CLT_OK;
  if (workspace_bytes < clt_decode_backward_workspace_bytes(T, L, nnz)) return CLT_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  // the per-target dot products clt_decode_backward_values left behind the slice pointers
  const float *part = (const float *)((const char *)workspace + (((size_t)L * (size_t)T * (BWV_XCDS + 1) * 4 + 255) & ~(size_t)255));
  if (dtype == CLT_BF16)
    k_affine_grad<bf16_t><<<256 * 8, BW_THREADS, 0, s>>>(list_ptr, list_src, (const bf16_t *)val, part, (const bf16_t *)feat_offset,
                                                         (const bf16_t *)feat_scale, F, L, nnz, src_mask, d_offset, d_scale);
  else
    k_affine_grad<float><<<256 * 8, BW_THREADS, 0, s>>>(list_ptr, list_src, (const float *)val, part, (const float *)feat_offset,
                                                        (const float *)feat_scale, F, L, nnz, src_mask, d_offset, d_scale);
  return clt_check_launch();
}

extern "C" int clt_skip_weight_grad(const float *g, const void *x, float *out, int64_t T, int64_t d, int accumulate, int dtype,
                                    void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || d <= 0 || !g || !x || !out) return CLT_ERR_ARG;
  if (clt_ceil_div(d, 64) > 65535) return CLT_ERR_RANGE;
  dim3 grid((unsigned)clt_ceil_div(d, 64), (unsigned)clt_ceil_div(d, 64));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_skip_grad<bf16_t><<<grid, 256, 0, s>>>(g, (const bf16_t *)x, out, T, d, accumulate);
  else k_skip_grad<float><<<grid, 256, 0, s>>>(g, (const float *)x, out, T, d, accumulate);
  return clt_check_launch();
}

// More than 64 KB of dynamic LDS has to be granted per kernel; false when the device does not have it.
static bool fl_lds_granted(size_t bytes) {
  if (bytes <= 64 * 1024) return true;
  int dev = 0, lds_max = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&lds_max, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess ||
      (size_t)lds_max < bytes ||
      hipFuncSetAttribute((const void *)k_fl_count, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess ||
      hipFuncSetAttribute((const void *)k_fl_fill, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return true;
}

extern "C" size_t clt_feature_lists_workspace_bytes(int64_t F, int64_t L) {
  if (F <= 0 || L <= 0) return 256;
  const size_t n = (size_t)L * (size_t)F;
  // counters + chunk sums + the per-block counts of the blocked route
  return ((n * 4 + 255) & ~(size_t)255) + ((((n + CSC_CHUNK - 1) / CSC_CHUNK) * 8 + 255) & ~(size_t)255) +
         n * FL_MAX_BLOCKS * sizeof(uint16_t);
}

extern "C" int clt_feature_lists(const int32_t *row_ptr, const int32_t *col, int64_t T, int64_t F, int64_t L,
                                 int32_t *list_ptr, int32_t *list_tok, int32_t *list_src, void *workspace,
                                 size_t workspace_bytes, void *stream) {
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || !row_ptr || !list_ptr || !workspace) return CLT_ERR_ARG;
  if ((double)L * (double)F >= 2147483647.0) return CLT_ERR_RANGE;
  if (T > 262144) return CLT_ERR_RANGE;   // a wavefront's two token bitmaps take T / 4 bytes of LDS (64 KB here)
  if (workspace_bytes < clt_feature_lists_workspace_bytes(F, L)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 7u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  uint32_t *cnt = (uint32_t *)workspace;
  const int64_t n = L * F;
  const unsigned nb = 256 * 8;
  const int64_t nchunk = clt_ceil_div(n, CSC_CHUNK);
  unsigned long long *sums = (unsigned long long *)((char *)workspace + (((size_t)n * 4 + 255) & ~(size_t)255));
  // blocked route: F counters in LDS, lists in token order by construction
  // one workgroup per (layer, block of tokens) and per CU (the counters fill its LDS): as many blocks as
  // give every CU one workgroup, at least FL_MIN_BLOCK_TOKENS tokens each
  int cus = 0, dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
    (void)hipGetLastError();
    cus = 256;
  }
  int64_t NB64 = cus / L > 0 ? cus / L : 1;
  if (NB64 > clt_ceil_div(T, FL_MIN_BLOCK_TOKENS)) NB64 = clt_ceil_div(T, FL_MIN_BLOCK_TOKENS);
  if (NB64 > FL_MAX_BLOCKS) NB64 = FL_MAX_BLOCKS;
  if (clt_ceil_div(T, NB64) > 1024) NB64 = clt_ceil_div(T, 1024);     // the staged token offsets and the counts are 16-bit
  const int NB = (int)NB64, TB = (int)clt_ceil_div(T, NB);
  // the staging buffer takes what the counters leave (6 bytes per entry)
  int64_t cap = ((int64_t)FL_LDS_MAX - ((int64_t)F + TB + 1) * 4) / 6;
  cap = cap > FL_MAX_CAP ? FL_MAX_CAP : cap & ~(int64_t)511;
  const size_t fl_lds = ((size_t)F + (size_t)(cap > 0 ? cap : 0) * 3 / 2 + (size_t)TB + 1) * 4;
  if (list_tok && list_src && NB <= FL_MAX_BLOCKS && cap >= FL_MIN_CAP && L * NB < 2147483647LL && fl_lds_granted(fl_lds)) {
    uint16_t *counts = (uint16_t *)((char *)sums + ((((size_t)nchunk * 8) + 255) & ~(size_t)255));
    k_fl_count<<<(unsigned)(L * NB), FL_THREADS, (size_t)F * 4, s>>>(row_ptr, col, T, F, TB, NB, counts, n);
    k_fl_total<<<nb, BW_THREADS, 0, s>>>(counts, NB, n, cnt);
    k_csc_chunk_sum<<<(unsigned)nchunk, BW_THREADS, 0, s>>>(cnt, n, sums);
    k_csc_chunk_offsets<<<1, BW_THREADS, 0, s>>>(sums, nchunk, list_ptr, n);
    k_csc_chunk_scan<<<(unsigned)nchunk, BW_THREADS, 0, s>>>(cnt, n, sums, list_ptr);
    k_fl_fill<<<(unsigned)(L * NB), FL_THREADS, fl_lds, s>>>(row_ptr, col, T, F, TB, NB, counts, n, list_ptr, list_tok, list_src, (int)cap);
    return clt_check_launch();
  }
  k_zero_u32<<<nb, BW_THREADS, 0, s>>>(cnt, n);
  k_csc_count<<<nb, BW_THREADS, 0, s>>>(row_ptr, col, T, F, L, cnt);
  k_csc_chunk_sum<<<(unsigned)nchunk, BW_THREADS, 0, s>>>(cnt, n, sums);
  k_csc_chunk_offsets<<<1, BW_THREADS, 0, s>>>(sums, nchunk, list_ptr, n);
  k_csc_chunk_scan<<<(unsigned)nchunk, BW_THREADS, 0, s>>>(cnt, n, sums, list_ptr);
  if (list_tok && list_src) {
    k_csc_fill<<<nb, BW_THREADS, 0, s>>>(row_ptr, col, T, F, L, list_ptr, cnt, list_tok, list_src);
    const int bm_words = (int)clt_ceil_div(T, 32);
    // as many wavefronts per workgroup as have room for their bitmaps in 64 KB: four up to 65536 tokens
    const int order_waves = T <= 65536 ? 4 : T <= 131072 ? 2 : 1;
    k_csc_order<<<nb, order_waves * 64, (size_t)order_waves * 2 * bm_words * 4, s>>>(list_ptr, n, list_tok, list_src, row_ptr, col,
                                                                                     T, F, bm_words);
  }
  return clt_check_launch();
}

extern "C" int clt_decoder_weight_grad(const int32_t *list_ptr, const int32_t *list_tok, const int32_t *list_src,
                                       const void *val, const void *g_model, const void *feat_offset, const void *feat_scale,
                                       float *dw_packed, int64_t T, int64_t d, int64_t F, int64_t L, int tying, int dtype,
                                       void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (tying < 0 || tying > 2) return CLT_ERR_ARG;
  if (T <= 0 || F <= 0 || L <= 0 || L > 64 || !list_ptr || !list_tok || !list_src || !val || !g_model || !dw_packed) return CLT_ERR_ARG;
  if (!bw_shape_ok(d, dtype)) return CLT_ERR_RANGE;
  hipStream_t s = (hipStream_t)stream;
  const int esz = dtype == CLT_BF16 ? 2 : 4, ev = 16 / esz;
  const int nc4 = (int)clt_ceil_div(d / ev, 64);   // 16-byte pieces per lane
#define CLT_DW(CT, N)                                                                                                      \
  do {                                                                                                                     \
    for (int64_t t = 0; t < L; ++t) {                                                                                      \
      k_feature_outer<CT, CT, N, true><<<bw_resident_blocks(k_feature_outer<CT, CT, N, true>), BW_THREADS, 0, s>>>(list_ptr, list_tok, list_src, (const CT *)val, (const CT *)g_model, dw_packed, nullptr, T, d, F, L, t, tying, (const CT *)feat_offset, (const CT *)feat_scale); \
    }                                                                                                                      \
  } while (0)
#define CLT_DW_N(CT)                                                                       \
  do {                                                                                     \
    switch (nc4) {                                                                         \
      case 1: CLT_DW(CT, 1); break; case 2: CLT_DW(CT, 2); break; case 3: CLT_DW(CT, 3); break; \
      case 4: CLT_DW(CT, 4); break; case 5: CLT_DW(CT, 5); break; case 6: CLT_DW(CT, 6); break; \
      case 7: CLT_DW(CT, 7); break; default: CLT_DW(CT, 8); break;                         \
    }                                                                                      \
  } while (0)
  if (dtype == CLT_BF16 && d == 768) {
    for (int64_t t = 0; t < L; ++t)
      k_feature_outer<bf16_t, bf16_t, 2, true, true><<<bw_resident_blocks(k_feature_outer<bf16_t, bf16_t, 2, true, true>), BW_THREADS, 0, s>>>(
          list_ptr, list_tok, list_src, (const bf16_t *)val, (const bf16_t *)g_model, dw_packed, nullptr, T, d, F, L, t, tying,
          (const bf16_t *)feat_offset, (const bf16_t *)feat_scale);
  } else if (dtype == CLT_BF16) CLT_DW_N(bf16_t);
  else if (nc4 <= 8) CLT_DW_N(float);
  else if (nc4 <= 10) CLT_DW(float, 10);
  else if (nc4 <= 12) CLT_DW(float, 12);
  else if (nc4 <= 14) CLT_DW(float, 14);
  else CLT_DW(float, 16);
#undef CLT_DW_N
#undef CLT_DW
  return clt_check_launch();
}

extern "C" int clt_decoder_weight_grad_adam(const int32_t *list_ptr, const int32_t *list_tok, const int32_t *list_src,
                                            const void *val, const void *g_model, void *w_packed, float *m, float *v,
                                            int64_t T, int64_t d, int64_t F, int64_t L, double lr, double beta1, double beta2,
                                            double eps, int64_t step, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 64 || step < 1 || !(beta1 >= 0 && beta1 < 1) || !(beta2 >= 0 && beta2 < 1) ||
      !list_ptr || !list_tok || !list_src || !val || !g_model || !w_packed || !m || !v)
    return CLT_ERR_ARG;
  if (!bw_shape_ok(d, dtype)) return CLT_ERR_RANGE;
  hipStream_t s = (hipStream_t)stream;
  const int esz = dtype == CLT_BF16 ? 2 : 4, ev = 16 / esz;
  const int nc4 = (int)clt_ceil_div(d / ev, 64);   // 16-byte pieces per lane
  AdamInPlace ad;
  ad.m = m; ad.v = v; ad.w_packed = w_packed; ad.pitch = clt_pitch(d, esz); ad.c = adam_coef(lr, beta1, beta2, eps, step);
#define CLT_DWA(CT, N, T8)                                                                                                 \
  do {                                                                                                                     \
    for (int64_t t = 0; t < L; ++t) {                                                                                      \
      k_feature_outer<CT, CT, N, true, T8, true><<<bw_resident_blocks(k_feature_outer<CT, CT, N, true, T8, true>), BW_THREADS, 0, s>>>(list_ptr, list_tok, list_src, (const CT *)val, (const CT *)g_model, nullptr, nullptr, T, d, F, L, t, CLT_TYING_NONE, nullptr, nullptr, ad); \
    }                                                                                                                      \
  } while (0)
#define CLT_DWA_N(CT)                                                                                \
  do {                                                                                               \
    switch (nc4) {                                                                                   \
      case 1: CLT_DWA(CT, 1, false); break; case 2: CLT_DWA(CT, 2, false); break; case 3: CLT_DWA(CT, 3, false); break; \
      case 4: CLT_DWA(CT, 4, false); break; case 5: CLT_DWA(CT, 5, false); break; case 6: CLT_DWA(CT, 6, false); break; \
      case 7: CLT_DWA(CT, 7, false); break; default: CLT_DWA(CT, 8, false); break;                     \
    }                                                                                                \
  } while (0)
  if (dtype == CLT_BF16 && d == 768) CLT_DWA(bf16_t, 2, true);
  else if (dtype == CLT_BF16) CLT_DWA_N(bf16_t);
  else if (nc4 <= 8) CLT_DWA_N(float);
  else if (nc4 <= 10) CLT_DWA(float, 10, false);
  else if (nc4 <= 12) CLT_DWA(float, 12, false);
  else if (nc4 <= 14) CLT_DWA(float, 14, false);
  else CLT_DWA(float, 16, false);
#undef CLT_DWA_N
#undef CLT_DWA
  return clt_check_launch();
}

extern "C" int clt_encoder_weight_grad(const int32_t *list_ptr, const int32_t *list_tok, const int32_t *list_src,
                                       const float *dval, const void *x, float *dw_enc, float *db_enc, int64_t T, int64_t d,
                                       int64_t F, int64_t L, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || !list_ptr || !list_tok || !list_src || !dval || !x || !dw_enc) return CLT_ERR_ARG;
  if (!bw_shape_ok(d, dtype)) return CLT_ERR_RANGE;
  hipStream_t s = (hipStream_t)stream;
  const int esz = dtype == CLT_BF16 ? 2 : 4, ev = 16 / esz;
  const int nc4 = (int)clt_ceil_div(d / ev, 64);   // 16-byte pieces per lane
#define CLT_EW(ST, N)                                                                                                      \
  do {                                                                                                                     \
    for (int64_t l = 0; l < L; ++l) {                                                                                      \
      k_feature_outer<ST, float, N, false><<<bw_resident_blocks(k_feature_outer<ST, float, N, false>), BW_THREADS, 0, s>>>(list_ptr, list_tok, list_src, dval, (const ST *)x, dw_enc, db_enc, T, d, F, L, l, CLT_TYING_NONE); \
    }                                                                                                                      \
  } while (0)
#define CLT_EW_N(ST)                                                                       \
  do {                                                                                     \
    switch (nc4) {                                                                         \
      case 1: CLT_EW(ST, 1); break; case 2: CLT_EW(ST, 2); break; case 3: CLT_EW(ST, 3); break; \
      case 4: CLT_EW(ST, 4); break; case 5: CLT_EW(ST, 5); break; case 6: CLT_EW(ST, 6); break; \
      case 7: CLT_EW(ST, 7); break; default: CLT_EW(ST, 8); break;                         \
    }                                                                                      \
  } while (0)
  if (dtype == CLT_BF16 && d == 768) {
    for (int64_t l = 0; l < L; ++l)
      k_feature_outer<bf16_t, float, 2, false, true><<<bw_resident_blocks(k_feature_outer<bf16_t, float, 2, false, true>), BW_THREADS, 0, s>>>(
          list_ptr, list_tok, list_src, dval, (const bf16_t *)x, dw_enc, db_enc, T, d, F, L, l, CLT_TYING_NONE);
  } else if (dtype == CLT_BF16) CLT_EW_N(bf16_t);
  else if (nc4 <= 8) CLT_EW_N(float);
  else if (nc4 <= 10) CLT_EW(float, 10);
  else if (nc4 <= 12) CLT_EW(float, 12);
  else if (nc4 <= 14) CLT_EW(float, 14);
  else CLT_EW(float, 16);
#undef CLT_EW_N
#undef CLT_EW
  return clt_check_launch();
}

extern "C" int clt_scatter_survivor_values(const int32_t *row_ptr, const int32_t *col, const float *src, int64_t layer,
                                           int64_t T, int64_t F, int64_t L, int dtype, void *dense, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T < 0 || F <= 0 || L <= 0 || layer < 0 || layer >= L) return CLT_ERR_ARG;
  if (T == 0) return CLT_OK;
  if (!row_ptr || !col || !src || !dense) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_scatter_layer<bf16_t><<<256 * 8, BW_THREADS, 0, s>>>(row_ptr, col, src, layer, T, F, (bf16_t *)dense);
  else k_scatter_layer<float><<<256 * 8, BW_THREADS, 0, s>>>(row_ptr, col, src, layer, T, F, (float *)dense);
  return clt_check_launch();
}

extern "C" size_t clt_jumprelu_theta_grad_workspace_bytes(int64_t F) { return F > 0 ? (size_t)TG_SPLIT * (size_t)F * 4 : 256; }

extern "C" int clt_jumprelu_theta_grad(const void *pre, const void *dact, const void *theta, int64_t T, int64_t F,
                                       double bandwidth, int dtype, float *grad_theta, void *workspace, size_t workspace_bytes,
                                       void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || !(bandwidth > 0.0) || !pre || !dact || !theta || !grad_theta || !workspace) return CLT_ERR_ARG;
  if (workspace_bytes < clt_jumprelu_theta_grad_workspace_bytes(F)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 3u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  float *part = (float *)workspace;
  const float bwf = (float)bandwidth;
  const int esz = dtype == CLT_BF16 ? 2 : 4, vec = 16 / esz;
  // whole 16-byte pieces per row and aligned rows: the vector kernel; anything else one column per thread
  if (F % vec == 0 && clt_aligned16(pre) && clt_aligned16(dact) && clt_aligned16(theta)) {
    int ex = 0;
    const bool pow2 = frexpf(bwf, &ex) == 0.5f && ex > -100 && ex < 100;    // 1 / bandwidth is exact and normal
    dim3 gridv((unsigned)clt_ceil_div(F / vec, BW_THREADS), TG_SPLIT);
#define CLT_TG(CT, P2) k_theta_grad_partial_vec<CT, P2><<<gridv, BW_THREADS, 0, s>>>((const CT *)pre, (const CT *)dact, (const CT *)theta, T, F, bwf, 1.0f / bwf, part)
    if (dtype == CLT_BF16) { if (pow2) CLT_TG(bf16_t, true); else CLT_TG(bf16_t, false); }
    else { if (pow2) CLT_TG(float, true); else CLT_TG(float, false); }
#undef CLT_TG
  } else {
    dim3 grid((unsigned)clt_ceil_div(F, BW_THREADS), TG_SPLIT);
    if (dtype == CLT_BF16)
      k_theta_grad_partial<bf16_t><<<grid, BW_THREADS, 0, s>>>((const bf16_t *)pre, (const bf16_t *)dact, (const bf16_t *)theta, T, F, bwf, part);
    else
      k_theta_grad_partial<float><<<grid, BW_THREADS, 0, s>>>((const float *)pre, (const float *)dact, (const float *)theta, T, F, bwf, part);
  }
  k_theta_grad_finish<<<(unsigned)clt_ceil_div(F, 256), 256, 0, s>>>(part, F, grad_theta);
  return clt_check_launch();
}
