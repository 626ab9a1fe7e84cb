// Evaluation reductions computed from the survivor list and from the reconstructions, without a
// dense [T, F] activation tensor:
//   * L0: entries != 0 per layer            (reference clt/training/evaluator.py:194-244)
//   * per-feature firing counts (value > eps) (reference clt/training/evaluator.py:350-405)
//   * dead-feature counters                   (reference clt/training/trainer.py:693-712)
//   * MSE, per-column variance of the target and of the error, after the reference's
//     de-normalisation in the model dtype     (reference clt/training/evaluator.py:246-345)
#include "clt_common.h"

namespace {

constexpr int MT_THREADS = 256;

__global__ void k_metrics_zero(uint32_t *fired, int64_t n, unsigned long long *nonzero, int L) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) fired[i] = 0u;
  if (blockIdx.x == 0)
    for (int i = threadIdx.x; i < L; i += blockDim.x) nonzero[i] = 0ull;
}

// Each wavefront takes a run of consecutive (layer, token) rows, so its non-zero count goes to the
// layer's counter once per run (a same-address atomic per row would serialise the whole grid).
template <typename T>
__global__ __launch_bounds__(MT_THREADS) void k_survivor_metrics(const int32_t *__restrict__ row_ptr, const int32_t *__restrict__ col,
                                                                 const T *__restrict__ val, int64_t Tn, int64_t F, int64_t L,
                                                                 float eps, unsigned long long *nonzero, uint32_t *fired) {
  const int lane = lane_id(), nwv = blockDim.x >> 6;
  const int64_t R = L * Tn, nwave = (int64_t)gridDim.x * nwv, w = (int64_t)blockIdx.x * nwv + (threadIdx.x >> 6);
  const int64_t per = (R + nwave - 1) / nwave, r0 = w * per, r1 = r0 + per < R ? r0 + per : R;
  uint32_t nz = 0;
  int64_t cur = r0 < R ? r0 / Tn : 0;
  auto flush = [&](int64_t layer) {
    uint32_t tot = nz;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) tot += __shfl_xor(tot, o);
    if (lane == 0 && tot) atomicAdd(&nonzero[layer], (unsigned long long)tot);
    nz = 0;
  };
  for (int64_t r = r0; r < r1; ++r) {
    const int64_t l = r / Tn;
    if (l != cur) { flush(cur); cur = l; }
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) {
      const float v = Elem<T>::to_f32(val[j]);
      nz += v != 0.0f ? 1u : 0u;            // NaN counts, as `!= 0` does
      if (v > eps) atomicAdd(&fired[l * F + col[j]], 1u);
    }
  }
  if (r0 < r1) flush(cur);
}

__global__ void k_dead_update(const uint32_t *fired, int64_t *passes, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    passes[i] = fired[i] ? 0 : passes[i] + 1;
}

// ---- reconstruction statistics --------------------------------------------------------------------
// A block covers 64 columns of one layer and one of RS_SPLIT row ranges, with 4 row lanes.  Sums
// are kept in double around a per-column pivot (the de-normalised first row), so one pass loses
// nothing to cancellation; every row range uses the same pivot and the partials add up.
constexpr int RS_SPLIT = 16;
constexpr int RS_ACC = 5;   // sum(t-p), sum((t-p)^2), sum(e-q), sum((e-q)^2), sum(e^2)

template <typename T>
__device__ __forceinline__ float denorm(float x, int mode, float mean, float stdv, float scale) {
  // each arithmetic step is rounded to the model dtype, as torch does for `x * std + mean` and `x / s`
  if (mode == CLT_DENORM_MEAN_STD) return Elem<T>::round(Elem<T>::round(x * stdv) + mean);
  if (mode == CLT_DENORM_SCALE) return Elem<T>::round(x / scale);
  return x;
}

template <typename T>
__global__ __launch_bounds__(MT_THREADS) void k_recon_partial(const T *__restrict__ rec, const T *__restrict__ tgt, int64_t Tn,
                                                              int64_t d, int mode, const T *__restrict__ mean,
                                                              const T *__restrict__ stdv, float scale, double *part) {
  __shared__ double red[4][RS_ACC][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t l = blockIdx.y, c = (int64_t)blockIdx.x * 64 + tx, z = blockIdx.z;
  const int64_t rows = (Tn + RS_SPLIT - 1) / RS_SPLIT, r0 = z * rows, r1 = (r0 + rows < Tn) ? r0 + rows : Tn;
  double a[RS_ACC] = {0, 0, 0, 0, 0};
  if (c < d) {
    const float mu = mode == CLT_DENORM_MEAN_STD ? Elem<T>::to_f32(mean[l * d + c]) : 0.0f;
    const float sd = mode == CLT_DENORM_MEAN_STD ? Elem<T>::to_f32(stdv[l * d + c]) : 1.0f;
    const T *rb = rec + l * Tn * d + c, *tb = tgt + l * Tn * d + c;
    const float pt = denorm<T>(Elem<T>::to_f32(tb[0]), mode, mu, sd, scale);
    const float pe = pt - denorm<T>(Elem<T>::to_f32(rb[0]), mode, mu, sd, scale);
    for (int64_t r = r0 + ty; r < r1; r += 4) {
      const float t = denorm<T>(Elem<T>::to_f32(tb[r * d]), mode, mu, sd, scale);
      const float x = denorm<T>(Elem<T>::to_f32(rb[r * d]), mode, mu, sd, scale);
      const float e = t - x;   // fp32, as the reference's `.float()` difference
      const double dt = (double)t - (double)pt, de = (double)e - (double)pe;
      a[0] += dt; a[1] += dt * dt; a[2] += de; a[3] += de * de; a[4] += (double)e * (double)e;
    }
  }
#pragma unroll
  for (int k = 0; k < RS_ACC; ++k) red[ty][k][tx] = a[k];
  __syncthreads();
  if (ty == 0 && c < d) {
#pragma unroll
    for (int k = 0; k < RS_ACC; ++k)
      part[((l * RS_SPLIT + z) * RS_ACC + k) * d + c] = red[0][k][tx] + red[1][k][tx] + red[2][k][tx] + red[3][k][tx];
  }
}

// one block per layer: column variances, their means, and the MSE
__global__ __launch_bounds__(MT_THREADS) void k_recon_finish(const double *part, int64_t Tn, int64_t d, double *stats) {
  __shared__ double red[3][MT_THREADS];
  const int64_t l = blockIdx.x;
  double vt = 0.0, ve = 0.0, ee = 0.0;
  for (int64_t c = threadIdx.x; c < d; c += blockDim.x) {
    double a[RS_ACC] = {0, 0, 0, 0, 0};
    for (int z = 0; z < RS_SPLIT; ++z)
#pragma unroll
      for (int k = 0; k < RS_ACC; ++k) a[k] += part[((l * RS_SPLIT + z) * RS_ACC + k) * d + c];
    const double n = (double)Tn;
    double v1 = (a[1] - a[0] * a[0] / n) / n, v2 = (a[3] - a[2] * a[2] / n) / n;
    vt += v1 > 0.0 ? v1 : 0.0;
    ve += v2 > 0.0 ? v2 : 0.0;
    ee += a[4];
  }
  red[0][threadIdx.x] = vt; red[1][threadIdx.x] = ve; red[2][threadIdx.x] = ee;
  __syncthreads();
  for (int o = MT_THREADS / 2; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o)
      for (int k = 0; k < 3; ++k) red[k][threadIdx.x] += red[k][threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    stats[l * 3 + 0] = red[2][0] / ((double)Tn * (double)d);   // MSE
    stats[l * 3 + 1] = red[0][0] / (double)d;                  // mean column variance of the target
    stats[l * 3 + 2] = red[1][0] / (double)d;                  // mean column variance of the error
  }
}

}  // namespace

extern "C" int clt_survivor_metrics(const int32_t *row_ptr, const int32_t *col, const void *val, int64_t T, int64_t F,
                                    int64_t L, int dtype, float fired_eps, uint64_t *nonzero_per_layer,
                                    uint32_t *fired_count, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || !row_ptr || !nonzero_per_layer || !fired_count) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  k_metrics_zero<<<1024, MT_THREADS, 0, s>>>(fired_count, L * F, (unsigned long long *)nonzero_per_layer, (int)L);
  if (col && val) {
    const unsigned nb = 256 * 8;
    if (dtype == CLT_BF16)
      k_survivor_metrics<bf16_t><<<nb, MT_THREADS, 0, s>>>(row_ptr, col, (const bf16_t *)val, T, F, L, fired_eps,
                                                           (unsigned long long *)nonzero_per_layer, fired_count);
    else if (dtype == CLT_F16)
      k_survivor_metrics<f16_t><<<nb, MT_THREADS, 0, s>>>(row_ptr, col, (const f16_t *)val, T, F, L, fired_eps,
                                                           (unsigned long long *)nonzero_per_layer, fired_count);
    else
      k_survivor_metrics<float><<<nb, MT_THREADS, 0, s>>>(row_ptr, col, (const float *)val, T, F, L, fired_eps,
                                                          (unsigned long long *)nonzero_per_layer, fired_count);
  }
  return clt_check_launch();
}

extern "C" int clt_dead_feature_update(const uint32_t *fired_count, int64_t *passes_since_fired, int64_t n, void *stream) {
  if (n < 0 || (n > 0 && (!fired_count || !passes_since_fired))) return CLT_ERR_ARG;
  if (n == 0) return CLT_OK;
  int64_t nb = clt_ceil_div(n, MT_THREADS);
  if (nb > 4096) nb = 4096;
  k_dead_update<<<(unsigned)nb, MT_THREADS, 0, (hipStream_t)stream>>>(fired_count, passes_since_fired, n);
  return clt_check_launch();
}

extern "C" size_t clt_reconstruction_stats_workspace_bytes(int64_t d, int64_t L) {
  if (d <= 0 || L <= 0) return 256;
  return (size_t)L * RS_SPLIT * RS_ACC * (size_t)d * 8;
}

extern "C" int clt_reconstruction_stats(const void *rec, const void *target, int64_t T, int64_t d, int64_t L, int dtype,
                                        int denorm_mode, const void *mean, const void *stdv, double scale, double *stats,
                                        void *workspace, size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || d <= 0 || L <= 0 || L > 65535 || !rec || !target || !stats || !workspace) return CLT_ERR_ARG;
  if (denorm_mode < CLT_DENORM_NONE || denorm_mode > CLT_DENORM_SCALE) return CLT_ERR_ARG;
  if (denorm_mode == CLT_DENORM_MEAN_STD && (!mean || !stdv)) return CLT_ERR_ARG;
  if (denorm_mode == CLT_DENORM_SCALE && !(scale != 0.0)) return CLT_ERR_ARG;
  if (workspace_bytes < clt_reconstruction_stats_workspace_bytes(d, L)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 7u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  double *part = (double *)workspace;
  dim3 grid((unsigned)clt_ceil_div(d, 64), (unsigned)L, RS_SPLIT);
  if (dtype == CLT_BF16)
    k_recon_partial<bf16_t><<<grid, MT_THREADS, 0, s>>>((const bf16_t *)rec, (const bf16_t *)target, T, d, denorm_mode,
                                                        (const bf16_t *)mean, (const bf16_t *)stdv, (float)scale, part);
  else if (dtype == CLT_F16)
    k_recon_partial<f16_t><<<grid, MT_THREADS, 0, s>>>((const f16_t *)rec, (const f16_t *)target, T, d, denorm_mode,
                                                        (const f16_t *)mean, (const f16_t *)stdv, (float)scale, part);
  else
    k_recon_partial<float><<<grid, MT_THREADS, 0, s>>>((const float *)rec, (const float *)target, T, d, denorm_mode,
                                                       (const float *)mean, (const float *)stdv, (float)scale, part);
  k_recon_finish<<<(unsigned)L, MT_THREADS, 0, s>>>(part, T, d, stats);
  return clt_check_launch();
}
