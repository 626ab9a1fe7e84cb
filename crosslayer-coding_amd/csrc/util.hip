// Library identity, error text, and the per-feature ranking statistics of the global
// BatchTopK / TokenTopK helper (reference clt/models/activations.py:281-283).
#include "clt_common.h"

namespace {

// One block = 64 feature columns x 4 row groups; two passes over the column
// (mean, then centred sum of squares) with double accumulation.
template <typename T>
__global__ __launch_bounds__(256) void k_colstats(const T *pre, float *mean, float *denom, float *stdv, int64_t Tn,
                                                  int64_t F, int64_t lstride) {
  __shared__ double red[4][64];
  __shared__ double smean[64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int64_t l = blockIdx.y, f = (int64_t)blockIdx.x * 64 + tx;
  const T *base = pre + l * lstride;
  double s = 0.0;
  if (f < F)
    for (int64_t t = ty; t < Tn; t += 4) s += (double)Elem<T>::to_f32(base[t * F + f]);
  red[ty][tx] = s;
  __syncthreads();
  if (ty == 0) smean[tx] = (red[0][tx] + red[1][tx] + red[2][tx] + red[3][tx]) / (double)Tn;
  __syncthreads();
  const double mu = smean[tx];
  double q = 0.0;
  if (f < F)
    for (int64_t t = ty; t < Tn; t += 4) { double dlt = (double)Elem<T>::to_f32(base[t * F + f]) - mu; q += dlt * dlt; }
  __syncthreads();
  red[ty][tx] = q;
  __syncthreads();
  if (ty == 0 && f < F) {
    double var = (red[0][tx] + red[1][tx] + red[2][tx] + red[3][tx]) / (double)(Tn - 1);  // T == 1 gives NaN, as torch.std does
    float m = Elem<T>::round((float)mu);
    float sd = Elem<T>::round((float)sqrt(var));
    mean[l * F + f] = m;
    denom[l * F + f] = Elem<T>::round(sd + 1e-6f);
    if (stdv) stdv[l * F + f] = sd;
  }
}

// Vector version: one pass.  A block covers 32 x V columns (V = elements per 16 bytes) with 8
// row lanes; sums of (x - p) and (x - p)^2 are kept in double, with the column's first value as
// the pivot p, so the single pass loses nothing to cancellation when the mean is far from zero.
template <typename T>
__global__ __launch_bounds__(256) void k_colstats_vec(const T *pre, float *mean, float *denom, float *stdv, int64_t Tn,
                                                      int64_t F, int64_t lstride) {
  constexpr int V = Elem<T>::VEC;
  constexpr int NU = 4;   // loads in flight per thread
  __shared__ double red[2][8][32 * V];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int64_t l = blockIdx.y, f0 = ((int64_t)blockIdx.x * 32 + tx) * V;
  const T *base = pre + l * lstride;
  const bool on = f0 < F;
  double s1[V], s2[V];
  float piv[V];
#pragma unroll
  for (int j = 0; j < V; ++j) { s1[j] = 0.0; s2[j] = 0.0; piv[j] = 0.0f; }
  auto unpack = [](const uint4 &w, float (&x)[V]) {
    if constexpr (sizeof(T) == 2) {
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) unpack_pair<T>(u[j], x[2 * j], x[2 * j + 1]);
    } else {
      x[0] = __uint_as_float(w.x); x[1] = __uint_as_float(w.y); x[2] = __uint_as_float(w.z); x[3] = __uint_as_float(w.w);
    }
  };
  if (on) {
    unpack(*reinterpret_cast<const uint4 *>(base + f0), piv);
    for (int64_t t0 = ty; t0 < Tn; t0 += 8 * NU) {
      uint4 w[NU];
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        const int64_t t = t0 + (int64_t)u * 8;
        w[u] = t < Tn ? *reinterpret_cast<const uint4 *>(base + t * F + f0) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        if (t0 + (int64_t)u * 8 >= Tn) break;
        float x[V];
        unpack(w[u], x);
#pragma unroll
        for (int j = 0; j < V; ++j) { const double dl = (double)x[j] - (double)piv[j]; s1[j] += dl; s2[j] = fma(dl, dl, s2[j]); }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < V; ++j) { red[0][ty][tx * V + j] = s1[j]; red[1][ty][tx * V + j] = s2[j]; }
  __syncthreads();
  // 256 threads finish the 32 * V columns: thread c < 32 * V takes column c
  const int c = threadIdx.x;
  if (c < 32 * V) {
    const int64_t f = (int64_t)blockIdx.x * 32 * V + c;
    if (f < F) {
      double a = 0.0, q = 0.0;
#pragma unroll
      for (int r = 0; r < 8; ++r) { a += red[0][r][c]; q += red[1][r][c]; }
      const double p = (double)Elem<T>::to_f32(base[f]);
      const double n = (double)Tn;
      const double mu = p + a / n;
      double var = (q - a * a / n) / (n - 1.0);   // T == 1 gives NaN, as torch.std does
      if (var < 0.0) var = 0.0;
      mean[l * F + f] = Elem<T>::round((float)mu);
      const float sd = Elem<T>::round((float)sqrt(var));
      denom[l * F + f] = Elem<T>::round(sd + 1e-6f);
      if (stdv) stdv[l * F + f] = sd;
    }
  }
}

// NaN (all-ones bit pattern) over a buffer when a device flag is set
__global__ void k_poison_if(uint32_t *buf, int64_t bytes, const int32_t *flag) {
  if (*flag == 0) return;
  const int64_t words = bytes / 4;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += (int64_t)gridDim.x * blockDim.x)
    buf[i] = 0xFFFFFFFFu;
  if (blockIdx.x == 0 && threadIdx.x < (unsigned)(bytes - words * 4)) ((uint8_t *)buf)[words * 4 + threadIdx.x] = 0xFFu;
}

}  // namespace

extern "C" int clt_version(void) { return 101; }

extern "C" int clt_poison_if(void *buf, int64_t bytes, const int32_t *flag, void *stream) {
  if (bytes < 0 || !flag || (bytes > 0 && !buf)) return CLT_ERR_ARG;
  if ((((uintptr_t)buf) & 3u) != 0) return CLT_ERR_ALIGN;
  if (bytes == 0) return CLT_OK;
  k_poison_if<<<1024, 256, 0, (hipStream_t)stream>>>((uint32_t *)buf, bytes, flag);
  return clt_check_launch();
}

extern "C" const char *clt_error_string(int code) {
  switch (code) {
    case CLT_OK: return "ok";
    case CLT_ERR_ARG: return "bad argument (null pointer, negative size or unsupported combination)";
    case CLT_ERR_DTYPE: return "dtype must be CLT_F32, CLT_BF16 or CLT_F16 (CLT_F16: forward-path entry points only)";
    case CLT_ERR_WORKSPACE: return "workspace too small";
    case CLT_ERR_LAUNCH: return "HIP reported an error at kernel launch";
    case CLT_ERR_ALIGN: return "pointer or row pitch not aligned as required";
    case CLT_ERR_RANGE: return "size beyond what the kernels index";
    default: return "unknown error code";
  }
}

static int run_colstats(const void *pre, float *mean, float *denom, float *stdv, int64_t T, int64_t F, int64_t L,
                        int64_t pre_layer_stride, int dtype, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || !pre || !mean || !denom) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int V = 16 / clt_elem_bytes(dtype);
  if (F % V == 0 && clt_aligned16(pre) && (pre_layer_stride % V) == 0) {
    dim3 gridv((unsigned)clt_ceil_div(F, 32 * V), (unsigned)L);
    if (dtype == CLT_BF16) k_colstats_vec<bf16_t><<<gridv, 256, 0, s>>>((const bf16_t *)pre, mean, denom, stdv, T, F, pre_layer_stride);
    else if (dtype == CLT_F16) k_colstats_vec<f16_t><<<gridv, 256, 0, s>>>((const f16_t *)pre, mean, denom, stdv, T, F, pre_layer_stride);
    else k_colstats_vec<float><<<gridv, 256, 0, s>>>((const float *)pre, mean, denom, stdv, T, F, pre_layer_stride);
    return clt_check_launch();
  }
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)L);
  if (dtype == CLT_BF16) k_colstats<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)pre, mean, denom, stdv, T, F, pre_layer_stride);
  else if (dtype == CLT_F16) k_colstats<f16_t><<<grid, 256, 0, s>>>((const f16_t *)pre, mean, denom, stdv, T, F, pre_layer_stride);
  else k_colstats<float><<<grid, 256, 0, s>>>((const float *)pre, mean, denom, stdv, T, F, pre_layer_stride);
  return clt_check_launch();
}

extern "C" int clt_colstats(const void *pre, float *mean, float *denom, int64_t T, int64_t F, int64_t L,
                            int64_t pre_layer_stride, int dtype, void *stream) {
  return run_colstats(pre, mean, denom, nullptr, T, F, L, pre_layer_stride, dtype, stream);
}

extern "C" int clt_colstats_full(const void *pre, float *mean, float *stdv, float *denom, int64_t T, int64_t F,
                                 int64_t L, int64_t pre_layer_stride, int dtype, void *stream) {
  if (!stdv) return CLT_ERR_ARG;
  return run_colstats(pre, mean, denom, stdv, T, F, L, pre_layer_stride, dtype, stream);
}

// ---- calibration: what a row gather can reach on this GPU -------------------------------------------
// Every wavefront sums the rows idx[...] of `table` ([n_rows][row_bytes], row_bytes a multiple of 16
// and at most 2048), PROBE_U rows in flight, 16 bytes per lane and load - the access pattern of the
// decode and backward gathers without any of their other work.  With a table that fits every XCD's L2
// this measures the L2 -> CU rate of such a gather; with larger tables, the rate from the memory-side
// cache and from HBM.  out [gridDim.x * 4 * 64] floats receives one value per lane so that the loads
// cannot be dropped.
namespace {
constexpr int PROBE_U = 6;
template <bool TO_LDS>
__global__ __launch_bounds__(256) void k_probe_gather(const uint4 *__restrict__ table, int pieces, const int32_t *__restrict__ idx,
                                                      int64_t n_idx, float *__restrict__ out, int32_t n_rows) {
  // TO_LDS: the same loads issued as direct-to-LDS loads (the encoder's way of bringing tiles in)
  __shared__ __attribute__((aligned(16))) unsigned char lds[TO_LDS ? 4 * PROBE_U * 2 * 1024 : 16];
  const int lane = lane_id(), wv = threadIdx.x >> 6;
  const int64_t nwave = (int64_t)gridDim.x * 4, w = (int64_t)blockIdx.x * 4 + wv;
  const int64_t per = (n_idx + nwave - 1) / nwave, b = w * per, e = b + per < n_idx ? b + per : n_idx;
  const bool on1 = lane + 64 < pieces, on0 = lane < pieces;
  uint32_t acc = 0;
  for (int64_t i0 = b; i0 < e; i0 += 64) {
    const int n = (e - i0) < 64 ? (int)(e - i0) : 64;
    int32_t mine = lane < n ? idx[i0 + lane] : 0;
    mine = mine < 0 ? 0 : (mine >= n_rows ? n_rows - 1 : mine);   // an index outside the table is clamped, never followed
    for (int i = 0; i < n; i += PROBE_U) {
      if constexpr (TO_LDS) {
        unsigned char *mybuf = lds + wv * (PROBE_U * 2 * 1024);
#pragma unroll
        for (int u = 0; u < PROBE_U; ++u) {
          const int k = i + u < n ? i + u : n - 1;
          const uint4 *row = table + (int64_t)__builtin_amdgcn_readlane(mine, k) * pieces;
          // whole 1-KB groups only: a row of 1536 bytes is fetched as 1 KB + the first 512 bytes again
          __builtin_amdgcn_global_load_lds(row + lane, (__attribute__((address_space(3))) void *)(mybuf + u * 2048), 16, 0, 0);
          __builtin_amdgcn_global_load_lds(row + (on1 ? lane + 64 : lane), (__attribute__((address_space(3))) void *)(mybuf + u * 2048 + 1024), 16, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0);
        acc += *reinterpret_cast<const uint32_t *>(mybuf + lane * 4);
      } else {
        uint4 v[PROBE_U][2];
#pragma unroll
        for (int u = 0; u < PROBE_U; ++u) {
          const int k = i + u < n ? i + u : n - 1;
          const uint4 *row = table + (int64_t)__builtin_amdgcn_readlane(mine, k) * pieces;
          v[u][0] = on0 ? row[lane] : make_uint4(0, 0, 0, 0);
          v[u][1] = on1 ? row[lane + 64] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < PROBE_U; ++u)
          acc += v[u][0].x ^ v[u][0].y ^ v[u][0].z ^ v[u][0].w ^ v[u][1].x ^ v[u][1].y ^ v[u][1].z ^ v[u][1].w;
      }
    }
  }
  out[w * 64 + lane] = __uint_as_float(acc & 0x3FFFFFFFu);
}
}  // namespace

extern "C" int clt_probe_gather(const void *table, int64_t n_rows, int64_t row_bytes, const int32_t *idx, int64_t n_idx,
                                int64_t blocks, int to_lds, float *out, void *stream) {
  if (!table || !idx || !out || n_rows <= 0 || n_rows > 2147483647LL || n_idx <= 0 || blocks <= 0 || blocks > 1048576) return CLT_ERR_ARG;
  if (row_bytes <= 0 || row_bytes % 16 != 0 || row_bytes > 2048 || !clt_aligned16(table)) return CLT_ERR_ARG;
  if (to_lds) {
    if (row_bytes < 1024) return CLT_ERR_ARG;   // the direct-to-LDS variant moves whole 1-KB groups
    k_probe_gather<true><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint4 *)table, (int)(row_bytes / 16), idx, n_idx, out, (int32_t)n_rows);
  } else {
    k_probe_gather<false><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint4 *)table, (int)(row_bytes / 16), idx, n_idx, out, (int32_t)n_rows);
  }
  return clt_check_launch();
}
