// Library identity, error text, and the per-feature ranking statistics of the global
// BatchTopK / TokenTopK helper (reference clt/models/activations.py:281-283).
#include "clt_common.h"

namespace {

// One block = 64 feature columns x 4 row groups; two passes over the column
// (mean, then centred sum of squares) with double accumulation.
template <typename T>
__global__ __launch_bounds__(256) void k_colstats(const T *pre, float *mean, float *denom, int64_t Tn, int64_t F,
                                                  int64_t lstride) {
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
  }
}

}  // namespace

extern "C" int clt_version(void) { return 100; }

extern "C" const char *clt_error_string(int code) {
  switch (code) {
    case CLT_OK: return "ok";
    case CLT_ERR_ARG: return "bad argument (null pointer, negative size or unsupported combination)";
    case CLT_ERR_DTYPE: return "dtype must be CLT_F32 or CLT_BF16";
    case CLT_ERR_WORKSPACE: return "workspace too small";
    case CLT_ERR_LAUNCH: return "HIP reported an error at kernel launch";
    case CLT_ERR_ALIGN: return "pointer or row pitch not aligned as required";
    case CLT_ERR_RANGE: return "size beyond what the kernels index";
    default: return "unknown error code";
  }
}

extern "C" int clt_colstats(const void *pre, float *mean, float *denom, int64_t T, int64_t F, int64_t L,
                            int64_t pre_layer_stride, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || !pre || !mean || !denom) return CLT_ERR_ARG;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)L);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) k_colstats<bf16_t><<<grid, 256, 0, s>>>((const bf16_t *)pre, mean, denom, T, F, pre_layer_stride);
  else k_colstats<float><<<grid, 256, 0, s>>>((const float *)pre, mean, denom, T, F, pre_layer_stride);
  return clt_check_launch();
}
