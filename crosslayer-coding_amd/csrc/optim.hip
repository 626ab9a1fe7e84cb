// Adam steps (the update itself is in adam.h) with fp32 moments and fp32 gradients on parameters in the
// model dtype.
#include "adam.h"

namespace {

// parameter, gradient and moments in the same layout
template <typename T>
__global__ __launch_bounds__(256) void k_adam(T *__restrict__ p, const float *__restrict__ g, float *__restrict__ m, float *__restrict__ v,
                                              int64_t n, AdamCoef c) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float mi = m[i], vi = v[i];
    const float np = adam_update(Elem<T>::to_f32(p[i]), g[i], mi, vi, c);
    m[i] = mi; v[i] = vi; p[i] = Elem<T>::from_f32(np);
  }
}

// Many small parameters of the same length n (the decoder biases): blockIdx.y picks the parameter,
// gradient and moments are [count][n] slabs.
template <typename T>
__global__ __launch_bounds__(256) void k_adam_many(T *const *params, const float *__restrict__ g, float *__restrict__ m,
                                                   float *__restrict__ v, int64_t n, AdamCoef c) {
  T *p = params[blockIdx.y];
  const int64_t o = (int64_t)blockIdx.y * n;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float mi = m[o + i], vi = v[o + i];
    const float np = adam_update(Elem<T>::to_f32(p[i]), g[o + i], mi, vi, c);
    m[o + i] = mi; v[o + i] = vi; p[i] = Elem<T>::from_f32(np);
  }
}

// Decoder matrix: the parameter lives in the checkpoint layout [d][F]; gradient, moments and the
// feature-major working copy are [F][d].  A block takes a 64 x 64 tile: the update runs on the
// feature-major side (all accesses contiguous), the new values go to the working copy directly and
// to the parameter through an LDS transpose.
template <typename T>
__global__ __launch_bounds__(256) void k_adam_decoder(T *w_ref, T *const *w_refs, T *w_packed, const float *g, float *m, float *v,
                                                      int64_t d, int64_t F, AdamCoef c) {
  __shared__ T tile[64][65];
  // blockIdx.z: decoder of a batch (w_refs holds one parameter pointer per decoder; the other arrays are slabs)
  const int64_t pitch = clt_pitch(d, (int)sizeof(T));   // row pitch of the working copy; gradient and moments are dense
  if (w_refs) { w_ref = w_refs[blockIdx.z]; const int64_t o = (int64_t)blockIdx.z * F * d; w_packed += (int64_t)blockIdx.z * F * pitch; g += o; m += o; v += o; }
  const int64_t f0 = (int64_t)blockIdx.x * 64, d0 = (int64_t)blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int64_t f = f0 + i, dd = d0 + tx;
    if (f < F && dd < d) {
      const int64_t at = f * d + dd, wat = f * pitch + dd;
      float mi = m[at], vi = v[at];
      const T np = Elem<T>::from_f32(adam_update(Elem<T>::to_f32(w_packed[wat]), g[at], mi, vi, c));
      m[at] = mi; v[at] = vi; w_packed[wat] = np;
      tile[i][tx] = np;
    }
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int64_t dd = d0 + i, f = f0 + tx;
    if (dd < d && f < F) w_ref[dd * F + f] = tile[tx][i];
  }
}

// Vector version (d % 4 == 0, F % 4 == 0): a thread updates 4 consecutive elements of a feature row
// (16-byte accesses to gradient and moments) and writes 4 consecutive features of a parameter row.
template <typename T>
__global__ __launch_bounds__(256) void k_adam_decoder_vec(T *__restrict__ w_ref, T *const *__restrict__ w_refs, T *__restrict__ w_packed,
                                                          const float *__restrict__ g, float *__restrict__ m, float *__restrict__ v,
                                                          int64_t d, int64_t F, AdamCoef c) {
  __shared__ T tile[64][68];
  const int64_t pitch = clt_pitch(d, (int)sizeof(T));   // row pitch of the working copy; gradient and moments are dense
  if (w_refs) { w_ref = w_refs[blockIdx.z]; const int64_t o = (int64_t)blockIdx.z * F * d; w_packed += (int64_t)blockIdx.z * F * pitch; g += o; m += o; v += o; }
  const int64_t f0 = (int64_t)blockIdx.x * 64, d0 = (int64_t)blockIdx.y * 64;
  const int q = threadIdx.x & 15, r = threadIdx.x >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int fl = r + 16 * i;
    const int64_t f = f0 + fl, dd = d0 + q * 4;
    if (f < F && dd < d) {
      const int64_t at = f * d + dd, wat = f * pitch + dd;
      const float4 gv = *reinterpret_cast<const float4 *>(g + at);
      float4 mv = *reinterpret_cast<const float4 *>(m + at), vv = *reinterpret_cast<const float4 *>(v + at);
      float p[4];
      if constexpr (sizeof(T) == 2) {
        const uint2 raw = *reinterpret_cast<const uint2 *>(w_packed + wat);
        p[0] = bf16_bits_to_f32(raw.x & 0xFFFFu); p[1] = bf16_bits_to_f32(raw.x >> 16);
        p[2] = bf16_bits_to_f32(raw.y & 0xFFFFu); p[3] = bf16_bits_to_f32(raw.y >> 16);
      } else {
        const float4 raw = *reinterpret_cast<const float4 *>(w_packed + wat);
        p[0] = raw.x; p[1] = raw.y; p[2] = raw.z; p[3] = raw.w;
      }
      p[0] = adam_update(p[0], gv.x, mv.x, vv.x, c); p[1] = adam_update(p[1], gv.y, mv.y, vv.y, c);
      p[2] = adam_update(p[2], gv.z, mv.z, vv.z, c); p[3] = adam_update(p[3], gv.w, mv.w, vv.w, c);
      *reinterpret_cast<float4 *>(m + at) = mv;
      *reinterpret_cast<float4 *>(v + at) = vv;
      T np[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) { np[k] = Elem<T>::from_f32(p[k]); tile[fl][q * 4 + k] = np[k]; }
      if constexpr (sizeof(T) == 2)
        *reinterpret_cast<uint2 *>(w_packed + wat) = make_uint2((uint32_t)np[0] | ((uint32_t)np[1] << 16), (uint32_t)np[2] | ((uint32_t)np[3] << 16));
      else
        *reinterpret_cast<float4 *>(w_packed + wat) = make_float4(np[0], np[1], np[2], np[3]);
    }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int dl = r + 16 * i;
    const int64_t dd = d0 + dl, f = f0 + q * 4;
    if (dd < d && f < F) {
      T o[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) o[k] = tile[q * 4 + k][dl];
      if constexpr (sizeof(T) == 2)
        *reinterpret_cast<uint2 *>(w_ref + dd * F + f) = make_uint2((uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16));
      else
        *reinterpret_cast<float4 *>(w_ref + dd * F + f) = make_float4(o[0], o[1], o[2], o[3]);
    }
  }
}

}  // namespace

extern "C" int clt_adam_step(void *param, const float *grad, float *m, float *v, int64_t n, double lr, double beta1,
                             double beta2, double eps, int64_t step, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (n < 0 || step < 1 || !(beta1 >= 0 && beta1 < 1) || !(beta2 >= 0 && beta2 < 1)) return CLT_ERR_ARG;
  if (n == 0) return CLT_OK;
  if (!param || !grad || !m || !v) return CLT_ERR_ARG;
  const AdamCoef c = adam_coef(lr, beta1, beta2, eps, step);
  hipStream_t s = (hipStream_t)stream;
  int64_t nb = clt_ceil_div(n, 256);
  if (nb > 256 * 64) nb = 256 * 64;
  if (dtype == CLT_BF16) k_adam<bf16_t><<<(unsigned)nb, 256, 0, s>>>((bf16_t *)param, grad, m, v, n, c);
  else k_adam<float><<<(unsigned)nb, 256, 0, s>>>((float *)param, grad, m, v, n, c);
  return clt_check_launch();
}

static int adam_decoders(void *w_ref, void *const *w_refs_dev, int64_t n_dec, bool refs_aligned, void *w_packed,
                         const float *grad_packed, float *m, float *v, int64_t d, int64_t F, double lr, double beta1,
                         double beta2, double eps, int64_t step, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (d <= 0 || F <= 0 || step < 1 || !(beta1 >= 0 && beta1 < 1) || !(beta2 >= 0 && beta2 < 1)) return CLT_ERR_ARG;
  if (!w_packed || !grad_packed || !m || !v || n_dec < 1 || n_dec > 65535) return CLT_ERR_ARG;
  if (clt_ceil_div(d, 64) > 65535) return CLT_ERR_RANGE;
  const AdamCoef c = adam_coef(lr, beta1, beta2, eps, step);
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)clt_ceil_div(d, 64), (unsigned)n_dec);
  const bool vec = d % 4 == 0 && F % 4 == 0 && refs_aligned && clt_aligned16(w_packed) && clt_aligned16(grad_packed) &&
                   clt_aligned16(m) && clt_aligned16(v);
  if (dtype == CLT_BF16) {
    if (vec) k_adam_decoder_vec<bf16_t><<<grid, 256, 0, s>>>((bf16_t *)w_ref, (bf16_t *const *)w_refs_dev, (bf16_t *)w_packed, grad_packed, m, v, d, F, c);
    else k_adam_decoder<bf16_t><<<grid, 256, 0, s>>>((bf16_t *)w_ref, (bf16_t *const *)w_refs_dev, (bf16_t *)w_packed, grad_packed, m, v, d, F, c);
  } else {
    if (vec) k_adam_decoder_vec<float><<<grid, 256, 0, s>>>((float *)w_ref, (float *const *)w_refs_dev, (float *)w_packed, grad_packed, m, v, d, F, c);
    else k_adam_decoder<float><<<grid, 256, 0, s>>>((float *)w_ref, (float *const *)w_refs_dev, (float *)w_packed, grad_packed, m, v, d, F, c);
  }
  return clt_check_launch();
}

extern "C" int clt_adam_step_decoder(void *w_ref, void *w_packed, const float *grad_packed, float *m, float *v, int64_t d,
                                     int64_t F, double lr, double beta1, double beta2, double eps, int64_t step, int dtype,
                                     void *stream) {
  if (!w_ref) return CLT_ERR_ARG;
  return adam_decoders(w_ref, nullptr, 1, clt_aligned16(w_ref), w_packed, grad_packed, m, v, d, F, lr, beta1, beta2, eps,
                       step, dtype, stream);
}

extern "C" int clt_adam_step_decoders(void *const *w_refs_dev, void *const *w_refs_host, int64_t n_dec, void *w_packed,
                                      const float *grad_packed, float *m, float *v, int64_t d, int64_t F, double lr,
                                      double beta1, double beta2, double eps, int64_t step, int dtype, void *stream) {
  if (!w_refs_dev || !w_refs_host || n_dec < 1) return CLT_ERR_ARG;
  bool aligned = true;
  for (int64_t i = 0; i < n_dec; ++i) {
    if (!w_refs_host[i]) return CLT_ERR_ARG;
    aligned = aligned && clt_aligned16(w_refs_host[i]);
  }
  return adam_decoders(nullptr, w_refs_dev, n_dec, aligned, w_packed, grad_packed, m, v, d, F, lr, beta1, beta2, eps, step,
                       dtype, stream);
}

extern "C" int clt_adam_step_many(void *const *params_dev, const float *grad, float *m, float *v, int64_t count, int64_t n,
                                  double lr, double beta1, double beta2, double eps, int64_t step, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (count < 0 || count > 65535 || n < 0 || step < 1 || !(beta1 >= 0 && beta1 < 1) || !(beta2 >= 0 && beta2 < 1)) return CLT_ERR_ARG;
  if (count == 0 || n == 0) return CLT_OK;
  if (!params_dev || !grad || !m || !v) return CLT_ERR_ARG;
  const AdamCoef c = adam_coef(lr, beta1, beta2, eps, step);
  int64_t nb = clt_ceil_div(n, 256);
  if (nb > 1024) nb = 1024;
  dim3 grid((unsigned)nb, (unsigned)count);
  if (dtype == CLT_BF16) k_adam_many<bf16_t><<<grid, 256, 0, (hipStream_t)stream>>>((bf16_t *const *)params_dev, grad, m, v, n, c);
  else k_adam_many<float><<<grid, 256, 0, (hipStream_t)stream>>>((float *const *)params_dev, grad, m, v, n, c);
  return clt_check_launch();
}
