// Activation-store feed: rows of a stored chunk (or of a fetched slice in the store's wire format
// Layer0_Inputs | Layer0_Targets | Layer1_Inputs | ..., reference
// clt/training/data/manifest_activation_store.py:555-560) are gathered in the sampler's order,
// normalised in fp32 and cast once, straight into the batch slabs x [L][T][d] and targets
// [L][T][d] the encoder and the loss read (reference manifest_activation_store.py:859-934:
// frombuffer, row re-ordering, torch.cat, .float(), (x - mean) / std or x * sqrt(d), .to(dtype)).
// The source may be device memory or pinned host memory: the kernel reads it in place, so a
// host-resident slice crosses the bus once, in its stored width.
#include "clt_common.h"

namespace {

constexpr int FD_THREADS = 256;

template <int SRC> struct Src;   // element decoding by source dtype code
template <> struct Src<CLT_F32> { typedef float T; __device__ static float get(float v) { return v; } };
template <> struct Src<CLT_BF16> { typedef uint16_t T; __device__ static float get(uint16_t v) { return bf16_bits_to_f32(v); } };
template <> struct Src<CLT_F16> {
  typedef uint16_t T;
  __device__ static float get(uint16_t v) { _Float16 h; __builtin_memcpy(&h, &v, 2); return (float)h; }
};

struct FeedNorm {
  int mode;                 // CLT_DENORM_NONE: cast only; _MEAN_STD: (x - mean) / std; _SCALE: x * scale
  const float *mean_in, *std_in, *mean_tg, *std_tg;   // [L][d] fp32
  float scale;
};

__device__ __forceinline__ float feed_norm(float x, int mode, float mean, float stdv, float scale) {
  if (mode == CLT_DENORM_MEAN_STD) return (x - mean) / stdv;
  if (mode == CLT_DENORM_SCALE) return x * scale;
  return x;
}

// grid: x = groups of rows, y = layer * 2 + (0 inputs, 1 targets).  A thread moves V = 8 elements.
template <int SRC, typename OutT>
__global__ __launch_bounds__(FD_THREADS) void k_feed_gather(const typename Src<SRC>::T *__restrict__ src, int64_t src_layer_stride,
                                                            int64_t src_target_offset, const int32_t *__restrict__ row_index,
                                                            int64_t n, int64_t d, FeedNorm nm, OutT *__restrict__ x_out,
                                                            OutT *__restrict__ tgt_out, int64_t out_row0, int64_t Tn,
                                                            int64_t src_rows) {
  typedef typename Src<SRC>::T ST;
  constexpr int V = 8;
  const int64_t l = blockIdx.y >> 1;
  const bool tg = blockIdx.y & 1;
  const ST *sbase = src + l * src_layer_stride + (tg ? src_target_offset : 0);
  OutT *obase = (tg ? tgt_out : x_out) + (l * Tn + out_row0) * d;
  const float *mean = tg ? nm.mean_tg : nm.mean_in, *stdv = tg ? nm.std_tg : nm.std_in;
  const int mode = (nm.mode == CLT_DENORM_MEAN_STD && !(mean && stdv)) ? CLT_DENORM_NONE : nm.mode;
  const int64_t vec_per_row = d / V, total = n * vec_per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t j = i / vec_per_row, c = (i - j * vec_per_row) * V;
    const int64_t r = row_index[j];
    const bool in_range = r >= 0 && r < src_rows;   // a row outside the chunk is never read: it becomes NaN
    const ST *sp = sbase + (in_range ? r : 0) * d + c;
    float x[V];
    if constexpr (sizeof(ST) == 2) {
      const uint4 w = *reinterpret_cast<const uint4 *>(sp);
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) { x[2 * k] = Src<SRC>::get((uint16_t)(u[k] & 0xFFFFu)); x[2 * k + 1] = Src<SRC>::get((uint16_t)(u[k] >> 16)); }
    } else {
      const float4 a = *reinterpret_cast<const float4 *>(sp), b = *reinterpret_cast<const float4 *>(sp + 4);
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
    if (mode == CLT_DENORM_MEAN_STD) {
      const float4 m0 = *reinterpret_cast<const float4 *>(mean + l * d + c), m1 = *reinterpret_cast<const float4 *>(mean + l * d + c + 4);
      const float4 s0 = *reinterpret_cast<const float4 *>(stdv + l * d + c), s1 = *reinterpret_cast<const float4 *>(stdv + l * d + c + 4);
      const float mm[V] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w};
      const float ss[V] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
      for (int k = 0; k < V; ++k) x[k] = (x[k] - mm[k]) / ss[k];
    } else if (mode == CLT_DENORM_SCALE) {
#pragma unroll
      for (int k = 0; k < V; ++k) x[k] *= nm.scale;
    }
    if (!in_range) {
#pragma unroll
      for (int k = 0; k < V; ++k) x[k] = __uint_as_float(0x7FC00000u);
    }
    OutT *op = obase + j * d + c;
    if constexpr (sizeof(OutT) == 2) {
      uint32_t p[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) p[k] = pack_pair<OutT>(x[2 * k], x[2 * k + 1]);
      *reinterpret_cast<uint4 *>(op) = make_uint4(p[0], p[1], p[2], p[3]);
    } else {
      *reinterpret_cast<float4 *>(op) = make_float4(x[0], x[1], x[2], x[3]);
      *reinterpret_cast<float4 *>(op + 4) = make_float4(x[4], x[5], x[6], x[7]);
    }
  }
}

// any d: one element per thread
template <int SRC, typename OutT>
__global__ __launch_bounds__(FD_THREADS) void k_feed_gather_scalar(const typename Src<SRC>::T *__restrict__ src, int64_t src_layer_stride,
                                                                   int64_t src_target_offset, const int32_t *__restrict__ row_index,
                                                                   int64_t n, int64_t d, FeedNorm nm, OutT *__restrict__ x_out,
                                                                   OutT *__restrict__ tgt_out, int64_t out_row0, int64_t Tn,
                                                                   int64_t src_rows) {
  typedef typename Src<SRC>::T ST;
  const int64_t l = blockIdx.y >> 1;
  const bool tg = blockIdx.y & 1;
  const ST *sbase = src + l * src_layer_stride + (tg ? src_target_offset : 0);
  OutT *obase = (tg ? tgt_out : x_out) + (l * Tn + out_row0) * d;
  const float *mean = tg ? nm.mean_tg : nm.mean_in, *stdv = tg ? nm.std_tg : nm.std_in;
  const int mode = (nm.mode == CLT_DENORM_MEAN_STD && !(mean && stdv)) ? CLT_DENORM_NONE : nm.mode;
  const int64_t total = n * d;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t j = i / d, c = i - j * d;
    const int64_t r = row_index[j];
    const bool in_range = r >= 0 && r < src_rows;
    const float x = Src<SRC>::get(sbase[(in_range ? r : 0) * d + c]);
    const float y = !in_range ? __uint_as_float(0x7FC00000u) : feed_norm(x, mode, mode == CLT_DENORM_MEAN_STD ? mean[l * d + c] : 0.0f,
                              mode == CLT_DENORM_MEAN_STD ? stdv[l * d + c] : 1.0f, nm.scale);
    obase[j * d + c] = Elem<OutT>::from_f32(y);
  }
}

template <int SRC, typename OutT>
int launch_feed(const void *src, int64_t src_rows, int64_t src_layer_stride, int64_t src_target_offset, const int32_t *row_index, int64_t n,
                int64_t d, int64_t L, const FeedNorm &nm, void *x_out, void *tgt_out, int64_t out_row0, int64_t T,
                hipStream_t s) {
  typedef typename Src<SRC>::T ST;
  const bool vec = d % 8 == 0 && clt_aligned16(src) && clt_aligned16(x_out) && clt_aligned16(tgt_out) &&
                   (src_layer_stride * (int64_t)sizeof(ST)) % 16 == 0 && (src_target_offset * (int64_t)sizeof(ST)) % 16 == 0 &&
                   (!nm.mean_in || clt_aligned16(nm.mean_in)) && (!nm.std_in || clt_aligned16(nm.std_in)) &&
                   (!nm.mean_tg || clt_aligned16(nm.mean_tg)) && (!nm.std_tg || clt_aligned16(nm.std_tg));
  const int64_t work = vec ? n * (d / 8) : n * d;
  int64_t nb = clt_ceil_div(work, FD_THREADS);
  if (nb > 4096) nb = 4096;
  dim3 grid((unsigned)nb, (unsigned)(2 * L));
  if (vec)
    k_feed_gather<SRC, OutT><<<grid, FD_THREADS, 0, s>>>((const ST *)src, src_layer_stride, src_target_offset, row_index, n, d, nm,
                                                         (OutT *)x_out, (OutT *)tgt_out, out_row0, T, src_rows);
  else
    k_feed_gather_scalar<SRC, OutT><<<grid, FD_THREADS, 0, s>>>((const ST *)src, src_layer_stride, src_target_offset, row_index, n,
                                                                d, nm, (OutT *)x_out, (OutT *)tgt_out, out_row0, T, src_rows);
  return clt_check_launch();
}

}  // namespace

extern "C" int clt_feed_gather(const void *src, int src_dtype, int64_t src_rows, int64_t src_layer_stride,
                               int64_t src_target_offset, const int32_t *row_index, int64_t n, int64_t d, int64_t L,
                               int norm_mode, const float *mean_in, const float *std_in, const float *mean_tg,
                               const float *std_tg, double scale, void *x_out, void *tgt_out, int64_t out_row0, int64_t T,
                               int out_dtype, void *stream) {
  if (!clt_model_dtype(out_dtype)) return CLT_ERR_DTYPE;
  if (src_dtype != CLT_F32 && src_dtype != CLT_BF16 && src_dtype != CLT_F16) return CLT_ERR_DTYPE;
  if (n < 0 || d <= 0 || L <= 0 || L > 32767 || T <= 0 || out_row0 < 0 || out_row0 + n > T || src_rows < 0) return CLT_ERR_ARG;
  if (norm_mode < CLT_DENORM_NONE || norm_mode > CLT_DENORM_SCALE) return CLT_ERR_ARG;
  if (n == 0) return CLT_OK;
  if (!src || !row_index || !x_out || !tgt_out || src_rows == 0) return CLT_ERR_ARG;
  // a layer's inputs and targets must not overlap the next layer's
  if (src_target_offset < src_rows * d || src_layer_stride < src_target_offset + src_rows * d) return CLT_ERR_ARG;
  // the kernel dereferences src: accept only memory the device can reach (device, managed, or pinned host)
  hipPointerAttribute_t at;
  if (hipPointerGetAttributes(&at, src) != hipSuccess) { (void)hipGetLastError(); return CLT_ERR_ARG; }
  if (at.type == hipMemoryTypeHost) {
    if (!at.devicePointer) return CLT_ERR_ARG;
    src = at.devicePointer;
  } else if (at.type != hipMemoryTypeDevice && at.type != hipMemoryTypeManaged) {
    return CLT_ERR_ARG;
  }
  FeedNorm nm{norm_mode, mean_in, std_in, mean_tg, std_tg, (float)scale};
  hipStream_t s = (hipStream_t)stream;
#define CLT_FEED(S)                                                                                                         \
  (out_dtype == CLT_BF16                                                                                                    \
       ? launch_feed<S, bf16_t>(src, src_rows, src_layer_stride, src_target_offset, row_index, n, d, L, nm, x_out, tgt_out, out_row0, T, s) \
   : out_dtype == CLT_F16                                                                                                   \
       ? launch_feed<S, f16_t>(src, src_rows, src_layer_stride, src_target_offset, row_index, n, d, L, nm, x_out, tgt_out, out_row0, T, s) \
       : launch_feed<S, float>(src, src_rows, src_layer_stride, src_target_offset, row_index, n, d, L, nm, x_out, tgt_out, out_row0, T, s))
  if (src_dtype == CLT_F32) return CLT_FEED(CLT_F32);
  if (src_dtype == CLT_BF16) return CLT_FEED(CLT_BF16);
  return CLT_FEED(CLT_F16);
#undef CLT_FEED
}
