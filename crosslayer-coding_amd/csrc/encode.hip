// Encoder projection  pre[l] = x[l] . W[l]^T + b[l]   (reference clt/models/parallel.py:286)
//
// MFMA kernel for gfx950.  Both operands are K-contiguous (x is [T][d], W is [F][d]), so
// one loader serves both: 16-byte chunks go global -> registers -> LDS, where rows are
// 128 bytes and the chunk index is XOR-swizzled with the row so that the 16-byte
// fragment reads of a wavefront spread over the banks.  The matrix-core "A" operand is
// the W tile and "B" the x tile, so every lane ends up with 4 consecutive features of one
// token per accumulator group and stores them with one 8-byte (bf16) / 16-byte (fp32) write.
//
//   block tile  256 tokens x 128 features, 4 wavefronts (2 x 2), wave tile 128 x 64
//   k step      128 bytes of K per LDS stage (64 bf16 / 32 fp32), next stage prefetched
//               into registers while the current one is multiplied
//   bf16        v_mfma_f32_32x32x16_bf16, fp32 accumulate, one rounding at the store
//   fp32        v_mfma_f32_32x32x2_f32
#include "clt_common.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int BM = 256;   // tokens per block
constexpr int BN = 128;   // features per block
constexpr int ROWB = 128; // bytes of K per LDS row
constexpr int XCH = BM * 8 / 256;  // 16-byte chunks of the x tile per thread
constexpr int WCH = BN * 8 / 256;

__device__ __forceinline__ int lds_off(int row, int ch) { return row * ROWB + ((ch ^ (row & 7)) << 4); }

template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  __device__ static __forceinline__ void run(f32x16_t &acc, const uint4 &a, const uint4 &b) {
    bf16x8_t av = __builtin_bit_cast(bf16x8_t, a), bv = __builtin_bit_cast(bf16x8_t, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
  }
};
template <> struct Mma<float> {
  __device__ static __forceinline__ void run(f32x16_t &acc, const uint4 &a, const uint4 &b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), acc, 0, 0, 0);
  }
};

template <typename T>
__global__ __launch_bounds__(256, 2) void k_encode_mfma(
    const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias, T *__restrict__ pre,
    int M, int K, int N, int tiles_m, int tiles_n, int64_t xs, int64_t wstr, int64_t bs, int64_t ps) {
  constexpr int CE = 16 / (int)sizeof(T);  // elements per 16-byte chunk
  constexpr int BK = ROWB / (int)sizeof(T);
  __shared__ __attribute__((aligned(16))) unsigned char lds[(BM + BN) * ROWB];
  unsigned char *xsm = lds, *wsm = lds + BM * ROWB;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  int bid = blockIdx.x;
  const int per_layer = tiles_m * tiles_n;
  const int layer = bid / per_layer;
  bid -= layer * per_layer;
  const int tn = bid / tiles_m, tm = bid - tn * tiles_m;  // token tiles vary fastest
  const int m0 = tm * BM, n0 = tn * BN;
  const T *xl = x + (int64_t)layer * xs;
  const T *wl = w + (int64_t)layer * wstr;

  const int lrow = tid >> 3, lch = tid & 7;  // loader: row (+32 per step) and chunk of this thread
  uint4 xr[XCH], wr[WCH];
  auto load_stage = [&](int k0) {
    const int kk = k0 + lch * CE;
    const bool kin = kk + CE <= K;
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int row = m0 + lrow + i * 32;
      xr[i] = (kin && row < M) ? *reinterpret_cast<const uint4 *>(xl + (int64_t)row * K + kk) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < WCH; ++i) {
      const int row = n0 + lrow + i * 32;
      wr[i] = (kin && row < N) ? *reinterpret_cast<const uint4 *>(wl + (int64_t)row * K + kk) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_stage = [&]() {
#pragma unroll
    for (int i = 0; i < XCH; ++i) *reinterpret_cast<uint4 *>(xsm + lds_off(lrow + i * 32, lch)) = xr[i];
#pragma unroll
    for (int i = 0; i < WCH; ++i) *reinterpret_cast<uint4 *>(wsm + lds_off(lrow + i * 32, lch)) = wr[i];
  };

  f32x16_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int l31 = lane & 31, lh = lane >> 5;
  load_stage(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    store_stage();
    __syncthreads();
    if (k0 + BK < K) load_stage(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int ch = kk * 2 + lh;
      uint4 xa[4], wa[2];
#pragma unroll
      for (int i = 0; i < 4; ++i) xa[i] = *reinterpret_cast<const uint4 *>(xsm + lds_off(wm * 128 + i * 32 + l31, ch));
#pragma unroll
      for (int j = 0; j < 2; ++j) wa[j] = *reinterpret_cast<const uint4 *>(wsm + lds_off(wn * 64 + j * 32 + l31, ch));
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) Mma<T>::run(acc[i][j], wa[j], xa[i]);
    }
    __syncthreads();
  }

  // epilogue: lane owns token (l31) and, per accumulator group rg, features 8*rg + 4*lh + 0..3
  T *pl = pre + (int64_t)layer * ps;
  const T *bl = bias ? bias + (int64_t)layer * bs : nullptr;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int n = n0 + wn * 64 + j * 32 + rg * 8 + lh * 4;
      if (n >= N) continue;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (bl) {
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[q] = Elem<T>::to_f32(bl[n + q]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 128 + i * 32 + l31;
        if (m >= M) continue;
        float y[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) y[q] = acc[i][j][rg * 4 + q] + bv[q];
        T *po = pl + (int64_t)m * N + n;
        if (sizeof(T) == 4) {
          *reinterpret_cast<float4 *>(po) = make_float4(y[0], y[1], y[2], y[3]);
        } else {
          uint2 o;
          o.x = f32_to_bf16_bits(y[0]) | (f32_to_bf16_bits(y[1]) << 16);
          o.y = f32_to_bf16_bits(y[2]) | (f32_to_bf16_bits(y[3]) << 16);
          *reinterpret_cast<uint2 *>(po) = o;
        }
      }
    }
  }
}

// Any shape: one thread per output, fp32 accumulation.
template <typename T>
__global__ void k_encode_generic(const T *x, const T *w, const T *bias, T *pre, int64_t M, int64_t K, int64_t N,
                                 int64_t L, int64_t xs, int64_t wstr, int64_t bs, int64_t ps) {
  const int64_t total = M * N * L;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t l = i / (M * N), rem = i - l * M * N, m = rem / N, n = rem - m * N;
    const T *xr = x + l * xs + m * K, *wr = w + l * wstr + n * K;
    float acc = 0.0f;
    for (int64_t k = 0; k < K; ++k) acc = fmaf(Elem<T>::to_f32(xr[k]), Elem<T>::to_f32(wr[k]), acc);
    if (bias) acc += Elem<T>::to_f32(bias[l * bs + n]);
    pre[l * ps + m * N + n] = Elem<T>::from_f32(acc);
  }
}

template <typename T>
static int launch_encode(const void *x, const void *w, const void *b, void *pre, int64_t T_, int64_t d, int64_t F,
                         int64_t L, int64_t xs, int64_t wstr, int64_t bs, int64_t ps, hipStream_t stream) {
  constexpr int CE = 16 / (int)sizeof(T);
  const bool fast = (d % CE == 0) && (F % 4 == 0) && clt_aligned16(x) && clt_aligned16(w) && clt_aligned16(pre) &&
                    (xs % CE == 0) && (wstr % CE == 0) && (ps % 4 == 0) && (ps * (int64_t)sizeof(T)) % 16 == 0 &&
                    (F * (int64_t)sizeof(T)) % 8 == 0 && T_ < (1 << 30) && F < (1 << 30) && d < (1 << 30) &&
                    (!b || (((uintptr_t)b) % 8 == 0 && bs % 4 == 0));
  if (fast) {
    const int64_t tm = clt_ceil_div(T_, BM), tn = clt_ceil_div(F, BN);
    const int64_t nblk = tm * tn * L;
    if (nblk > 2147483647LL) return CLT_ERR_RANGE;
    k_encode_mfma<T><<<(unsigned)nblk, 256, 0, stream>>>((const T *)x, (const T *)w, (const T *)b, (T *)pre, (int)T_,
                                                         (int)d, (int)F, (int)tm, (int)tn, xs, wstr, bs, ps);
  } else {
    k_encode_generic<T><<<256 * 8, 256, 0, stream>>>((const T *)x, (const T *)w, (const T *)b, (T *)pre, T_, d, F, L,
                                                     xs, wstr, bs, ps);
  }
  return clt_check_launch();
}

}  // namespace

extern "C" int clt_encode(const void *x, const void *w, const void *b, void *pre, int64_t T, int64_t d, int64_t F,
                          int64_t L, int64_t x_layer_stride, int64_t w_layer_stride, int64_t b_layer_stride,
                          int64_t pre_layer_stride, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T < 0 || d <= 0 || F <= 0 || L <= 0) return CLT_ERR_ARG;
  if (T == 0) return CLT_OK;
  if (!x || !w || !pre) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16)
    return launch_encode<bf16_t>(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride, pre_layer_stride, s);
  return launch_encode<float>(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride, pre_layer_stride, s);
}
