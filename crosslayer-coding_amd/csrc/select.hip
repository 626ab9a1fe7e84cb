// BatchTopK selection and threshold activations -> compact survivor lists.
//
// BatchTopK (reference clt/models/activations.py:11-36, 261-357) is an exact
// "K largest of N" with deterministic ties.  N is 1e8..1e9 and K is ~1 % of it, so
// the work is one streaming read of the pre-activations:
//
//   sample   a hashed sample of the ranking values gives a conservative cut key
//            (about 2x K elements lie above it);
//   pass     ONE read of every row (one wavefront per row, four 16-byte loads in flight
//            per lane): elements at or above the cut are collected, in column order (wave
//            ballot + mbcnt prefix), in an LDS buffer of the wavefront, counted into an
//            LDS histogram of (key - cut), and flushed in coalesced extents to a
//            candidate pool (one atomic per extent; a row's extents are chained);
//   scan     a single block walks the histogram from the top and finds the bin that
//            holds the K-th largest key; bins are one key wide near the cut (16-bit
//            keys) so this usually ends the search, otherwise further levels
//            re-histogram the candidates only;
//   count / allot / emit   work on the candidate pool: survivors per row, the tie
//            budget handed out in flat-index order, then the ordered write of
//            (feature, value) pairs.
//
// A row that could not get pool space is re-read from the dense matrix by the later
// stages, and a cut that turns out too high (fewer than K candidates) makes the pass run
// again with the lowest cut, so the result is exact for any input; only the speed depends
// on the sample being representative.
#include "select_state.h"
#include <mutex>

namespace {

constexpr int NBINS = 2048;
constexpr uint32_t FINE16 = 1984;  // 16-bit keys: bins [0,FINE16) are one key wide
constexpr int SAMPLE_N = 16384;
constexpr int SAMPLE_WAVES = 64;         // sample taken before the pre-activations exist: wavefronts per layer,
constexpr int SAMPLE_PRE_N = SAMPLE_WAVES * 1024;   // each 32 hashed tokens x 32 hashed features
constexpr int SAMPLE_BLOCKS = 16;        // blocks per problem that gather the sample
constexpr int SCAN_THREADS = 1024;
constexpr int WBUF = 512;                // candidate entries buffered in LDS per wavefront
constexpr int PASS_NV = 4;               // 16-byte loads in flight per lane in the pass
constexpr int TOK_MAX_LAYERS = 1024;         // layers of a TokenTopK problem (per-layer counters in LDS)
constexpr uint32_t ROW_NONE = 0xFFFFFFFFu;   // row has no candidates
constexpr uint32_t ROW_DENSE = 0xFFFFFFFEu;  // row did not fit the pool: read it from the matrix

template <int KB> __device__ __forceinline__ uint32_t min_key() {
  return KB == 32 ? 0x007FFFFFu : 0x007Fu;  // key(-inf); nothing ranks below it
}
// key(-inf) of the element type
template <typename T> __device__ __forceinline__ uint32_t min_key_of() {
  return IsHalf<T>::value ? 0x03FFu : min_key<Elem<T>::KEYBITS>();
}
template <int KB> __device__ __forceinline__ uint32_t bin_level0(uint32_t diff) {
  if (KB == 16) return diff < FINE16 ? diff : FINE16 + (diff >> 10);
  return diff >> 21;
}

// ---- ranking value ---------------------------------------------------------------
struct RankRaw {
  __device__ __forceinline__ float operator()(float x, int64_t) const { return x; }
};
// z-score in the model dtype: round(round(x - mean) / denom)  (activations.py:283)
template <typename T> struct RankZ {
  const float *mean, *denom;  // this layer's rows of the [L][F] statistics
  __device__ __forceinline__ float operator()(float x, int64_t col) const {
    float a = Elem<T>::round(x - mean[col]);
    return Elem<T>::round(a / denom[col]);
  }
};
template <typename T, bool GLOBAL> struct RankOf;
template <typename T> struct RankOf<T, false> {
  typedef RankRaw type;
  __device__ static RankRaw make(const float *, const float *, int64_t, int64_t) { return RankRaw(); }
};
template <typename T> struct RankOf<T, true> {
  typedef RankZ<T> type;
  __device__ static RankZ<T> make(const float *mean, const float *denom, int64_t l, int64_t F) {
    RankZ<T> r; r.mean = mean + l * F; r.denom = denom + l * F; return r;
  }
};

// ---- vector loads -----------------------------------------------------------------
template <typename T, int V> struct VecLoad;
template <> struct VecLoad<float, 4> {
  __device__ static __forceinline__ void load(const float *p, float (&x)[4], uint32_t (&raw)[4]) {
    float4 v = *reinterpret_cast<const float4 *>(p);
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
#pragma unroll
    for (int j = 0; j < 4; ++j) raw[j] = __float_as_uint(x[j]);
  }
};
template <> struct VecLoad<float, 1> {
  __device__ static __forceinline__ void load(const float *p, float (&x)[1], uint32_t (&raw)[1]) {
    x[0] = *p; raw[0] = __float_as_uint(x[0]);
  }
};
template <> struct VecLoad<bf16_t, 8> {
  __device__ static __forceinline__ void load(const bf16_t *p, float (&x)[8], uint32_t (&raw)[8]) {
    uint4 v = *reinterpret_cast<const uint4 *>(p);
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      raw[2 * j] = w[j] & 0xFFFFu; raw[2 * j + 1] = w[j] >> 16;
      x[2 * j] = __uint_as_float(w[j] << 16); x[2 * j + 1] = __uint_as_float(w[j] & 0xFFFF0000u);
    }
  }
};
template <> struct VecLoad<f16_t, 8> {
  __device__ static __forceinline__ void load(const f16_t *p, float (&x)[8], uint32_t (&raw)[8]) {
    uint4 v = *reinterpret_cast<const uint4 *>(p);
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      raw[2 * j] = w[j] & 0xFFFFu; raw[2 * j + 1] = w[j] >> 16;
      unpack_pair<f16_t>(w[j], x[2 * j], x[2 * j + 1]);
    }
  }
};
template <> struct VecLoad<f16_t, 1> {
  __device__ static __forceinline__ void load(const f16_t *p, float (&x)[1], uint32_t (&raw)[1]) {
    raw[0] = p->bits; x[0] = f16_bits_to_f32(raw[0]);
  }
};
template <> struct VecLoad<bf16_t, 1> {
  __device__ static __forceinline__ void load(const bf16_t *p, float (&x)[1], uint32_t (&raw)[1]) {
    raw[0] = *p; x[0] = bf16_bits_to_f32(raw[0]);
  }
};

// exclusive prefix over the wave (lane order, then bit order) of the set bits of m
template <int V> __device__ __forceinline__ uint32_t wave_mask_prefix(uint32_t m, uint32_t &total) {
  uint32_t pre = 0; total = 0;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    uint64_t b = ballot64((m >> j) & 1u);
    pre += mbcnt64(b);
    total += (uint32_t)__popcll(b);
  }
  return pre;
}

// ---- block scan helper --------------------------------------------------------------
// Walks hist[nb-1] .. hist[0] and finds the bin where the running count first reaches k.
// All SCAN_THREADS threads call it; returns false when the histogram holds fewer than k.
__device__ bool block_find_from_top(const uint32_t *hist, int nb, unsigned long long k,
                                    int &bin_out, unsigned long long &above_out,
                                    unsigned long long &total_out) {
  __shared__ unsigned long long wsum[SCAN_THREADS / CLT_WAVE];
  __shared__ int s_bin;
  __shared__ unsigned long long s_above, s_total;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  int b0 = nb - 1 - 2 * tid, b1 = nb - 2 - 2 * tid;
  unsigned long long h0 = b0 >= 0 ? hist[b0] : 0, h1 = b1 >= 0 ? hist[b1] : 0;
  unsigned long long s = h0 + h1, inc = s;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    unsigned long long y = __shfl_up(inc, o);
    if (lane >= o) inc += y;
  }
  if (tid == 0) { s_bin = -1; s_above = 0; }
  if (lane == 63) wsum[wv] = inc;
  __syncthreads();
  unsigned long long base = 0, tot = 0;
  for (int i = 0; i < SCAN_THREADS / CLT_WAVE; ++i) {
    unsigned long long w = wsum[i];
    if (i < wv) base += w;
    tot += w;
  }
  unsigned long long excl = base + inc - s, incl = base + inc;
  if (k > 0 && excl < k && k <= incl) {
    if (excl + h0 >= k) { s_bin = b0; s_above = excl; }
    else { s_bin = b1; s_above = excl + h0; }
  }
  if (tid == 0) s_total = tot;
  __syncthreads();
  bin_out = s_bin; above_out = s_above; total_out = s_total;
  bool ok = s_bin >= 0;
  __syncthreads();
  return ok;
}

// ---- kernels ------------------------------------------------------------------------
__global__ void k_fill_u32(uint32_t *p, uint32_t v, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}

__device__ __forceinline__ uint64_t hash_index(uint64_t i, uint64_t n) {
  uint64_t x = (i + 1) * 0x9E3779B97F4A7C15ull;
  x ^= x >> 29; x *= 0xBF58476D1CE4E5B9ull; x ^= x >> 32;
  return __umul64hi(x, n);
}

// SAMPLE_BLOCKS blocks per problem: ranking keys of a hashed sample.
template <typename T, bool GLOBAL>
__global__ __launch_bounds__(256) void k_sample_keys(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, unsigned long long N, uint32_t *sample) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int p = blockIdx.y;
  const unsigned long long ns = N < (unsigned long long)SAMPLE_N ? N : (unsigned long long)SAMPLE_N;
  for (unsigned long long si = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; si < ns;
       si += (unsigned long long)gridDim.x * blockDim.x) {
    unsigned long long idx = (ns == N) ? si : hash_index(si, N);
    int64_t l, t, f;
    if (GLOBAL) { int64_t rowlen = L * F; t = idx / rowlen; int64_t rem = idx - t * rowlen; l = rem / F; f = rem - l * F; }
    else { l = p; t = idx / F; f = idx - t * F; }
    float x = Elem<T>::to_f32(pre[l * lstride + t * F + f]);
    typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
    sample[(int64_t)p * SAMPLE_N + si] = rank_key_of<T>(rk(x, f));
  }
}

// One block per problem: the cut key = the r-th largest sample key, r chosen so that the
// expected number of elements above the cut is about 1.25 K plus six standard deviations.
// Also resets the problem's histogram, pool counter and state.
template <typename T, int SN>
__global__ __launch_bounds__(SCAN_THREADS) void k_sample_cut(
    const uint32_t *sample, unsigned long long N, unsigned long long K, SelState *st, uint32_t *hist,
    uint32_t *pool_count, uint32_t *aux_count, uint32_t path) {
  constexpr int KB = Elem<T>::KEYBITS;
  constexpr int PER = SN / SCAN_THREADS;
  __shared__ uint32_t lh[NBINS];
  const int p = blockIdx.x, tid = threadIdx.x;
  const unsigned long long ns = N < (unsigned long long)SN ? N : (unsigned long long)SN;
  for (int i = tid; i < NBINS; i += SCAN_THREADS) hist[(int64_t)p * NBINS + i] = 0;
  if (tid == 0) { pool_count[p] = 0; if (aux_count) aux_count[p] = 0; }
  uint32_t keys[PER];
  bool valid[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    unsigned long long si = (unsigned long long)tid + (unsigned long long)i * SCAN_THREADS;
    valid[i] = si < ns;
    keys[i] = valid[i] ? sample[(int64_t)p * SN + si] : 0u;
  }
  unsigned long long r;
  if (ns == N && path != PATH_TILES) r = K;   // the sample is the whole problem
  else {
    double e = (double)K / (double)N * (double)ns;
    // the sample taken ahead of the projection (PATH_TILES) is four times larger and made of 32 x 32
    // blocks of tokens x features: a smaller relative margin, the same six standard deviations
    r = path == PATH_TILES ? (unsigned long long)(1.2 * e + 6.0 * sqrt(e) + 16.0) + 1
                           : (unsigned long long)(1.25 * e + 6.0 * sqrt(e) + 16.0) + 1;
  }
  uint32_t cut = min_key_of<T>();
  if (r <= ns && r > 0) {
    constexpr int NLEV = KB == 32 ? 3 : 2;
    const int shifts[3] = {KB == 32 ? 21 : 5, KB == 32 ? 10 : 0, 0};
    const int widths[3] = {11, KB == 32 ? 11 : 5, 10};
    uint32_t prefix = 0, prefix_mask = 0;  // decided high bits
    unsigned long long k_rem = r;
    for (int lev = 0; lev < NLEV; ++lev) {
      for (int i = tid; i < NBINS; i += SCAN_THREADS) lh[i] = 0;
      __syncthreads();
      const int sh = shifts[lev];
      const uint32_t dm = (1u << widths[lev]) - 1u;
#pragma unroll
      for (int i = 0; i < PER; ++i)
        if (valid[i] && (keys[i] & prefix_mask) == prefix) atomicAdd(&lh[(keys[i] >> sh) & dm], 1u);
      __syncthreads();
      int bin; unsigned long long above, total;
      block_find_from_top(lh, (int)dm + 1, k_rem, bin, above, total);
      if (bin < 0) bin = 0;  // cannot happen (r <= ns); keep the cut low if it does
      k_rem -= above;
      prefix |= (uint32_t)bin << sh;
      prefix_mask |= dm << sh;
    }
    cut = prefix;
    if (cut < min_key_of<T>()) cut = min_key_of<T>();
  }
  if (tid == 0) {
    SelState s;
    s.cut_key = cut; s.status = ST_RUN; s.level = 0; s.flo = 0; s.fhi = 0; s.bbase = 0; s.shift = 0;
    s.thr_key = 0; s.k_rem = K; s.tie_budget = 0; s.path = path; s.overflow = 0;
    st[p] = s;
  }
}

// Inclusive prefix sum over the 64 lanes of a wavefront with DPP row shifts / broadcasts.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return v;
}

// 16 bytes of a row as loaded, and the float value of element j of it.
template <typename T> __device__ __forceinline__ float vec_elem(const uint4 &w, int j);
template <> __device__ __forceinline__ float vec_elem<float>(const uint4 &w, int j) {
  return __uint_as_float(j == 0 ? w.x : j == 1 ? w.y : j == 2 ? w.z : w.w);
}
template <> __device__ __forceinline__ float vec_elem<bf16_t>(const uint4 &w, int j) {
  const uint32_t u = (j >> 1) == 0 ? w.x : (j >> 1) == 1 ? w.y : (j >> 1) == 2 ? w.z : w.w;
  return __uint_as_float((j & 1) ? (u & 0xFFFF0000u) : (u << 16));
}

template <> __device__ __forceinline__ float vec_elem<f16_t>(const uint4 &w, int j) {
  const uint32_t u = (j >> 1) == 0 ? w.x : (j >> 1) == 1 ? w.y : (j >> 1) == 2 ? w.z : w.w;
  return f16_bits_to_f32((j & 1) ? (u >> 16) : (u & 0xFFFFu));
}

// Global ranking: for every (layer, feature) the lowest value x whose z-score reaches the cut
// key (binary search over the ordered keys of the element type; the z-score with its two
// roundings is monotone in x).  NaN when only a NaN reaches the cut.
template <typename T>
__global__ __launch_bounds__(256) void k_col_cut(const float *mean, const float *denom, const SelState *st, int64_t F,
                                                 int64_t L, T *xcut) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= L * F) return;
  const uint32_t cut_key = st[0].cut_key;
  RankZ<T> rk; rk.mean = mean; rk.denom = denom;   // indexed with the flat (layer, feature) position
  uint32_t lo = min_key_of<T>(), hi = KB == 32 ? 0xFFFFFFFFu : 0xFFFFu;
  while (lo < hi) {
    const uint32_t mid = lo + ((hi - lo) >> 1);
    const float xv = __uint_as_float(key_value_bits<T>(mid));
    if (rank_key_of<T>(rk(xv, i)) >= cut_key) hi = mid; else lo = mid + 1u;
  }
  const uint32_t bits = key_value_bits<T>(lo);
  xcut[i] = Elem<T>::from_f32(__uint_as_float(bits));   // exact: the value is one of T
}

// The streaming pass: one wavefront per row.  A step covers PASS_NV vectors of 64 lanes x 16
// bytes.  Lanes keep a bit per element that reaches the cut; when any lane has one, the raw
// vectors are staged in LDS (column order), two packed prefix scans give every candidate its
// place in column order, each lane writes the columns of its set bits, and then the lanes
// finish the candidates in parallel (value, histogram).
template <typename T, int V, bool GLOBAL>
__global__ __launch_bounds__(256) void k_select_pass(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, const SelState *st, uint32_t *hist, uint32_t *pool_count, uint2 *pool,
    unsigned long long pool_cap, uint32_t *row_first, int phase, const T *xcut) {
  constexpr int KB = Elem<T>::KEYBITS;
  static_assert(PASS_NV == 4, "the packed prefix below holds four 16-bit fields");
  constexpr int STEP = PASS_NV * 64 * V;  // elements per step
  __shared__ uint32_t lh[NBINS];
  __shared__ uint2 wbuf_all[4][WBUF];
  __shared__ __attribute__((aligned(16))) T stage_all[4][STEP];
  const int l = blockIdx.y, p = GLOBAL ? 0 : l;
  const uint32_t status = st[p].status;
  if (phase == 0 ? status != ST_RUN : status != ST_RETRY) return;
  const uint32_t cut_key = st[p].cut_key;
  const uint32_t cut_bits = key_value_bits<T>(cut_key);
  const float cutf = __uint_as_float(cut_bits);
  const bool cut_nan = (cut_bits & 0x7FFFFFFFu) > 0x7F800000u;  // only NaNs reach such a cut
  for (int i = threadIdx.x; i < NBINS; i += blockDim.x) lh[i] = 0;
  __syncthreads();
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  uint2 *wbuf = wbuf_all[wv];
  T *stage = stage_all[wv];
  uint2 *mypool = pool + (unsigned long long)p * pool_cap;
  typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    const int64_t r = (int64_t)l * Tn + t;
    const T *row = pre + l * lstride + t * F;
    uint32_t n_buf = 0, first = ROW_NONE, prev = ROW_NONE;
    bool dense = false;
    auto flush = [&]() {
      if (n_buf == 0) return;
      if (!dense) {
        uint32_t off = 0;
        if (lane == 0) off = atomicAdd(&pool_count[p], n_buf + 1u);
        off = __builtin_amdgcn_readfirstlane(off);
        if ((unsigned long long)off + n_buf + 1ull > pool_cap) dense = true;
        else {
          if (lane == 0) {
            mypool[off] = make_uint2(ROW_NONE, n_buf);           // extent header: (next, count)
            if (prev != ROW_NONE) mypool[prev].x = off;
          }
          if (prev == ROW_NONE) first = off;
          prev = off;
          for (uint32_t i = lane; i < n_buf; i += 64) mypool[off + 1u + i] = wbuf[i];
        }
      }
      n_buf = 0;
    };
    // global ranking, first pass: the z-score is monotone in x, so "z reaches the cut" is
    // "x reaches the column's own bound" (k_col_cut), one compare instead of a division
    const bool by_column = GLOBAL && V > 1 && phase == 0 && xcut != nullptr;
    for (int64_t c0 = 0; c0 < F; c0 += STEP) {
      // all loads of the step - values and, when ranking by column, the bounds - go out together,
      // unpredicated (a vector past the end of the row reads the row's start and is masked below)
      uint4 w[PASS_NV], xc[PASS_NV];
      bool on[PASS_NV];
#pragma unroll
      for (int q = 0; q < PASS_NV; ++q) {
        const int64_t col = c0 + (int64_t)q * 64 * V + (int64_t)lane * V;
        on[q] = col < F;
        const int64_t cl = on[q] ? col : 0;
        if (V > 1) w[q] = *reinterpret_cast<const uint4 *>(row + cl);
        else w[q] = make_uint4(sizeof(T) == 2 ? ((uint32_t)Elem<T>::raw(row[cl]) << 16) : (uint32_t)Elem<T>::raw(row[cl]), 0, 0, 0);
        xc[q] = make_uint4(0, 0, 0, 0);
        if (V > 1 && by_column) xc[q] = *reinterpret_cast<const uint4 *>(xcut + (int64_t)l * F + cl);
      }
      uint32_t m = 0;  // bit q*V + j: element j of vector q reaches the cut
#pragma unroll
      for (int q = 0; q < PASS_NV; ++q) {
        const int64_t col = c0 + (int64_t)q * 64 * V + (int64_t)lane * V;
        uint32_t mq = 0;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float xv = V > 1 ? vec_elem<T>(w[q], j) : Elem<T>::to_f32(Elem<T>::from_raw(sizeof(T) == 2 ? (w[q].x >> 16) : w[q].x));
          bool c;
          if (by_column) c = xv >= vec_elem<T>(xc[q], j) || xv != xv;
          else {
            const float rv = rk(xv, col + j);
            c = cut_nan ? (rv != rv) : !(rv < cutf);
          }
          mq |= (c ? 1u : 0u) << j;
        }
        if (on[q]) m |= mq << (q * V);
      }
      if (ballot64(m != 0) == 0) continue;
      // stage the step in column order: stage[col - c0]
#pragma unroll
      for (int q = 0; q < PASS_NV; ++q) {
        if (V > 1) *reinterpret_cast<uint4 *>(stage + (q * 64 + lane) * V) = w[q];
        else stage[q * 64 + lane] = Elem<T>::from_raw(sizeof(T) == 2 ? (w[q].x >> 16) : w[q].x);
      }
      // per-vector counts, packed 16 bits each, prefix-summed over the lanes
      constexpr uint32_t FM = (1u << V) - 1u;
      const uint32_t cA = __popc(m & FM) | (__popc((m >> V) & FM) << 16);
      const uint32_t cB = __popc((m >> (2 * V)) & FM) | (__popc((m >> (3 * V)) & FM) << 16);
      const uint32_t iA = wave_inclusive_scan(cA), iB = wave_inclusive_scan(cB);
      const uint32_t tA = __builtin_amdgcn_readlane(iA, 63), tB = __builtin_amdgcn_readlane(iB, 63);
      const uint32_t t0 = tA & 0xFFFFu, t1 = tA >> 16, t2 = tB & 0xFFFFu, t3 = tB >> 16;
      const uint32_t total = t0 + t1 + t2 + t3;
      if (n_buf + total > (uint32_t)WBUF) flush();
      const bool fits = total <= (uint32_t)WBUF;
      // start of each vector's candidates in the buffer, plus this lane's exclusive prefix
      const uint32_t sA = (iA - cA) + (n_buf | ((n_buf + t0) << 16));
      const uint32_t sB = (iB - cB) + ((n_buf + t0 + t1) | ((n_buf + t0 + t1 + t2) << 16));
      const uint32_t c0u = (uint32_t)c0;
      // the lanes finish `cnt` new entries (step-relative columns at wbuf[n_buf ..]) in parallel
      auto finish = [&](uint32_t cnt) {
        for (uint32_t i = lane; i < cnt; i += 64) {
          const uint32_t rel = wbuf[n_buf + i].x;
          const T rawv = stage[rel];
          const uint32_t col = c0u + rel;
          const uint32_t key = rank_key_of<T>(rk(Elem<T>::to_f32(rawv), (int64_t)col));
          atomicAdd(&lh[bin_level0<KB>(key - cut_key)], 1u);
          wbuf[n_buf + i] = make_uint2(col, Elem<T>::raw(rawv));
        }
        n_buf += cnt;
      };
      if (fits) {
        // each lane drops the step-relative column of its candidates at their ordered slots
        uint32_t mm = m;
        while (ballot64(mm != 0)) {
          if (mm) {
            const int bit = __ffs(mm) - 1;
            mm &= mm - 1u;
            const int q = bit / V;
            const uint32_t sw = q < 2 ? sA : sB;
            const uint32_t start = (q & 1) ? (sw >> 16) : (sw & 0xFFFFu);
            const uint32_t below = __popc(m & ((1u << bit) - 1u) & (FM << (q * V)));
            wbuf[start + below].x = (uint32_t)(q * 64 * V + lane * V + (bit % V));
          }
        }
        finish(total);
      } else {
        // A step with more candidates than the buffer holds (a token whose activations stand out from
        // the batch): one vector at a time - 64 * V elements always fit - with a flush in between, so
        // the row keeps its extents and is not left to the slow dense readers.
        static_assert(64 * V <= WBUF, "one vector of candidates must fit the buffer");
        const uint32_t exA = iA - cA, exB = iB - cB;
        const uint32_t tq[PASS_NV] = {t0, t1, t2, t3};
        const uint32_t exq[PASS_NV] = {exA & 0xFFFFu, exA >> 16, exB & 0xFFFFu, exB >> 16};
#pragma unroll
        for (int q = 0; q < PASS_NV; ++q) {
          if (tq[q] == 0) continue;
          if (n_buf + tq[q] > (uint32_t)WBUF) flush();
          uint32_t mm = (m >> (q * V)) & FM, slot = n_buf + exq[q];
          while (mm) {
            const int bit = __ffs(mm) - 1;
            mm &= mm - 1u;
            wbuf[slot++].x = (uint32_t)(q * 64 * V + lane * V + bit);
          }
          finish(tq[q]);
        }
      }
    }
    flush();
    if (lane == 0) row_first[r] = dense ? ROW_DENSE : first;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < NBINS; i += blockDim.x) {
    uint32_t c = lh[i];
    if (c) atomicAdd(&hist[(int64_t)p * NBINS + i], c);
  }
}

// One block per problem: consume the histogram of the current level.
template <typename T>
__global__ __launch_bounds__(SCAN_THREADS) void k_select_scan(SelState *st, uint32_t *hist, uint32_t *pool_count, int phase, int level) {
  constexpr int KB = Elem<T>::KEYBITS;
  __shared__ uint32_t lh[NBINS];
  const int p = blockIdx.x, tid = threadIdx.x;
  SelState s = st[p];
  // phase 0: first look at level 0; phase 1: level 0 again after a retry pass; phase 2: levels >= 1
  if (phase == 0 && !(s.status == ST_RUN && s.level == 0)) return;
  if (phase == 1 && s.status != ST_RETRY) return;
  if (phase == 2 && !(s.status == ST_RUN && (int)s.level == level)) return;
  uint32_t *h = hist + (int64_t)p * NBINS;
  for (int i = tid; i < NBINS; i += SCAN_THREADS) { lh[i] = h[i]; h[i] = 0; }
  __syncthreads();
  int bin; unsigned long long above, total;
  bool found = block_find_from_top(lh, NBINS, s.k_rem, bin, above, total);
  if (tid != 0) return;
  if (s.overflow) found = false;   // the collecting encoder dropped candidates: start over from the matrix
  if (!found) {
    // fewer candidates than K: the sampled cut was too high -> run the pass again from the bottom
    s.status = ST_RETRY; s.cut_key = min_key_of<T>(); s.level = 0; s.path = PATH_ROWS; s.overflow = 0;
    pool_count[p] = 0;  // the retry pass refills the pool from scratch
    st[p] = s;
    return;
  }
  s.k_rem -= above;
  if (s.level == 0) {
    if (KB == 16) {
      if ((uint32_t)bin < FINE16) { s.thr_key = s.cut_key + bin; s.tie_budget = s.k_rem; s.status = ST_DONE; }
      else {
        uint32_t c = (uint32_t)bin - FINE16;
        s.bbase = c << 10; s.flo = s.bbase > FINE16 ? s.bbase : FINE16; s.fhi = s.bbase + 1023u;
        s.shift = 0; s.level = 1; s.status = ST_RUN;
      }
    } else {
      s.bbase = (uint32_t)bin << 21; s.flo = s.bbase; s.fhi = s.bbase + ((1u << 21) - 1u);
      s.shift = 10; s.level = 1; s.status = ST_RUN;
    }
  } else {
    if (s.shift == 0) { s.thr_key = s.cut_key + s.bbase + bin; s.tie_budget = s.k_rem; s.status = ST_DONE; }
    else {
      s.bbase = s.bbase + ((uint32_t)bin << s.shift); s.flo = s.bbase; s.fhi = s.bbase + ((1u << s.shift) - 1u);
      s.shift = 0; s.level = s.level + 1;
    }
  }
  st[p] = s;
}

// Visit the candidates of one row (its chain of pool extents, or the dense row when the
// row got no pool space) with one wavefront.  `f(active, col, raw, key)` is called once per
// wave step with one element per lane (active=false for idle lanes), in ascending column
// order across steps and lanes.
template <typename T, bool GLOBAL, typename Fn>
__device__ __forceinline__ void visit_candidates(
    const T *pre, int64_t Tn, int64_t F, int64_t lstride, int l, int64_t t,
    typename RankOf<T, GLOBAL>::type rk, uint32_t cut_key, const uint32_t *row_first,
    const uint2 *mypool, Fn f) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int lane = lane_id();
  const int64_t r = (int64_t)l * Tn + t;
  uint32_t off = row_first[r];
  if (off != ROW_DENSE) {
    // Up to four steps of 64 entries are fetched together and their keys computed before the first
    // callback, and the header of the next extent is requested before this extent's entries are used: a
    // row with thousands of candidates (a token with outlying activations under a batch-wide cut) is
    // walked by one wavefront, so every serial round trip here is multiplied by its extent count.
    constexpr int NS = 4;
    uint2 hdr = make_uint2(ROW_NONE, 0u);
    if (off != ROW_NONE) hdr = mypool[off];
    while (off != ROW_NONE) {
      const uint2 *sg = mypool + off + 1u;
      const uint32_t cnt = hdr.y, next = hdr.x;
      if (next != ROW_NONE) hdr = mypool[next];
      for (uint32_t i0 = 0; i0 < cnt; i0 += 64 * NS) {
        bool act[NS]; uint2 e[NS]; uint32_t key[NS];
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          const uint32_t i = i0 + u * 64 + lane;
          act[u] = i < cnt;
          e[u] = act[u] ? sg[i] : make_uint2(0, 0);
        }
#pragma unroll
        for (int u = 0; u < NS; ++u) {
          key[u] = 0;
          if (act[u]) key[u] = rank_key_of<T>(rk(Elem<T>::to_f32(Elem<T>::from_raw(e[u].y)), (int64_t)e[u].x));
        }
#pragma unroll
        for (int u = 0; u < NS; ++u)
          if (i0 + u * 64 < cnt) f(act[u], e[u].x, e[u].y, key[u]);
      }
      off = next;
    }
  } else {
    // The dense row, 64 consecutive columns per load.  The values of the next block of NQ loads are
    // requested before the current block is ranked, and all keys of a block are computed (the
    // statistics they need fetched) before its first callback: such a row keeps one wavefront busy for
    // F / 64 steps, and anything serial per step would make it the tail of the whole launch.
    constexpr int NQ = 16;
    const T *row = pre + l * lstride + t * F;
    T v[NQ], vn[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) { const int64_t col = (int64_t)q * 64 + lane; v[q] = col < F ? row[col] : Elem<T>::from_raw(0u); }
    for (int64_t c0 = 0; c0 < F; c0 += 64 * NQ) {
      const int64_t cn = c0 + 64 * NQ;
#pragma unroll
      for (int q = 0; q < NQ; ++q) { const int64_t col = cn + q * 64 + lane; vn[q] = col < F ? row[col] : Elem<T>::from_raw(0u); }
      uint32_t key[NQ];
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int64_t col = c0 + q * 64 + lane;
        key[q] = col < F ? rank_key_of<T>(rk(Elem<T>::to_f32(v[q]), col)) : 0u;
      }
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        const int64_t col = c0 + q * 64 + lane;
        if (c0 + q * 64 >= F) break;
        const bool act = col < F && key[q] >= cut_key;
        f(act, (uint32_t)col, (uint32_t)Elem<T>::raw(v[q]), key[q]);
      }
#pragma unroll
      for (int q = 0; q < NQ; ++q) v[q] = vn[q];
    }
  }
}

// Levels >= 1: histogram of the candidates inside the active key range.
template <typename T, bool GLOBAL>
__global__ __launch_bounds__(256) void k_select_level(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, const SelState *st, uint32_t *hist, const uint32_t *row_first,
    const uint2 *pool, unsigned long long pool_cap, int level) {
  __shared__ uint32_t lh[NBINS];
  const int l = blockIdx.y, p = GLOBAL ? 0 : l;
  const SelState s = st[p];
  if (!(s.status == ST_RUN && (int)s.level == level) || s.path != PATH_ROWS) return;
  for (int i = threadIdx.x; i < NBINS; i += blockDim.x) lh[i] = 0;
  __syncthreads();
  const int wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    visit_candidates<T, GLOBAL>(pre, Tn, F, lstride, l, t, rk, s.cut_key, row_first, pool + (unsigned long long)p * pool_cap,
      [&](bool act, uint32_t, uint32_t, uint32_t key) {
        if (act) {
          uint32_t diff = key - s.cut_key;
          if (diff >= s.flo && diff <= s.fhi) atomicAdd(&lh[(diff - s.bbase) >> s.shift], 1u);
        }
      });
  }
  __syncthreads();
  for (int i = threadIdx.x; i < NBINS; i += blockDim.x) {
    uint32_t c = lh[i];
    if (c) atomicAdd(&hist[(int64_t)p * NBINS + i], c);
  }
}

// Per row: how many candidates beat the threshold key and how many equal it.
template <typename T, bool GLOBAL>
__global__ __launch_bounds__(256) void k_select_count(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, const SelState *st, const uint32_t *row_first, const uint2 *pool,
    unsigned long long pool_cap, uint32_t *row_gt, uint32_t *row_eq) {
  const int l = blockIdx.y, p = GLOBAL ? 0 : l;
  const SelState s = st[p];
  if (s.path != PATH_ROWS) return;
  const int wv = threadIdx.x >> 6, nwv = blockDim.x >> 6, lane = lane_id();
  typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    uint32_t ngt = 0, neq = 0;
    visit_candidates<T, GLOBAL>(pre, Tn, F, lstride, l, t, rk, s.cut_key, row_first, pool + (unsigned long long)p * pool_cap,
      [&](bool act, uint32_t, uint32_t, uint32_t key) {
        ngt += (uint32_t)__popcll(ballot64(act && key > s.thr_key));
        neq += (uint32_t)__popcll(ballot64(act && key == s.thr_key));
      });
    if (lane == 0) { row_gt[(int64_t)l * Tn + t] = ngt; row_eq[(int64_t)l * Tn + t] = neq; }
  }
}

__device__ __forceinline__ unsigned long long block_excl_scan_u64(unsigned long long v, unsigned long long &total) {
  __shared__ unsigned long long ws[SCAN_THREADS / CLT_WAVE];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  unsigned long long inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    unsigned long long y = __shfl_up(inc, o);
    if (lane >= o) inc += y;
  }
  __syncthreads();
  if (lane == 63) ws[wv] = inc;
  __syncthreads();
  unsigned long long base = 0, tot = 0;
  for (int i = 0; i < (int)(blockDim.x >> 6); ++i) { unsigned long long w = ws[i]; if (i < wv) base += w; tot += w; }
  total = tot;
  return base + inc - v;
}

// One block per problem: hand the tie budget out in flat-index order; in per-layer mode
// also write this layer's part of row_ptr (every layer keeps exactly K rows' worth).  A thread takes
// SCAN_ITEMS consecutive rows per sweep, so a sweep's round trip to memory and its two block-wide
// scans are paid once per SCAN_THREADS * SCAN_ITEMS rows.
constexpr int SCAN_ITEMS = 4;
template <bool GLOBAL>
__global__ __launch_bounds__(SCAN_THREADS) void k_select_allot(
    const SelState *st, int64_t Tn, int64_t L, const uint32_t *row_gt, const uint32_t *row_eq,
    uint32_t *allot, uint32_t *keep, int32_t *row_ptr, unsigned long long K) {
  const int p = blockIdx.x, tid = threadIdx.x;
  const unsigned long long budget = st[p].tie_budget;
  const int64_t nrows = GLOBAL ? Tn * L : Tn;
  unsigned long long eq_run = 0, keep_run = 0;
  for (int64_t i0 = 0; i0 < nrows; i0 += (int64_t)SCAN_THREADS * SCAN_ITEMS) {
    int64_t r[SCAN_ITEMS];
    unsigned long long eq[SCAN_ITEMS], gt[SCAN_ITEMS], kp[SCAN_ITEMS], eq_sum = 0, kp_sum = 0, tot;
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) {
      const int64_t i = i0 + (int64_t)tid * SCAN_ITEMS + j;
      r[j] = i < nrows ? (GLOBAL ? ((i % L) * Tn + i / L) : ((int64_t)p * Tn + i)) : -1;
      eq[j] = r[j] >= 0 ? row_eq[r[j]] : 0;
      gt[j] = r[j] >= 0 ? row_gt[r[j]] : 0;
      eq_sum += eq[j];
    }
    unsigned long long before = eq_run + block_excl_scan_u64(eq_sum, tot);
    eq_run += tot;
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) {
      const unsigned long long a = before >= budget ? 0 : (budget - before < eq[j] ? budget - before : eq[j]);
      before += eq[j];
      kp[j] = gt[j] + a;
      kp_sum += kp[j];
      if (r[j] >= 0) { allot[r[j]] = (uint32_t)a; keep[r[j]] = (uint32_t)kp[j]; }
    }
    if (!GLOBAL) {
      unsigned long long kt;
      unsigned long long kbefore = keep_run + block_excl_scan_u64(kp_sum, kt);
      keep_run += kt;
#pragma unroll
      for (int j = 0; j < SCAN_ITEMS; ++j) {
        if (r[j] >= 0) row_ptr[r[j]] = (int32_t)((unsigned long long)p * K + kbefore);
        kbefore += kp[j];
      }
    }
  }
  if (!GLOBAL && tid == 0 && p == (int)gridDim.x - 1) row_ptr[(int64_t)gridDim.x * Tn] = (int32_t)((unsigned long long)gridDim.x * K);
}

// Single block: row_ptr = exclusive scan of keep[] in storage order (row = layer*T + token), one
// coalesced sweep of SCAN_THREADS * SCAN_ITEMS rows at a time with a running carry.
// A total beyond what an int32 row pointer can hold is written as -2 (the prefixes before it are then
// meaningless); `skip` (may be NULL) gates the whole launch on a device flag.
__global__ __launch_bounds__(SCAN_THREADS) void k_rowptr_scan(const uint32_t *keep, int64_t R, int32_t *row_ptr,
                                                              const int32_t *skip = nullptr) {
  if (skip && *skip != 0) return;
  const int tid = threadIdx.x;
  unsigned long long carry = 0;
  for (int64_t i0 = 0; i0 < R; i0 += (int64_t)SCAN_THREADS * SCAN_ITEMS) {
    const int64_t i = i0 + (int64_t)tid * SCAN_ITEMS;
    unsigned long long v[SCAN_ITEMS], sum = 0, tot;
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) { v[j] = i + j < R ? keep[i + j] : 0; sum += v[j]; }
    unsigned long long before = carry + block_excl_scan_u64(sum, tot);
#pragma unroll
    for (int j = 0; j < SCAN_ITEMS; ++j) {
      if (i + j < R) row_ptr[i + j] = (int32_t)before;
      before += v[j];
    }
    carry += tot;
  }
  if (tid == 0) row_ptr[R] = carry > 0x7FFFFFFFull ? -2 : (int32_t)carry;
}

// Ordered write of the survivors of each row.
template <typename T, bool GLOBAL>
__global__ __launch_bounds__(256) void k_select_emit(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, const SelState *st, const uint32_t *row_first, const uint2 *pool,
    unsigned long long pool_cap, const uint32_t *allot, const int32_t *row_ptr, int32_t *col_out, T *val_out) {
  const int l = blockIdx.y, p = GLOBAL ? 0 : l;
  const SelState s = st[p];
  if (s.path != PATH_ROWS) return;
  const int wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    const int64_t r = (int64_t)l * Tn + t;
    const int64_t base = row_ptr[r];
    const uint32_t my_allot = allot[r];
    uint32_t kept = 0, ties = 0;
    visit_candidates<T, GLOBAL>(pre, Tn, F, lstride, l, t, rk, s.cut_key, row_first, pool + (unsigned long long)p * pool_cap,
      [&](bool act, uint32_t col, uint32_t raw, uint32_t key) {
        bool eq = act && key == s.thr_key;
        uint64_t beq = ballot64(eq);
        bool keepit = act && (key > s.thr_key || (eq && ties + mbcnt64(beq) < my_allot));
        uint64_t bk = ballot64(keepit);
        if (keepit) {
          int64_t pos = base + kept + mbcnt64(bk);
          col_out[pos] = (int32_t)col;
          val_out[pos] = Elem<T>::from_raw(raw);
        }
        kept += (uint32_t)__popcll(bk);
        ties += (uint32_t)__popcll(beq);
      });
  }
}

// ---- candidates collected by the encoder epilogue (PATH_TILES) -------------------------
// Ranking keys of a sample taken BEFORE the pre-activations exist.  Per layer SAMPLE_WAVES wavefronts
// each compute a 32 x 32 block of pre-activations with the matrix core, for 32 hashed tokens and 32
// hashed features of their own (so a layer's sample covers 2048 tokens and 2048 features): a lane reads
// 16 bytes of "its" x row and W row per step straight from global memory - the K order inside a step is
// the same permutation for both operands, which a dot product does not mind - fp32 accumulation, bias,
// one rounding to the model dtype.  The sample only has to give a cut of the right size; the selection
// stays exact whatever the cut is.
typedef __attribute__((ext_vector_type(8))) __bf16 smp_bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 smp_f16x8_t;
typedef __attribute__((ext_vector_type(16))) float smp_f32x16_t;
template <typename T>
__global__ __launch_bounds__(256) void k_sample_mfma(
    const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ b, int64_t Tn, int64_t d, int64_t F,
    int64_t xs, int64_t wstr, int64_t bs, uint32_t *sample) {
  constexpr int KB = Elem<T>::KEYBITS;
  constexpr int V = 16 / (int)sizeof(T);   // elements of one 16-byte piece
  const int l = blockIdx.y, lane = lane_id();
  const int g = (int)blockIdx.x * (int)(blockDim.x >> 6) + (int)(threadIdx.x >> 6);   // block of the sample
  const int l31 = lane & 31, lh = lane >> 5;
  const uint64_t salt = (uint64_t)l * 7919u + (uint64_t)g * 104729u;
  const int64_t tok = (int64_t)hash_index(salt * 64u + (uint64_t)l31, (uint64_t)Tn);
  const int64_t f = (int64_t)hash_index(salt * 64u + 32u + (uint64_t)l31, (uint64_t)F);
  const T *xr = x + (int64_t)l * xs + tok * d + lh * V;
  const T *wr = w + (int64_t)l * wstr + f * d + lh * V;
  smp_f32x16_t acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  const int64_t nstep = d / (2 * V);       // the collecting encoder needs d to be a multiple of 2 V
#pragma unroll 4
  for (int64_t st = 0; st < nstep; ++st) {
    const uint4 a = *reinterpret_cast<const uint4 *>(wr + st * 2 * V);
    const uint4 q = *reinterpret_cast<const uint4 *>(xr + st * 2 * V);
    if constexpr (IsHalf<T>::value) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(smp_f16x8_t, a), __builtin_bit_cast(smp_f16x8_t, q), acc, 0, 0, 0);
    } else if constexpr (sizeof(T) == 2) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(smp_bf16x8_t, a), __builtin_bit_cast(smp_bf16x8_t, q), acc, 0, 0, 0);
    } else {
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(q.x), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(q.y), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(q.z), acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(q.w), acc, 0, 0, 0);
    }
  }
  // accumulator rg*4+q of a lane: feature row rg*8 + lh*4 + q of the block, token column l31
  const float bown = b ? Elem<T>::to_f32(b[(int64_t)l * bs + f]) : 0.0f;   // bias of feature row l31
  uint32_t *out = sample + (int64_t)l * SAMPLE_PRE_N + (int64_t)g * 1024;
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int m = rg * 8 + lh * 4 + q;
      const float bv = __shfl(bown, m);
      out[m * 32 + l31] = rank_key_of<T>(Elem<T>::round(acc[rg * 4 + q] + bv));
    }
}

// Histogram of the collected candidates of every layer that is at `level`: one wavefront per
// tile extent.
template <typename T>
__global__ __launch_bounds__(256) void k_pool_hist(const SelState *st, const uint2 *tile_meta, int ntile,
                                                   const uint2 *pool, unsigned long long pool_cap, uint32_t *hist,
                                                   int level) {
  constexpr int KB = Elem<T>::KEYBITS;
  __shared__ uint32_t lh[NBINS];
  const int p = blockIdx.y;
  const SelState s = st[p];
  if (s.path != PATH_TILES || s.status != ST_RUN || (int)s.level != level) return;
  for (int i = threadIdx.x; i < NBINS; i += blockDim.x) lh[i] = 0;
  __syncthreads();
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const uint2 *mypool = pool + (unsigned long long)p * pool_cap;
  for (int i = blockIdx.x * nwv + wv; i < ntile; i += gridDim.x * nwv) {
    const uint2 tm = tile_meta[(int64_t)p * ntile + i];
    for (uint32_t e0 = 0; e0 < tm.y; e0 += 256) {
      uint32_t raw[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) { const uint32_t e = e0 + q * 64 + lane; raw[q] = e < tm.y ? mypool[tm.x + e].y : 0u; }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (e0 + q * 64 + lane >= tm.y) continue;
        const uint32_t diff = rank_key_of<T>(Elem<T>::to_f32(Elem<T>::from_raw(raw[q]))) - s.cut_key;
        if (level == 0) atomicAdd(&lh[bin_level0<KB>(diff)], 1u);
        else if (diff >= s.flo && diff <= s.fhi) atomicAdd(&lh[(diff - s.bbase) >> s.shift], 1u);
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < NBINS; i += blockDim.x) {
    uint32_t c = lh[i];
    if (c) atomicAdd(&hist[(int64_t)p * NBINS + i], c);
  }
}

// The three kernels below finish the selection on the encoder-collected candidates.  They all
// map a wavefront to 64 consecutive token rows of one feature segment (lane = row): the rows'
// bookkeeping entries are adjacent in seg_meta and their runs are adjacent in the tile extent,
// so every access of a wavefront is (nearly) contiguous.
//
// k_tile_count: per (row, segment), how many entries beat the threshold key / equal it.
// Grid: x = blocks of 256 rows, y = segment, z = layer.
constexpr int TILE_NE = 4;   // entries of a run fetched in one batch
template <typename T>
__global__ __launch_bounds__(256) void k_tile_count(
    int Tn, int Tp, const SelState *st, const uint2 *seg_meta, int nseg, const uint2 *pool, unsigned long long pool_cap,
    uint8_t *cgt, uint8_t *ceq) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int l = blockIdx.z, seg = blockIdx.y;
  const SelState s = st[l];
  if (s.path != PATH_TILES || s.status != ST_DONE) return;
  const uint2 *mypool = pool + (unsigned long long)l * pool_cap;
  const int row = blockIdx.x * 256 + threadIdx.x;
  if (row >= Tn) return;
  const int64_t at = ((int64_t)l * nseg + seg) * Tp + collect_grid_row(row, Tn, Tp);
  const uint2 m = seg_meta[at];
  uint32_t raw[TILE_NE];
#pragma unroll
  for (int e = 0; e < TILE_NE; ++e) raw[e] = (uint32_t)e < m.y ? mypool[m.x + e].y : 0u;
  uint32_t ngt = 0, neq = 0;
#pragma unroll
  for (int e = 0; e < TILE_NE; ++e)
    if ((uint32_t)e < m.y) {
      const uint32_t key = rank_key_of<T>(Elem<T>::to_f32(Elem<T>::from_raw(raw[e])));
      ngt += key > s.thr_key ? 1u : 0u;
      neq += key == s.thr_key ? 1u : 0u;
    }
  for (uint32_t e = TILE_NE; e < m.y; ++e) {
    const uint32_t key = rank_key_of<T>(Elem<T>::to_f32(Elem<T>::from_raw(mypool[m.x + e].y)));
    ngt += key > s.thr_key ? 1u : 0u;
    neq += key == s.thr_key ? 1u : 0u;
  }
  cgt[at] = (uint8_t)ngt; ceq[at] = (uint8_t)neq;   // a run has at most 128 entries
}

// k_row_prefix: per row, exclusive prefix of those counts over the segments, and the row totals.
__global__ __launch_bounds__(256) void k_row_prefix(
    int64_t Tn, int64_t Tp, const SelState *st, int nseg, const uint8_t *cgt, const uint8_t *ceq, uint32_t *pgt,
    uint32_t *peq, uint32_t *row_gt, uint32_t *row_eq) {
  const int l = blockIdx.y;
  const SelState s = st[l];
  if (s.path != PATH_TILES || s.status != ST_DONE) return;
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= Tn) return;
  uint32_t g = 0, q = 0;
  const int64_t base = (int64_t)l * nseg * Tp + collect_grid_row(row, Tn, Tp);
  int seg = 0;
  for (; seg + 8 <= nseg; seg += 8) {
    uint32_t a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = cgt[base + (int64_t)(seg + i) * Tp]; b[i] = ceq[base + (int64_t)(seg + i) * Tp]; }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pgt[base + (int64_t)(seg + i) * Tp] = g; peq[base + (int64_t)(seg + i) * Tp] = q;
      g += a[i]; q += b[i];
    }
  }
  for (; seg < nseg; ++seg) {
    const uint32_t a = cgt[base + (int64_t)seg * Tp], b = ceq[base + (int64_t)seg * Tp];
    pgt[base + (int64_t)seg * Tp] = g; peq[base + (int64_t)seg * Tp] = q;
    g += a; q += b;
  }
  row_gt[(int64_t)l * Tn + row] = g; row_eq[(int64_t)l * Tn + row] = q;
}

// k_tile_emit: the ordered write.  An entry's place in its row = the row's start + the entries
// kept in earlier segments (all that beat the key, and ties while the row's allotment lasts) +
// the entries kept before it in its own run.
template <typename T>
__global__ __launch_bounds__(256) void k_tile_emit(
    int Tn, int Tp, const SelState *st, const uint2 *seg_meta, int nseg, const uint2 *pool, unsigned long long pool_cap,
    const uint32_t *pgt, const uint32_t *peq, const uint32_t *allot, const int32_t *row_ptr, int32_t *col_out,
    T *val_out) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int l = blockIdx.z, seg = blockIdx.y;
  const SelState s = st[l];
  if (s.path != PATH_TILES || s.status != ST_DONE) return;
  const uint2 *mypool = pool + (unsigned long long)l * pool_cap;
  const int row = blockIdx.x * 256 + threadIdx.x;
  if (row >= Tn) return;
  const int64_t at = ((int64_t)l * nseg + seg) * Tp + collect_grid_row(row, Tn, Tp);
  const uint2 m = seg_meta[at];
  if (m.y == 0) return;
  const int64_t r = (int64_t)l * Tn + row;
  uint2 en[TILE_NE];
#pragma unroll
  for (int e = 0; e < TILE_NE; ++e) en[e] = (uint32_t)e < m.y ? mypool[m.x + e] : make_uint2(0u, 0u);
  const uint32_t al = allot[r];
  uint32_t tie = peq[at];
  int64_t pos = (int64_t)row_ptr[r] + pgt[at] + (tie < al ? tie : al);
  auto put = [&](const uint2 &e2) {
    const uint32_t key = rank_key_of<T>(Elem<T>::to_f32(Elem<T>::from_raw(e2.y)));
    bool keepit = key > s.thr_key;
    if (key == s.thr_key) { keepit = tie < al; ++tie; }
    if (keepit) { col_out[pos] = (int32_t)e2.x; val_out[pos] = Elem<T>::from_raw(e2.y); ++pos; }
  };
#pragma unroll
  for (int e = 0; e < TILE_NE; ++e)
    if ((uint32_t)e < m.y) put(en[e]);
  for (uint32_t e = TILE_NE; e < m.y; ++e) put(mypool[m.x + e]);
}

// ---- post-hoc threshold estimation: per-feature minimum of the selected z-scores ---------------
// keys[l][f] = min over the survivors (l, token, f, v) with v > 0 of key32(z(v)), z evaluated in
// the model dtype like the ranking value (reference clt/models/theta.py:127-139, which takes the
// minimum of the NORMALISED pre-activations where the gated activation is positive).
template <typename T>
__global__ __launch_bounds__(256) void k_selected_min(const int32_t *row_ptr, const int32_t *col, const T *val,
                                                      const float *mean, const float *denom, int64_t Tn, int64_t F,
                                                      int64_t L, uint32_t *keys) {
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const int64_t R = L * Tn;
  for (int64_t r = (int64_t)blockIdx.x * nwv + wv; r < R; r += (int64_t)gridDim.x * nwv) {
    const int64_t l = r / Tn;
    RankZ<T> rk; rk.mean = mean + l * F; rk.denom = denom + l * F;
    for (int32_t j = row_ptr[r] + lane; j < row_ptr[r + 1]; j += 64) {
      const float v = Elem<T>::to_f32(val[j]);
      if (v > 0.0f) atomicMin(&keys[l * F + col[j]], rank_key32(rk(v, col[j])));
    }
  }
}

// sum[l][f] += min, count[l][f] += 1 where a finite minimum was seen (both buffers in the model
// dtype, every addition rounded to it: theta.py:163-167).
template <typename T>
__global__ void k_selected_min_accumulate(const uint32_t *keys, int64_t n, T *sum, T *count) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const uint32_t k = keys[i];
    const float z = __uint_as_float(key_to_f32_bits<32>(k));
    if (k != 0xFFFFFFFFu && z == z && fabsf(z) != __uint_as_float(0x7F800000u)) {
      sum[i] = Elem<T>::from_f32(Elem<T>::to_f32(sum[i]) + z);
      count[i] = Elem<T>::from_f32(Elem<T>::to_f32(count[i]) + 1.0f);
    }
  }
}

// ---- threshold activation on encoder-collected entries (every entry is a survivor) ----------
// Per row: exclusive prefix of the run lengths over the segments, and the row total.
__global__ __launch_bounds__(256) void k_row_prefix_meta(int64_t Tn, int64_t Tp, int nseg, const uint2 *seg_meta,
                                                         uint32_t *pfx, uint32_t *row_cnt) {
  const int l = blockIdx.y;
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= Tn) return;
  uint32_t g = 0;
  const int64_t base = (int64_t)l * nseg * Tp + collect_grid_row(row, Tn, Tp);
  int seg = 0;
  for (; seg + 8 <= nseg; seg += 8) {
    uint32_t a[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) a[i] = seg_meta[base + (int64_t)(seg + i) * Tp].y;
#pragma unroll
    for (int i = 0; i < 8; ++i) { pfx[base + (int64_t)(seg + i) * Tp] = g; g += a[i]; }
  }
  for (; seg < nseg; ++seg) {
    const uint32_t a = seg_meta[base + (int64_t)seg * Tp].y;
    pfx[base + (int64_t)seg * Tp] = g; g += a;
  }
  row_cnt[(int64_t)l * Tn + row] = g;
}

// row_ptr[R] = -1 when some layer ran out of pool space (the caller then takes the separate route)
__global__ void k_thresh_finish(const SelState *st, int L, int32_t *row_ptr, int64_t R) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  bool over = false;
  for (int l = 0; l < L; ++l) over = over || st[l].overflow != 0;
  if (over) row_ptr[R] = -1;
}

// Grid: x = blocks of 256 rows, y = segment, z = layer.
template <typename T>
__global__ __launch_bounds__(256) void k_tile_emit_all(
    int Tn, int Tp, const uint2 *seg_meta, int nseg, const uint2 *pool, unsigned long long pool_cap, const uint32_t *pfx,
    const int32_t *row_ptr, int32_t *col_out, T *val_out, const int32_t *skip) {
  if (skip && *skip != 0) return;             // the list did not fit the caller's arrays: it was emptied
  const int l = blockIdx.z, seg = blockIdx.y;
  const uint2 *mypool = pool + (unsigned long long)l * pool_cap;
  const int row = blockIdx.x * 256 + threadIdx.x;
  if (row >= Tn) return;
  const int64_t at = ((int64_t)l * nseg + seg) * Tp + collect_grid_row(row, Tn, Tp);
  const uint2 m = seg_meta[at];
  if (m.y == 0) return;
  uint2 en[TILE_NE];
#pragma unroll
  for (int e = 0; e < TILE_NE; ++e) en[e] = (uint32_t)e < m.y ? mypool[m.x + e] : make_uint2(0u, 0u);
  int64_t pos = (int64_t)row_ptr[(int64_t)l * Tn + row] + pfx[at];
#pragma unroll
  for (int e = 0; e < TILE_NE; ++e)
    if ((uint32_t)e < m.y) { col_out[pos] = (int32_t)en[e].x; val_out[pos] = Elem<T>::from_raw(en[e].y); ++pos; }
  for (uint32_t e = TILE_NE; e < m.y; ++e) {
    const uint2 e2 = mypool[m.x + e];
    col_out[pos] = (int32_t)e2.x; val_out[pos] = Elem<T>::from_raw(e2.y); ++pos;
  }
}

// ---- threshold activations ----------------------------------------------------------
template <typename T, int PRED> __device__ __forceinline__ bool pred_keep(float x, float th) {
  if (PRED == CLT_PRED_GE_THETA) return x >= th;
  if (PRED == CLT_PRED_GT_ZERO) return x > 0.0f;
  return x != 0.0f;
}

template <typename T, int V, int PRED, bool EMIT>
__global__ __launch_bounds__(256) void k_threshold(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const T *theta,
    uint32_t *row_cnt, const int32_t *row_ptr, int32_t *col_out, T *val_out, const int32_t *skip) {
  if (skip && *skip != 0) return;             // gated off by a device flag (another route holds the list, or it was emptied)
  const int l = blockIdx.y;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  const T *th_row = PRED == CLT_PRED_GE_THETA ? theta + (int64_t)l * F : nullptr;
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    const int64_t r = (int64_t)l * Tn + t;
    const T *row = pre + l * lstride + t * F;
    const int64_t base = EMIT ? (int64_t)row_ptr[r] : 0;
    uint32_t n = 0;
    for (int64_t c0 = 0; c0 < F; c0 += 64 * V) {
      const int64_t col = c0 + (int64_t)lane * V;
      float x[V]; uint32_t raw[V];
      uint32_t m = 0;
      if (col < F) {
        VecLoad<T, V>::load(row + col, x, raw);
        float th[V];
        if (PRED == CLT_PRED_GE_THETA) { uint32_t traw[V]; VecLoad<T, V>::load(th_row + col, th, traw); }
#pragma unroll
        for (int j = 0; j < V; ++j) if (pred_keep<T, PRED>(x[j], PRED == CLT_PRED_GE_THETA ? th[j] : 0.0f)) m |= 1u << j;
      }
      if (EMIT) {
        if (ballot64(m != 0) == 0) continue;
        uint32_t total, pre_cnt = wave_mask_prefix<V>(m, total);
#pragma unroll
        for (int j = 0; j < V; ++j)
          if ((m >> j) & 1u) {
            int64_t pos = base + n + pre_cnt + __popc(m & ((1u << j) - 1u));
            col_out[pos] = (int32_t)(col + j);
            val_out[pos] = Elem<T>::from_raw(raw[j]);
          }
        n += total;
      } else {
        n += __popc(m);
      }
    }
    if (!EMIT) {
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) n += __shfl_xor(n, o);
      if (lane == 0) row_cnt[r] = n;
    }
  }
}

// ---- TokenTopK ------------------------------------------------------------------------
// Row-wise top-k (reference clt/models/activations.py:99-128, 391-491).  A "problem" is one
// token row: F entries of one layer (per-layer mode) or the L*F entries of all layers ranked
// on the z-score (global mode).  One block per problem finds the kk-th largest key by MSD
// radix select over the row (11-bit digits, LDS histogram), then counts per (layer, token)
// row how many entries beat the threshold and hands the tie budget out in column order
// (layers in ascending order in global mode).  A second kernel writes the survivors in order.
template <typename T, bool GLOBAL>
__global__ __launch_bounds__(SCAN_THREADS) void k_token_threshold(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, unsigned long long kk, uint32_t *thr_key, uint32_t *allot, uint32_t *keep) {
  constexpr int KB = Elem<T>::KEYBITS;
  constexpr int NLEV = KB == 32 ? 3 : 2;
  __shared__ uint32_t lh[NBINS];
  __shared__ uint32_t cnt_gt[TOK_MAX_LAYERS], cnt_eq[TOK_MAX_LAYERS];   // per layer of a token's global problem
  const int tid = threadIdx.x;
  // per-layer: problem = (layer, token); global: problem = token
  const int64_t prob = blockIdx.x;
  const int64_t l0 = GLOBAL ? 0 : prob / Tn, t = GLOBAL ? prob : prob - l0 * Tn;
  const int nl = GLOBAL ? (int)L : 1;
  const int shifts[3] = {KB == 32 ? 21 : 5, KB == 32 ? 10 : 0, 0};
  const int widths[3] = {11, KB == 32 ? 11 : 5, 10};
  uint32_t prefix = 0, prefix_mask = 0;
  unsigned long long k_rem = kk;
  for (int lev = 0; lev < NLEV; ++lev) {
    for (int i = tid; i < NBINS; i += SCAN_THREADS) lh[i] = 0;
    __syncthreads();
    const int sh = shifts[lev];
    const uint32_t dm = (1u << widths[lev]) - 1u;
    for (int li = 0; li < nl; ++li) {
      const int64_t l = l0 + li;
      const T *row = pre + l * lstride + t * F;
      typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
      for (int64_t f = tid; f < F; f += SCAN_THREADS) {
        const uint32_t key = rank_key_of<T>(rk(Elem<T>::to_f32(row[f]), f));
        if ((key & prefix_mask) == prefix) atomicAdd(&lh[(key >> sh) & dm], 1u);
      }
    }
    __syncthreads();
    int bin; unsigned long long above, total;
    block_find_from_top(lh, (int)dm + 1, k_rem, bin, above, total);
    if (bin < 0) bin = 0;   // kk <= row length, so the bin exists
    k_rem -= above;
    prefix |= (uint32_t)bin << sh;
    prefix_mask |= dm << sh;
  }
  const uint32_t thr = prefix;          // key of the kk-th largest entry; k_rem ties survive
  for (int i = tid; i < TOK_MAX_LAYERS; i += SCAN_THREADS) { cnt_gt[i] = 0; cnt_eq[i] = 0; }
  __syncthreads();
  for (int li = 0; li < nl; ++li) {
    const int64_t l = l0 + li;
    const T *row = pre + l * lstride + t * F;
    typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
    uint32_t g = 0, e = 0;
    for (int64_t f = tid; f < F; f += SCAN_THREADS) {
      const uint32_t key = rank_key_of<T>(rk(Elem<T>::to_f32(row[f]), f));
      g += key > thr; e += key == thr;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { g += __shfl_xor(g, o); e += __shfl_xor(e, o); }
    if ((tid & 63) == 0) { atomicAdd(&cnt_gt[li], g); atomicAdd(&cnt_eq[li], e); }
  }
  __syncthreads();
  if (tid == 0) {
    thr_key[prob] = thr;
    unsigned long long budget = k_rem;
    for (int li = 0; li < nl; ++li) {
      const int64_t r = (l0 + li) * Tn + t;
      const unsigned long long a = budget < cnt_eq[li] ? budget : cnt_eq[li];
      budget -= a;
      allot[r] = (uint32_t)a;
      keep[r] = cnt_gt[li] + (uint32_t)a;
    }
  }
}

// One wavefront per (layer, token) row: survivors in ascending column order.
template <typename T, int V, bool GLOBAL>
__global__ __launch_bounds__(256) void k_token_emit(
    const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, const float *mean,
    const float *denom, const uint32_t *thr_key, const uint32_t *allot, const int32_t *row_ptr,
    int32_t *col_out, T *val_out) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int l = blockIdx.y;
  const int lane = lane_id(), wv = threadIdx.x >> 6, nwv = blockDim.x >> 6;
  typename RankOf<T, GLOBAL>::type rk = RankOf<T, GLOBAL>::make(mean, denom, l, F);
  for (int64_t t = (int64_t)blockIdx.x * nwv + wv; t < Tn; t += (int64_t)gridDim.x * nwv) {
    const int64_t r = (int64_t)l * Tn + t;
    const uint32_t thr = thr_key[GLOBAL ? t : r];
    const uint32_t my_allot = allot[r];
    const int64_t base = row_ptr[r];
    const T *row = pre + l * lstride + t * F;
    uint32_t kept = 0, ties = 0;
    for (int64_t c0 = 0; c0 < F; c0 += 64 * V) {
      const int64_t col = c0 + (int64_t)lane * V;
      float x[V]; uint32_t raw[V];
      uint32_t mg = 0, me = 0;
      if (col < F) {
        VecLoad<T, V>::load(row + col, x, raw);
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const uint32_t key = rank_key_of<T>(rk(x[j], col + j));
          if (key > thr) mg |= 1u << j;
          if (key == thr) me |= 1u << j;
        }
      }
      if (ballot64((mg | me) != 0) == 0) continue;
      // ties first: their rank in column order decides which of them survive
      uint32_t te, pe = wave_mask_prefix<V>(me, te);
      uint32_t mk = mg;
#pragma unroll
      for (int j = 0; j < V; ++j)
        if ((me >> j) & 1u) {
          const uint32_t rank = ties + pe + __popc(me & ((1u << j) - 1u));
          if (rank < my_allot) mk |= 1u << j;
        }
      ties += te;
      uint32_t tk, pk = wave_mask_prefix<V>(mk, tk);
#pragma unroll
      for (int j = 0; j < V; ++j)
        if ((mk >> j) & 1u) {
          const int64_t pos = base + kept + pk + __popc(mk & ((1u << j) - 1u));
          col_out[pos] = (int32_t)(col + j);
          val_out[pos] = Elem<T>::from_raw(raw[j]);
        }
      kept += tk;
    }
  }
}

struct TokLayout { size_t off_thr, off_allot, off_keep, total; };
static TokLayout tok_layout(int64_t T, int64_t L) {
  TokLayout lo; size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += (bytes + 255) & ~(size_t)255; return at; };
  lo.off_thr = take(4 * (size_t)(L * T));
  lo.off_allot = take(4 * (size_t)(L * T));
  lo.off_keep = take(4 * (size_t)(L * T));
  lo.total = o;
  return lo;
}

template <typename T, bool GLOBAL>
static int run_tokentopk(const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, int64_t kk,
                         const float *mean, const float *denom, int32_t *row_ptr, int32_t *col, T *val,
                         char *ws, hipStream_t stream) {
  constexpr int VV = Elem<T>::VEC;
  const TokLayout lo = tok_layout(Tn, L);
  uint32_t *thr = (uint32_t *)(ws + lo.off_thr), *allot = (uint32_t *)(ws + lo.off_allot);
  uint32_t *keep = (uint32_t *)(ws + lo.off_keep);
  const int64_t nprob = GLOBAL ? Tn : L * Tn;
  if (nprob > 2147483647LL) return CLT_ERR_RANGE;
  k_token_threshold<T, GLOBAL><<<(unsigned)nprob, SCAN_THREADS, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom,
                                                                           (unsigned long long)kk, thr, allot, keep);
  k_rowptr_scan<<<1, SCAN_THREADS, 0, stream>>>(keep, L * Tn, row_ptr);
  int gx = (int)clt_ceil_div(Tn, 4);
  int maxgx = (int)clt_ceil_div(256 * 8, L);
  if (maxgx < 1) maxgx = 1;
  if (gx > maxgx) gx = maxgx;
  dim3 grid(gx, (unsigned)L);
  const bool vec = (F % VV == 0) && clt_aligned16(pre) && ((lstride * (int64_t)sizeof(T)) % 16 == 0);
  if (vec) k_token_emit<T, VV, GLOBAL><<<grid, 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, thr, allot, row_ptr, col, val);
  else k_token_emit<T, 1, GLOBAL><<<grid, 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, thr, allot, row_ptr, col, val);
  return clt_check_launch();
}

// ---- host side ------------------------------------------------------------------------
struct SelLayout {
  size_t off_state, off_hist, off_poolcnt, off_sample, off_first, off_gt, off_eq, off_allot, off_keep, off_xcut, off_pool, total;
  unsigned long long pool_cap;  // entries per problem
  int nprob;
};

static SelLayout sel_layout(int64_t T, int64_t F, int64_t L, int64_t k, int mode) {
  SelLayout lo;
  lo.nprob = mode == CLT_TOPK_GLOBAL ? 1 : (int)L;
  const size_t R = (size_t)(L * T);
  const unsigned long long rows_p = mode == CLT_TOPK_GLOBAL ? (unsigned long long)R : (unsigned long long)T;
  const unsigned long long N = (unsigned long long)T * F * (mode == CLT_TOPK_GLOBAL ? L : 1);
  unsigned long long K = (unsigned long long)k * T;
  if (K > N) K = N;
  // about 2x K candidates are expected; every extent also stores one header entry
  unsigned long long cap = 4ull * K + 2ull * rows_p + 4096ull;
  const unsigned long long hard = N + 2ull * rows_p + 4096ull;
  if (cap > hard) cap = hard;
  if (cap > 0xFFF00000ull) cap = 0xFFF00000ull;
  lo.pool_cap = cap;
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += (bytes + 255) & ~(size_t)255; return at; };
  lo.off_state = take(sizeof(SelState) * (size_t)lo.nprob);
  lo.off_hist = take(sizeof(uint32_t) * NBINS * (size_t)lo.nprob);
  lo.off_poolcnt = take(4 * (size_t)lo.nprob);
  lo.off_sample = take(4 * (size_t)(SAMPLE_PRE_N > SAMPLE_N ? SAMPLE_PRE_N : SAMPLE_N) * (size_t)lo.nprob);
  lo.off_first = take(4 * R);
  lo.off_gt = take(4 * R);
  lo.off_eq = take(4 * R);
  lo.off_allot = take(4 * R);
  lo.off_keep = take(4 * R);
  lo.off_xcut = take(mode == CLT_TOPK_GLOBAL ? 4 * (size_t)F * (size_t)L : 0);   // per-column bounds, element type
  lo.off_pool = take(8 * (size_t)cap * (size_t)lo.nprob);
  lo.total = o;
  return lo;
}

template <typename T, int V, bool GLOBAL>
static int run_batchtopk(const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, int64_t k,
                         const float *mean, const float *denom, int32_t *row_ptr, int32_t *col, T *val,
                         char *ws, hipStream_t stream) {
  constexpr int KB = Elem<T>::KEYBITS;
  const int mode = GLOBAL ? CLT_TOPK_GLOBAL : CLT_TOPK_PER_LAYER;
  const SelLayout lo = sel_layout(Tn, F, L, k, mode);
  SelState *st = (SelState *)(ws + lo.off_state);
  uint32_t *hist = (uint32_t *)(ws + lo.off_hist);
  uint32_t *poolcnt = (uint32_t *)(ws + lo.off_poolcnt);
  uint32_t *sample = (uint32_t *)(ws + lo.off_sample);
  uint32_t *first = (uint32_t *)(ws + lo.off_first);
  uint32_t *rgt = (uint32_t *)(ws + lo.off_gt), *req = (uint32_t *)(ws + lo.off_eq);
  uint32_t *allot = (uint32_t *)(ws + lo.off_allot), *keep = (uint32_t *)(ws + lo.off_keep);
  uint2 *pool = (uint2 *)(ws + lo.off_pool);
  const unsigned long long N = (unsigned long long)Tn * (unsigned long long)F * (GLOBAL ? (unsigned long long)L : 1ull);
  unsigned long long K = (unsigned long long)k * (unsigned long long)Tn;
  if (K > N) K = N;
  const int nprob = lo.nprob;
  k_sample_keys<T, GLOBAL><<<dim3(SAMPLE_BLOCKS, nprob), 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, N, sample);
  k_sample_cut<T, SAMPLE_N><<<nprob, SCAN_THREADS, 0, stream>>>(sample, N, K, st, hist, poolcnt, nullptr, PATH_ROWS);
  // two rows per wavefront: many more blocks than fit at once, so rows of very different
  // candidate counts balance out over the CUs
  int gx = (int)clt_ceil_div(Tn, 8);
  if (gx > 65535 * 8) gx = 65535 * 8;
  dim3 grid(gx, (unsigned)L);
  T *xcut = nullptr;
  if (GLOBAL && V > 1) {
    xcut = (T *)(ws + lo.off_xcut);
    k_col_cut<T><<<(unsigned)clt_ceil_div(L * F, 256), 256, 0, stream>>>(mean, denom, st, F, L, xcut);
  }
  for (int phase = 0; phase < 2; ++phase) {
    k_select_pass<T, V, GLOBAL><<<grid, 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, st, hist, poolcnt, pool, lo.pool_cap, first, phase, xcut);
    k_select_scan<T><<<nprob, SCAN_THREADS, 0, stream>>>(st, hist, poolcnt, phase, 0);
  }
  int gx2 = (int)clt_ceil_div(Tn, 4);
  int maxgx2 = (int)clt_ceil_div(256 * 8, L);
  if (maxgx2 < 1) maxgx2 = 1;
  if (gx2 > maxgx2) gx2 = maxgx2;
  dim3 grid2(gx2, (unsigned)L);
  const int nlev = KB == 32 ? 3 : 2;
  for (int level = 1; level < nlev; ++level) {
    k_select_level<T, GLOBAL><<<grid2, 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, st, hist, first, pool, lo.pool_cap, level);
    k_select_scan<T><<<nprob, SCAN_THREADS, 0, stream>>>(st, hist, poolcnt, 2, level);
  }
  k_select_count<T, GLOBAL><<<grid2, 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, st, first, pool, lo.pool_cap, rgt, req);
  k_select_allot<GLOBAL><<<nprob, SCAN_THREADS, 0, stream>>>(st, Tn, L, rgt, req, allot, keep, row_ptr, K);
  if (GLOBAL) k_rowptr_scan<<<1, SCAN_THREADS, 0, stream>>>(keep, L * Tn, row_ptr);
  k_select_emit<T, GLOBAL><<<grid2, 256, 0, stream>>>(pre, Tn, F, L, lstride, mean, denom, st, first, pool, lo.pool_cap, allot, row_ptr, col, val);
  return clt_check_launch();
}

template <typename T, bool GLOBAL>
static int run_batchtopk_v(const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, int64_t k,
                           const float *mean, const float *denom, int32_t *row_ptr, int32_t *col, T *val,
                           char *ws, hipStream_t stream) {
  constexpr int VV = Elem<T>::VEC;
  bool vec = (F % VV == 0) && clt_aligned16(pre) && ((lstride * (int64_t)sizeof(T)) % 16 == 0);
  if (vec) return run_batchtopk<T, VV, GLOBAL>(pre, Tn, F, L, lstride, k, mean, denom, row_ptr, col, val, ws, stream);
  return run_batchtopk<T, 1, GLOBAL>(pre, Tn, F, L, lstride, k, mean, denom, row_ptr, col, val, ws, stream);
}

template <typename T, int V, int PRED>
static int run_threshold(bool emit, const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride,
                         const T *theta, uint32_t *row_cnt, int32_t *row_ptr, int32_t *col, T *val,
                         const int32_t *skip, hipStream_t stream) {
  int gx = (int)clt_ceil_div(Tn, 4);
  int maxgx = (int)clt_ceil_div(256 * 8, L);
  if (maxgx < 1) maxgx = 1;
  if (gx > maxgx) gx = maxgx;
  dim3 grid(gx, (unsigned)L);
  if (!emit) {
    k_threshold<T, V, PRED, false><<<grid, 256, 0, stream>>>(pre, Tn, F, L, lstride, theta, row_cnt, nullptr, nullptr, nullptr, skip);
    k_rowptr_scan<<<1, SCAN_THREADS, 0, stream>>>(row_cnt, L * Tn, row_ptr, skip);
  } else {
    k_threshold<T, V, PRED, true><<<grid, 256, 0, stream>>>(pre, Tn, F, L, lstride, theta, nullptr, row_ptr, col, val, skip);
  }
  return clt_check_launch();
}

template <typename T>
static int dispatch_threshold(bool emit, const void *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride,
                              const void *theta, int pred, uint32_t *row_cnt, int32_t *row_ptr,
                              int32_t *col, void *val, const int32_t *skip, hipStream_t stream) {
  constexpr int VV = Elem<T>::VEC;
  bool vec = (F % VV == 0) && clt_aligned16(pre) && ((lstride * (int64_t)sizeof(T)) % 16 == 0) &&
             (pred != CLT_PRED_GE_THETA || clt_aligned16(theta));
  const T *p = (const T *)pre; const T *th = (const T *)theta; T *v = (T *)val;
#define CLT_TH(PR)                                                                                       \
  return vec ? run_threshold<T, VV, PR>(emit, p, Tn, F, L, lstride, th, row_cnt, row_ptr, col, v, skip, stream) \
             : run_threshold<T, 1, PR>(emit, p, Tn, F, L, lstride, th, row_cnt, row_ptr, col, v, skip, stream)
  if (pred == CLT_PRED_GE_THETA) { CLT_TH(CLT_PRED_GE_THETA); }
  if (pred == CLT_PRED_GT_ZERO) { CLT_TH(CLT_PRED_GT_ZERO); }
  CLT_TH(CLT_PRED_NONZERO);
#undef CLT_TH
}

// ---- encoder-collected candidates: workspace and the two halves of the fused path ---------
struct TileLayout {
  SelLayout sel;
  size_t off_tmeta, off_meta, off_tpool, off_cgt, off_ceq, off_pgt, off_peq, off_tcount, total;
  unsigned long long tpool_cap;              // entries per layer
  uint32_t caps;                             // entries per fixed tile slot
  int nseg, ntile;
};

static TileLayout tile_layout(int64_t T, int64_t F, int64_t L, int64_t k, int dtype) {
  TileLayout tl;
  tl.sel = sel_layout(T, F, L, k, CLT_TOPK_PER_LAYER);
  const int segw = dtype != CLT_F32 ? 128 : 64;
  tl.nseg = (int)(collect_grid_rows(F) / segw);   // whole feature tiles too (COLLECT_TILE_ROWS is the tile's side)
  const int64_t Tp = collect_grid_rows(T);   // the epilogue's books cover whole token tiles
  tl.ntile = tl.nseg * (int)(Tp / COLLECT_ROWS);
  // about 1.5x K candidates are expected, i.e. 1.5 * k / F of a tile's 64 * segw elements; a
  // slot holds three times that (at least 64, at most the whole tile)
  unsigned long long caps = (unsigned long long)(3.0 * 1.5 * (double)k / (double)F * (double)COLLECT_ROWS * segw) + 64ull;
  if (caps > (unsigned long long)COLLECT_ROWS * segw) caps = (unsigned long long)COLLECT_ROWS * segw;
  tl.caps = (uint32_t)caps;
  const unsigned long long N = (unsigned long long)T * F;
  unsigned long long K = (unsigned long long)k * T;
  if (K > N) K = N;
  unsigned long long dyn = 2ull * K + 4096ull;
  if (dyn > N) dyn = N;
  tl.tpool_cap = (unsigned long long)tl.ntile * caps + dyn;
  size_t o = tl.sel.total;
  auto take = [&](size_t bytes) { size_t at = o; o += (bytes + 255) & ~(size_t)255; return at; };
  tl.off_tmeta = take(8 * (size_t)tl.ntile * (size_t)L);
  tl.off_meta = take(8 * (size_t)tl.nseg * (size_t)Tp * (size_t)L);
  tl.off_tpool = take(8 * (size_t)tl.tpool_cap * (size_t)L);
  const size_t cells = (size_t)tl.nseg * (size_t)Tp * (size_t)L;   // (row, segment) pairs
  tl.off_cgt = take(cells);
  tl.off_ceq = take(cells);
  tl.off_pgt = take(4 * cells);
  tl.off_peq = take(4 * cells);
  tl.off_tcount = take(4 * (size_t)L);
  tl.total = o;
  return tl;
}

template <typename T>
static int run_encode_collect(const void *x, const void *w, const void *b, void *pre, int64_t Tn, int64_t d,
                              int64_t F, int64_t L, int64_t xs, int64_t wstr, int64_t bs, int64_t ps, int64_t k,
                              int dtype, char *ws, hipStream_t stream) {
  constexpr int KB = Elem<T>::KEYBITS;
  const TileLayout tl = tile_layout(Tn, F, L, k, dtype);
  const SelLayout &lo = tl.sel;
  SelState *st = (SelState *)(ws + lo.off_state);
  uint32_t *hist = (uint32_t *)(ws + lo.off_hist);
  uint32_t *poolcnt = (uint32_t *)(ws + lo.off_poolcnt);
  uint32_t *sample = (uint32_t *)(ws + lo.off_sample);
  const unsigned long long N = (unsigned long long)Tn * (unsigned long long)F;
  unsigned long long K = (unsigned long long)k * (unsigned long long)Tn;
  if (K > N) K = N;
  k_sample_mfma<T><<<dim3(SAMPLE_WAVES / 4, (unsigned)L), 256, 0, stream>>>((const T *)x, (const T *)w, (const T *)b, Tn, d,
                                                                          F, xs, wstr, bs, sample);
  k_sample_cut<T, SAMPLE_PRE_N><<<(unsigned)L, SCAN_THREADS, 0, stream>>>(sample, N, K, st, hist, poolcnt,
                                                              (uint32_t *)(ws + tl.off_tcount), PATH_TILES);
  uint2 *tpool = (uint2 *)(ws + tl.off_tpool);
  CollectArgs ca;
  ca.st = st; ca.pool_count = (uint32_t *)(ws + tl.off_tcount); ca.pool = tpool; ca.pool_cap = tl.tpool_cap;
  ca.tile_meta = (uint2 *)(ws + tl.off_tmeta); ca.seg_meta = (uint2 *)(ws + tl.off_meta); ca.caps = tl.caps;
  ca.theta = nullptr; ca.theta_stride = 0;
  int rc = clt_launch_encode(x, w, b, nullptr, Tn, d, F, L, xs, wstr, bs, ps, dtype, 1, nullptr, &ca, stream);
  if (rc != CLT_OK) return rc;
  k_pool_hist<T><<<dim3(256, (unsigned)L), 256, 0, stream>>>(st, ca.tile_meta, tl.ntile, tpool, tl.tpool_cap, hist, 0);
  k_select_scan<T><<<(unsigned)L, SCAN_THREADS, 0, stream>>>(st, hist, poolcnt, 0, 0);
  // layers whose cut failed (too few candidates, or no pool space left) get their pre-activations
  // written out and go through the streaming pass; the launch does nothing for the others
  return clt_launch_encode(x, w, b, pre, Tn, d, F, L, xs, wstr, bs, ps, dtype, 0, st, nullptr, stream);
}

template <typename T>
static int run_collect_select(const T *pre, int64_t Tn, int64_t F, int64_t L, int64_t lstride, int64_t k, int dtype,
                              int32_t *row_ptr, int32_t *col, T *val, char *ws, hipStream_t stream) {
  constexpr int KB = Elem<T>::KEYBITS;
  constexpr int VV = Elem<T>::VEC;
  const TileLayout tl = tile_layout(Tn, F, L, k, dtype);
  const SelLayout &lo = tl.sel;
  SelState *st = (SelState *)(ws + lo.off_state);
  uint32_t *hist = (uint32_t *)(ws + lo.off_hist);
  uint32_t *poolcnt = (uint32_t *)(ws + lo.off_poolcnt);
  uint32_t *first = (uint32_t *)(ws + lo.off_first);
  uint32_t *rgt = (uint32_t *)(ws + lo.off_gt), *req = (uint32_t *)(ws + lo.off_eq);
  uint32_t *allot = (uint32_t *)(ws + lo.off_allot), *keep = (uint32_t *)(ws + lo.off_keep);
  uint2 *pool = (uint2 *)(ws + lo.off_pool);
  const uint2 *meta = (const uint2 *)(ws + tl.off_meta);
  const uint2 *tmeta = (const uint2 *)(ws + tl.off_tmeta);
  const uint2 *tpool = (const uint2 *)(ws + tl.off_tpool);
  const unsigned long long N = (unsigned long long)Tn * (unsigned long long)F;
  unsigned long long K = (unsigned long long)k * (unsigned long long)Tn;
  if (K > N) K = N;
  int gx = (int)clt_ceil_div(Tn, 8);
  if (gx > 65535 * 8) gx = 65535 * 8;
  // retry of the layers whose cut failed: streaming pass from the bottom key over `pre`
  k_select_pass<T, VV, false><<<dim3(gx, (unsigned)L), 256, 0, stream>>>(pre, Tn, F, L, lstride, nullptr, nullptr, st, hist,
                                                                        poolcnt, pool, lo.pool_cap, first, 1, nullptr);
  k_select_scan<T><<<(unsigned)L, SCAN_THREADS, 0, stream>>>(st, hist, poolcnt, 1, 0);
  int gx2 = (int)clt_ceil_div(Tn, 4);
  int maxgx2 = (int)clt_ceil_div(256 * 8, L);
  if (maxgx2 < 1) maxgx2 = 1;
  if (gx2 > maxgx2) gx2 = maxgx2;
  dim3 grid2(gx2, (unsigned)L);
  const int nlev = KB == 32 ? 3 : 2;
  for (int level = 1; level < nlev; ++level) {
    k_pool_hist<T><<<dim3(256, (unsigned)L), 256, 0, stream>>>(st, tmeta, tl.ntile, tpool, tl.tpool_cap, hist, level);
    k_select_level<T, false><<<grid2, 256, 0, stream>>>(pre, Tn, F, L, lstride, nullptr, nullptr, st, hist, first, pool, lo.pool_cap, level);
    k_select_scan<T><<<(unsigned)L, SCAN_THREADS, 0, stream>>>(st, hist, poolcnt, 2, level);
  }
  dim3 grid3((unsigned)clt_ceil_div(Tn, 256), (unsigned)tl.nseg, (unsigned)L);
  uint8_t *cgt = (uint8_t *)(ws + tl.off_cgt), *ceq = (uint8_t *)(ws + tl.off_ceq);
  uint32_t *pgt = (uint32_t *)(ws + tl.off_pgt), *peq = (uint32_t *)(ws + tl.off_peq);
  const int64_t Tp = collect_grid_rows(Tn);
  k_tile_count<T><<<grid3, 256, 0, stream>>>((int)Tn, (int)Tp, st, meta, tl.nseg, tpool, tl.tpool_cap, cgt, ceq);
  k_row_prefix<<<dim3((unsigned)clt_ceil_div(Tn, 64), (unsigned)L), 64, 0, stream>>>(Tn, Tp, st, tl.nseg, cgt, ceq, pgt, peq, rgt, req);
  k_select_count<T, false><<<grid2, 256, 0, stream>>>(pre, Tn, F, L, lstride, nullptr, nullptr, st, first, pool, lo.pool_cap, rgt, req);
  k_select_allot<false><<<(unsigned)L, SCAN_THREADS, 0, stream>>>(st, Tn, L, rgt, req, allot, keep, row_ptr, K);
  k_tile_emit<T><<<grid3, 256, 0, stream>>>((int)Tn, (int)Tp, st, meta, tl.nseg, tpool, tl.tpool_cap, pgt, peq, allot, row_ptr, col, val);
  k_select_emit<T, false><<<grid2, 256, 0, stream>>>(pre, Tn, F, L, lstride, nullptr, nullptr, st, first, pool, lo.pool_cap, allot,
                                                     row_ptr, col, val);
  return clt_check_launch();
}

// ---- JumpReLU on the encoder epilogue -----------------------------------------------------------
struct ThreshLayout {
  size_t off_state, off_tcount, off_tmeta, off_meta, off_tpool, off_pfx, off_rowcnt, total;
  unsigned long long tpool_cap;
  uint32_t caps;
  int nseg, ntile;
};

static ThreshLayout thresh_layout(int64_t T, int64_t F, int64_t L, int64_t density_ppm, int dtype) {
  ThreshLayout tl;
  const int segw = dtype != CLT_F32 ? 128 : 64;
  tl.nseg = (int)(collect_grid_rows(F) / segw);   // whole feature tiles too (COLLECT_TILE_ROWS is the tile's side)
  const int64_t Tp = collect_grid_rows(T);   // the epilogue's books cover whole token tiles
  tl.ntile = tl.nseg * (int)(Tp / COLLECT_ROWS);
  const double dens = (double)(density_ppm < 1 ? 1 : density_ppm) * 1e-6;
  // a fixed slot holds three times the expected entries of a tile (at least 64, at most the tile)
  unsigned long long caps = (unsigned long long)(3.0 * dens * (double)COLLECT_ROWS * segw) + 64ull;
  if (caps > (unsigned long long)COLLECT_ROWS * segw) caps = (unsigned long long)COLLECT_ROWS * segw;
  tl.caps = (uint32_t)caps;
  const unsigned long long N = (unsigned long long)T * F;
  unsigned long long dyn = (unsigned long long)(2.0 * dens * (double)N) + 4096ull;
  if (dyn > N) dyn = N;
  tl.tpool_cap = (unsigned long long)tl.ntile * caps + dyn;
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += (bytes + 255) & ~(size_t)255; return at; };
  tl.off_state = take(sizeof(SelState) * (size_t)L);
  tl.off_tcount = take(4 * (size_t)L);
  tl.off_tmeta = take(8 * (size_t)tl.ntile * (size_t)L);
  tl.off_meta = take(8 * (size_t)tl.nseg * (size_t)Tp * (size_t)L);
  tl.off_tpool = take(8 * (size_t)tl.tpool_cap * (size_t)L);
  tl.off_pfx = take(4 * (size_t)tl.nseg * (size_t)Tp * (size_t)L);
  tl.off_rowcnt = take(4 * (size_t)T * (size_t)L);
  tl.total = o;
  return tl;
}

}  // namespace

extern "C" int clt_encode_threshold_supported(const void *x, const void *w, const void *b, const void *theta,
                                              int64_t T, int64_t d, int64_t F, int64_t L, int64_t x_layer_stride,
                                              int64_t w_layer_stride, int64_t b_layer_stride,
                                              int64_t theta_layer_stride, int64_t density_ppm, int dtype) {
  if (!clt_model_dtype(dtype)) return 0;
  if (T <= 0 || d <= 0 || F <= 0 || L <= 0 || L > 65535 || !x || !w || !theta) return 0;
  if ((double)T * (double)F >= 4294967296.0 || (double)T * (double)L >= 2147483647.0) return 0;
  if (!clt_aligned16(theta) || (theta_layer_stride * clt_elem_bytes(dtype)) % 16 != 0) return 0;
  if (thresh_layout(T, F, L, density_ppm, dtype).tpool_cap >= 0xFFF00000ull) return 0;
  return clt_encode_can_collect(x, w, b, T, d, F, x_layer_stride, w_layer_stride, b_layer_stride, dtype) ? 1 : 0;
}

extern "C" size_t clt_encode_threshold_workspace_bytes(int64_t T, int64_t d, int64_t F, int64_t L,
                                                       int64_t density_ppm, int dtype) {
  (void)d;
  if (T <= 0 || F <= 0 || L <= 0) return 256;
  return thresh_layout(T, F, L, density_ppm, dtype).total;
}

extern "C" int clt_encode_threshold_count(const void *x, const void *w, const void *b, const void *theta, int64_t T,
                                          int64_t d, int64_t F, int64_t L, int64_t x_layer_stride,
                                          int64_t w_layer_stride, int64_t b_layer_stride,
                                          int64_t theta_layer_stride, int64_t density_ppm, int dtype,
                                          int32_t *row_ptr, void *workspace, size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (!row_ptr || !workspace) return CLT_ERR_ARG;
  if (!clt_encode_threshold_supported(x, w, b, theta, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                                      theta_layer_stride, density_ppm, dtype))
    return CLT_ERR_ARG;
  const ThreshLayout tl = thresh_layout(T, F, L, density_ppm, dtype);
  if (workspace_bytes < tl.total) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  char *ws = (char *)workspace;
  SelState *st = (SelState *)(ws + tl.off_state);
  // state (only the overflow flags are used) and the pool counters start at zero; they are adjacent
  k_fill_u32<<<8, 256, 0, s>>>((uint32_t *)(ws + tl.off_state), 0u, (int64_t)((tl.off_tmeta - tl.off_state) / 4));
  CollectArgs ca;
  ca.st = st; ca.pool_count = (uint32_t *)(ws + tl.off_tcount); ca.pool = (uint2 *)(ws + tl.off_tpool);
  ca.pool_cap = tl.tpool_cap; ca.tile_meta = (uint2 *)(ws + tl.off_tmeta); ca.seg_meta = (uint2 *)(ws + tl.off_meta);
  ca.caps = tl.caps; ca.theta = theta; ca.theta_stride = theta_layer_stride;
  int rc = clt_launch_encode(x, w, b, nullptr, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride, 0, dtype, 2,
                             nullptr, &ca, s);
  if (rc != CLT_OK) return rc;
  uint32_t *rowcnt = (uint32_t *)(ws + tl.off_rowcnt);
  k_row_prefix_meta<<<dim3((unsigned)clt_ceil_div(T, 64), (unsigned)L), 64, 0, s>>>(T, collect_grid_rows(T), tl.nseg, ca.seg_meta,
                                                                                    (uint32_t *)(ws + tl.off_pfx), rowcnt);
  k_rowptr_scan<<<1, SCAN_THREADS, 0, s>>>(rowcnt, L * T, row_ptr);
  k_thresh_finish<<<1, 64, 0, s>>>(st, (int)L, row_ptr, L * T);
  return clt_check_launch();
}

__global__ void k_survivors_fit_clear(int32_t *row_ptr, int64_t n, const int32_t *status);

// ---- the fused threshold route's fallback, decided and run on the device ---------------------------------
// status[0] != 0: the pool list is not the one to emit (the dense route holds the list, or there is none)
// status[1] != 0: the dense route is not the one to emit
// status[2] != 0: the batch has no survivor list (more entries than `capacity`); the list was emptied
__global__ void k_recover_flag(SelState *st, int L, const int32_t *row_ptr, int64_t R, int32_t *status) {
  const bool over = row_ptr[R] == -1;
  for (int l = threadIdx.x; l < L; l += blockDim.x) st[l].status = over ? ST_RETRY : ST_RUN;
  if (threadIdx.x == 0) { status[0] = over ? 1 : 0; status[1] = over ? 0 : 1; status[2] = 0; }
}
__global__ void k_recover_guard(const int32_t *row_ptr, int64_t R, int64_t capacity, int32_t *status) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const int32_t tot = row_ptr[R];
  if (tot < 0 || (int64_t)tot > capacity) { status[0] = 1; status[1] = 1; status[2] = 1; }
}

extern "C" int clt_encode_threshold_recover(const void *x, const void *w, const void *b, const void *theta, void *pre,
                                            int64_t T, int64_t d, int64_t F, int64_t L, int64_t x_layer_stride,
                                            int64_t w_layer_stride, int64_t b_layer_stride, int64_t theta_layer_stride,
                                            int64_t pre_layer_stride, int64_t density_ppm, int dtype, int32_t *row_ptr,
                                            int64_t capacity, int32_t *status, void *workspace, size_t workspace_bytes,
                                            void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (!row_ptr || !workspace || !status || !pre || capacity < 0) return CLT_ERR_ARG;
  if (!clt_encode_threshold_supported(x, w, b, theta, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                                      theta_layer_stride, density_ppm, dtype))
    return CLT_ERR_ARG;
  if (theta_layer_stride != F) return CLT_ERR_ARG;       // the dense compare walks theta as [L][F]
  const ThreshLayout tl = thresh_layout(T, F, L, density_ppm, dtype);
  if (workspace_bytes < tl.total) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  char *ws = (char *)workspace;
  SelState *st = (SelState *)(ws + tl.off_state);
  const int64_t R = L * T;
  k_recover_flag<<<1, 64, 0, s>>>(st, (int)L, row_ptr, R, status);
  // every launch below returns at once unless the pool overflowed: the projection is stored densely (all
  // layers carry ST_RETRY then), counted against the thresholds, and the row pointers are rebuilt
  int rc = clt_launch_encode(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                             pre_layer_stride, dtype, 0, st, nullptr, s);
  if (rc != CLT_OK) return rc;
  uint32_t *rowcnt = (uint32_t *)(ws + tl.off_rowcnt);
  if (dtype == CLT_BF16)
    rc = dispatch_threshold<bf16_t>(false, pre, T, F, L, pre_layer_stride, theta, CLT_PRED_GE_THETA, rowcnt, row_ptr, nullptr,
                                    nullptr, status + 1, s);
  else if (dtype == CLT_F16)
    rc = dispatch_threshold<f16_t>(false, pre, T, F, L, pre_layer_stride, theta, CLT_PRED_GE_THETA, rowcnt, row_ptr, nullptr,
                                    nullptr, status + 1, s);
  else
    rc = dispatch_threshold<float>(false, pre, T, F, L, pre_layer_stride, theta, CLT_PRED_GE_THETA, rowcnt, row_ptr, nullptr,
                                   nullptr, status + 1, s);
  if (rc != CLT_OK) return rc;
  k_recover_guard<<<1, 64, 0, s>>>(row_ptr, R, capacity, status);
  k_survivors_fit_clear<<<256, 256, 0, s>>>(row_ptr, R + 1, status + 2);
  return clt_check_launch();
}

extern "C" int clt_encode_threshold_emit(int64_t T, int64_t F, int64_t L, int64_t density_ppm, int dtype,
                                         const int32_t *row_ptr, int32_t *col, void *val, const int32_t *skip,
                                         void *workspace, size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || !row_ptr || !col || !val || !workspace) return CLT_ERR_ARG;
  const ThreshLayout tl = thresh_layout(T, F, L, density_ppm, dtype);
  if (workspace_bytes < tl.total) return CLT_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char *ws = (char *)workspace;
  dim3 grid((unsigned)clt_ceil_div(T, 256), (unsigned)tl.nseg, (unsigned)L);
  if (dtype == CLT_BF16)
    k_tile_emit_all<bf16_t><<<grid, 256, 0, s>>>((int)T, (int)collect_grid_rows(T), (const uint2 *)(ws + tl.off_meta), tl.nseg, (const uint2 *)(ws + tl.off_tpool),
                                                  tl.tpool_cap, (const uint32_t *)(ws + tl.off_pfx), row_ptr, col, (bf16_t *)val, skip);
  else if (dtype == CLT_F16)
    k_tile_emit_all<f16_t><<<grid, 256, 0, s>>>((int)T, (int)collect_grid_rows(T), (const uint2 *)(ws + tl.off_meta), tl.nseg, (const uint2 *)(ws + tl.off_tpool),
                                                  tl.tpool_cap, (const uint32_t *)(ws + tl.off_pfx), row_ptr, col, (f16_t *)val, skip);
  else
    k_tile_emit_all<float><<<grid, 256, 0, s>>>((int)T, (int)collect_grid_rows(T), (const uint2 *)(ws + tl.off_meta), tl.nseg, (const uint2 *)(ws + tl.off_tpool),
                                                 tl.tpool_cap, (const uint32_t *)(ws + tl.off_pfx), row_ptr, col, (float *)val, skip);
  return clt_check_launch();
}

extern "C" int clt_encode_collect_supported(const void *x, const void *w, const void *b, int64_t T, int64_t d,
                                            int64_t F, int64_t L, int64_t x_layer_stride, int64_t w_layer_stride,
                                            int64_t b_layer_stride, int64_t k, int dtype) {
  if (!clt_model_dtype(dtype)) return 0;
  if (T <= 0 || d <= 0 || F <= 0 || L <= 0 || L > 65535 || k <= 0 || !x || !w) return 0;
  if ((double)T * (double)F >= 4294967296.0) return 0;
  if (tile_layout(T, F, L, k, dtype).tpool_cap >= 0xFFF00000ull) return 0;
  return clt_encode_can_collect(x, w, b, T, d, F, x_layer_stride, w_layer_stride, b_layer_stride, dtype) ? 1 : 0;
}

extern "C" size_t clt_encode_collect_workspace_bytes(int64_t T, int64_t d, int64_t F, int64_t L, int64_t k, int dtype) {
  (void)d;
  if (T <= 0 || F <= 0 || L <= 0) return 256;
  if (k < 0) k = 0;
  return tile_layout(T, F, L, k, dtype).total;
}

extern "C" int clt_encode_collect(const void *x, const void *w, const void *b, void *pre, int64_t T, int64_t d,
                                  int64_t F, int64_t L, int64_t x_layer_stride, int64_t w_layer_stride,
                                  int64_t b_layer_stride, int64_t pre_layer_stride, int64_t k, int dtype,
                                  void *workspace, size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (!pre || !workspace) return CLT_ERR_ARG;
  if (!clt_encode_collect_supported(x, w, b, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride, k, dtype))
    return CLT_ERR_ARG;
  if (workspace_bytes < clt_encode_collect_workspace_bytes(T, d, F, L, k, dtype)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16)
    return run_encode_collect<bf16_t>(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                                      pre_layer_stride, k, dtype, (char *)workspace, s);
  if (dtype == CLT_F16)
    return run_encode_collect<f16_t>(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                                      pre_layer_stride, k, dtype, (char *)workspace, s);
  return run_encode_collect<float>(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                                   pre_layer_stride, k, dtype, (char *)workspace, s);
}

extern "C" int clt_collect_select(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride, int64_t k,
                                  int dtype, int32_t *row_ptr, int32_t *col, void *val, void *workspace,
                                  size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 65535 || k <= 0) return CLT_ERR_ARG;
  if (!pre || !row_ptr || !col || !val || !workspace) return CLT_ERR_ARG;
  if (workspace_bytes < clt_encode_collect_workspace_bytes(T, 0, F, L, k, dtype)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16)
    return run_collect_select<bf16_t>((const bf16_t *)pre, T, F, L, pre_layer_stride, k, dtype, row_ptr, col, (bf16_t *)val, (char *)workspace, s);
  if (dtype == CLT_F16)
    return run_collect_select<f16_t>((const f16_t *)pre, T, F, L, pre_layer_stride, k, dtype, row_ptr, col, (f16_t *)val, (char *)workspace, s);
  return run_collect_select<float>((const float *)pre, T, F, L, pre_layer_stride, k, dtype, row_ptr, col, (float *)val, (char *)workspace, s);
}

extern "C" size_t clt_batchtopk_workspace_bytes(int64_t T, int64_t F, int64_t L, int64_t k, int mode, int dtype) {
  (void)dtype;
  if (T <= 0 || F <= 0 || L <= 0) return 256;
  if (k < 0) k = 0;
  return sel_layout(T, F, L, k, mode).total;
}

extern "C" int clt_batchtopk_select(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                                    int64_t k, int mode, const float *mean, const float *denom, int dtype,
                                    int32_t *row_ptr, int32_t *col, void *val, void *workspace,
                                    size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0 || L > 65535 || !row_ptr) return CLT_ERR_ARG;
  if (mode != CLT_TOPK_PER_LAYER && mode != CLT_TOPK_GLOBAL) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int64_t R = L * T;
  if (k <= 0 || T == 0 || F == 0) {
    k_fill_u32<<<64, 256, 0, s>>>((uint32_t *)row_ptr, 0u, R + 1);
    return clt_check_launch();
  }
  if (!pre || !col || !val || !workspace) return CLT_ERR_ARG;
  if (mode == CLT_TOPK_GLOBAL && (!mean || !denom)) return CLT_ERR_ARG;
  if ((double)T * (double)F * (double)L >= 4294967296.0) return CLT_ERR_RANGE;
  if (workspace_bytes < clt_batchtopk_workspace_bytes(T, F, L, k, mode, dtype)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0) return CLT_ERR_ALIGN;
  char *ws = (char *)workspace;
  if (dtype == CLT_BF16) {
    if (mode == CLT_TOPK_GLOBAL)
      return run_batchtopk_v<bf16_t, true>((const bf16_t *)pre, T, F, L, pre_layer_stride, k, mean, denom, row_ptr, col, (bf16_t *)val, ws, s);
    return run_batchtopk_v<bf16_t, false>((const bf16_t *)pre, T, F, L, pre_layer_stride, k, mean, denom, row_ptr, col, (bf16_t *)val, ws, s);
  }
  if (dtype == CLT_F16) {
    if (mode == CLT_TOPK_GLOBAL)
      return run_batchtopk_v<f16_t, true>((const f16_t *)pre, T, F, L, pre_layer_stride, k, mean, denom, row_ptr, col, (f16_t *)val, ws, s);
    return run_batchtopk_v<f16_t, false>((const f16_t *)pre, T, F, L, pre_layer_stride, k, mean, denom, row_ptr, col, (f16_t *)val, ws, s);
  }
  if (mode == CLT_TOPK_GLOBAL)
    return run_batchtopk_v<float, true>((const float *)pre, T, F, L, pre_layer_stride, k, mean, denom, row_ptr, col, (float *)val, ws, s);
  return run_batchtopk_v<float, false>((const float *)pre, T, F, L, pre_layer_stride, k, mean, denom, row_ptr, col, (float *)val, ws, s);
}

extern "C" int clt_threshold_count(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                                   const void *theta, int pred, int dtype, int32_t *row_ptr, void *workspace,
                                   size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0 || L > 65535 || !row_ptr) return CLT_ERR_ARG;
  if (pred < 0 || pred > 2 || (pred == CLT_PRED_GE_THETA && !theta)) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int64_t R = L * T;
  if (T == 0 || F == 0) {
    k_fill_u32<<<64, 256, 0, s>>>((uint32_t *)row_ptr, 0u, R + 1);
    return clt_check_launch();
  }
  if (!pre || !workspace) return CLT_ERR_ARG;
  if (F >= 2147483648LL || R >= 2147483647LL) return CLT_ERR_RANGE;   // the survivor total must also stay below 2^31
  if (workspace_bytes < (size_t)R * 4) return CLT_ERR_WORKSPACE;
  uint32_t *cnt = (uint32_t *)workspace;
  if (dtype == CLT_BF16) return dispatch_threshold<bf16_t>(false, pre, T, F, L, pre_layer_stride, theta, pred, cnt, row_ptr, nullptr, nullptr, nullptr, s);
  if (dtype == CLT_F16) return dispatch_threshold<f16_t>(false, pre, T, F, L, pre_layer_stride, theta, pred, cnt, row_ptr, nullptr, nullptr, nullptr, s);
  return dispatch_threshold<float>(false, pre, T, F, L, pre_layer_stride, theta, pred, cnt, row_ptr, nullptr, nullptr, nullptr, s);
}

// ---- threshold activation kept dense ----------------------------------------------------------------------
// x[l][t][f] <- x if the predicate holds, else 0, in place; total += the number kept.  One 16-byte piece per
// thread and step where rows are whole pieces, else element by element.
template <typename T, int PRED, bool VEC>
__global__ __launch_bounds__(256) void k_threshold_dense(T *__restrict__ x, const T *__restrict__ theta, int64_t Tn, int64_t F,
                                                         int64_t lstride, unsigned long long *__restrict__ total) {
  constexpr int V = VEC ? 16 / (int)sizeof(T) : 1;
  const int l = blockIdx.y;
  T *xl = x + (int64_t)l * lstride;
  const T *th = PRED == CLT_PRED_GE_THETA ? theta + (int64_t)l * F : nullptr;
  const int64_t per_row = F / V, n = Tn * per_row;
  uint32_t kept = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / per_row, c = (i - r * per_row) * V;
    T *p = xl + r * F + c;
    if constexpr (VEC) {
      uint4 v = *reinterpret_cast<const uint4 *>(p), t4 = make_uint4(0, 0, 0, 0);
      if (PRED == CLT_PRED_GE_THETA) t4 = *reinterpret_cast<const uint4 *>(th + c);
      uint32_t w[4] = {v.x, v.y, v.z, v.w};
      const uint32_t tw[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (sizeof(T) == 4) {
          const bool keep = pred_keep<T, PRED>(__uint_as_float(w[k]), __uint_as_float(tw[k]));
          kept += keep ? 1u : 0u;
          w[k] = keep ? w[k] : 0u;
        } else {
          float xa, xb, ta, tb;
          unpack_pair<T>(w[k], xa, xb);
          unpack_pair<T>(tw[k], ta, tb);
          const bool ka = pred_keep<T, PRED>(xa, ta), kb = pred_keep<T, PRED>(xb, tb);
          kept += (ka ? 1u : 0u) + (kb ? 1u : 0u);
          w[k] &= (ka ? 0x0000FFFFu : 0u) | (kb ? 0xFFFF0000u : 0u);
        }
      }
      *reinterpret_cast<uint4 *>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
      const float xv = Elem<T>::to_f32(*p);
      const bool keep = pred_keep<T, PRED>(xv, PRED == CLT_PRED_GE_THETA ? Elem<T>::to_f32(th[c]) : 0.0f);
      kept += keep ? 1u : 0u;
      if (!keep) *p = Elem<T>::from_raw(0u);
    }
  }
  __shared__ uint32_t red[4];
  for (int o = 32; o > 0; o >>= 1) kept += __shfl_xor(kept, o);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = kept;
  __syncthreads();
  if (threadIdx.x == 0) atomicAdd(total, (unsigned long long)red[0] + red[1] + red[2] + red[3]);
}

extern "C" int clt_threshold_dense(void *x, int64_t T, int64_t F, int64_t L, int64_t layer_stride, const void *theta,
                                   int pred, int dtype, uint64_t *total, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0 || L > 65535 || !total) return CLT_ERR_ARG;
  if ((pred != CLT_PRED_GE_THETA && pred != CLT_PRED_GT_ZERO) || (pred == CLT_PRED_GE_THETA && !theta)) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  k_fill_u32<<<1, 64, 0, s>>>((uint32_t *)total, 0u, 2);
  if (T == 0 || F == 0) return clt_check_launch();
  if (!x) return CLT_ERR_ARG;
  const int esz = clt_elem_bytes(dtype), vec = 16 / esz;
  const bool vecok = F % vec == 0 && clt_aligned16(x) && (layer_stride * esz) % 16 == 0 && (!theta || clt_aligned16(theta));
  dim3 grid(2048, (unsigned)L);
#define CLT_TD(CT, P, VK) k_threshold_dense<CT, P, VK><<<grid, 256, 0, s>>>((CT *)x, (const CT *)theta, T, F, layer_stride, (unsigned long long *)total)
#define CLT_TD_T(CT)                                                                            \
  do {                                                                                          \
    if (pred == CLT_PRED_GE_THETA) { if (vecok) CLT_TD(CT, CLT_PRED_GE_THETA, true); else CLT_TD(CT, CLT_PRED_GE_THETA, false); } \
    else { if (vecok) CLT_TD(CT, CLT_PRED_GT_ZERO, true); else CLT_TD(CT, CLT_PRED_GT_ZERO, false); }                             \
  } while (0)
  if (dtype == CLT_BF16) CLT_TD_T(bf16_t);
  else if (dtype == CLT_F16) CLT_TD_T(f16_t);
  else CLT_TD_T(float);
#undef CLT_TD_T
#undef CLT_TD
  return clt_check_launch();
}

// ---- sizing col / val without reading the total back -------------------------------------------------
__global__ void k_survivors_fit_flag(const int32_t *row_ptr, int64_t R, int64_t capacity, int32_t *status) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    const int32_t tot = row_ptr[R];
    *status = (tot < 0 || (int64_t)tot > capacity) ? 1 : 0;
  }
}
__global__ void k_survivors_fit_clear(int32_t *row_ptr, int64_t n, const int32_t *status) {
  if (*status == 0) return;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) row_ptr[i] = 0;
}

extern "C" int clt_survivors_fit(int32_t *row_ptr, int64_t R, int64_t capacity, int32_t *status, void *stream) {
  if (!row_ptr || !status || R < 0 || capacity < 0) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  k_survivors_fit_flag<<<1, 64, 0, s>>>(row_ptr, R, capacity, status);
  k_survivors_fit_clear<<<256, 256, 0, s>>>(row_ptr, R + 1, status);
  return clt_check_launch();
}

// ---- clt_threshold_count for callers that cannot allocate ---------------------------------------
// The per-row counters of clt_threshold_count live in a file-scope device array instead of a caller
// workspace.  In host code `scratch` is only a handle for the symbol: the address a kernel can use is
// looked up once per device with hipGetSymbolAddress (every GPU holds its own copy of the array at
// its own address) and that pointer is what the launches get.
constexpr int64_t STATIC_ROWS_MAX = 1 << 20;          // L*T rows: 4 MiB of counters per GPU
constexpr int STATIC_MAX_DEVICES = 64;
static __device__ __align__(256) uint32_t scratch[STATIC_ROWS_MAX];
static uint32_t *g_scratch_ptr[STATIC_MAX_DEVICES];   // device address of `scratch`, per device
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(uint32_t **out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) return CLT_ERR_ARG;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return CLT_ERR_LAUNCH;
    g_scratch_ptr[dev] = (uint32_t *)p;
  }
  *out = g_scratch_ptr[dev];
  return CLT_OK;
}

extern "C" int clt_threshold_count_static(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                                          const void *theta, int pred, int dtype, int32_t *row_ptr, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0 || L > 65535 || !row_ptr) return CLT_ERR_ARG;
  if (L * T > STATIC_ROWS_MAX) return CLT_ERR_RANGE;
  uint32_t *cnt = nullptr;
  const int rc = scratch_of_current_device(&cnt);
  if (rc != CLT_OK) return rc;
  // every counter of the L*T rows in use is written before it is read, so nothing has to be cleared
  return clt_threshold_count(pre, T, F, L, pre_layer_stride, theta, pred, dtype, row_ptr, cnt,
                             (size_t)STATIC_ROWS_MAX * 4, stream);
}

extern "C" int clt_threshold_emit(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                                  const void *theta, int pred, int dtype, const int32_t *row_ptr, int32_t *col,
                                  void *val, const int32_t *skip, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0 || L > 65535 || !row_ptr) return CLT_ERR_ARG;
  if (pred < 0 || pred > 2 || (pred == CLT_PRED_GE_THETA && !theta)) return CLT_ERR_ARG;
  if (T == 0 || F == 0) return CLT_OK;
  if (!pre || !col || !val) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == CLT_BF16) return dispatch_threshold<bf16_t>(true, pre, T, F, L, pre_layer_stride, theta, pred, nullptr, (int32_t *)row_ptr, col, val, skip, s);
  if (dtype == CLT_F16) return dispatch_threshold<f16_t>(true, pre, T, F, L, pre_layer_stride, theta, pred, nullptr, (int32_t *)row_ptr, col, val, skip, s);
  return dispatch_threshold<float>(true, pre, T, F, L, pre_layer_stride, theta, pred, nullptr, (int32_t *)row_ptr, col, val, skip, s);
}

extern "C" int clt_selected_min_accumulate(const int32_t *row_ptr, const int32_t *col, const void *val, const float *mean,
                                           const float *denom, int64_t T, int64_t F, int64_t L, int dtype, void *sum,
                                           void *count, void *workspace, size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || !row_ptr || !mean || !denom || !sum || !count || !workspace) return CLT_ERR_ARG;
  if (workspace_bytes < (size_t)L * (size_t)F * 4) return CLT_ERR_WORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  uint32_t *keys = (uint32_t *)workspace;
  const int64_t n = L * F;
  k_fill_u32<<<256, 256, 0, s>>>(keys, 0xFFFFFFFFu, n);
  if (dtype == CLT_BF16) {
    k_selected_min<bf16_t><<<2048, 256, 0, s>>>(row_ptr, col, (const bf16_t *)val, mean, denom, T, F, L, keys);
    k_selected_min_accumulate<bf16_t><<<256, 256, 0, s>>>(keys, n, (bf16_t *)sum, (bf16_t *)count);
  } else if (dtype == CLT_F16) {
    k_selected_min<f16_t><<<2048, 256, 0, s>>>(row_ptr, col, (const f16_t *)val, mean, denom, T, F, L, keys);
    k_selected_min_accumulate<f16_t><<<256, 256, 0, s>>>(keys, n, (f16_t *)sum, (f16_t *)count);
  } else {
    k_selected_min<float><<<2048, 256, 0, s>>>(row_ptr, col, (const float *)val, mean, denom, T, F, L, keys);
    k_selected_min_accumulate<float><<<256, 256, 0, s>>>(keys, n, (float *)sum, (float *)count);
  }
  return clt_check_launch();
}

extern "C" size_t clt_tokentopk_workspace_bytes(int64_t T, int64_t F, int64_t L, int64_t kk, int mode, int dtype) {
  (void)F; (void)kk; (void)mode; (void)dtype;
  if (T <= 0 || L <= 0) return 256;
  return tok_layout(T, L).total;
}

extern "C" int clt_tokentopk_select(const void *pre, int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                                    int64_t kk, int mode, const float *mean, const float *denom, int dtype,
                                    int32_t *row_ptr, int32_t *col, void *val, void *workspace,
                                    size_t workspace_bytes, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || F < 0 || L <= 0 || L > TOK_MAX_LAYERS || !row_ptr) return CLT_ERR_ARG;
  if (mode != CLT_TOPK_PER_LAYER && mode != CLT_TOPK_GLOBAL) return CLT_ERR_ARG;
  hipStream_t s = (hipStream_t)stream;
  const int64_t R = L * T;
  if (kk <= 0 || T == 0 || F == 0) {
    k_fill_u32<<<64, 256, 0, s>>>((uint32_t *)row_ptr, 0u, R + 1);
    return clt_check_launch();
  }
  if (!pre || !col || !val || !workspace) return CLT_ERR_ARG;
  if (mode == CLT_TOPK_GLOBAL && (!mean || !denom)) return CLT_ERR_ARG;
  if ((double)T * (double)L * (double)(kk < F * L ? kk : F * L) >= 2147483648.0 || F >= 2147483648LL) return CLT_ERR_RANGE;
  if (workspace_bytes < clt_tokentopk_workspace_bytes(T, F, L, kk, mode, dtype)) return CLT_ERR_WORKSPACE;
  const int64_t rowlen = mode == CLT_TOPK_GLOBAL ? L * F : F;
  if (kk > rowlen) kk = rowlen;
  char *ws = (char *)workspace;
  if (dtype == CLT_BF16) {
    if (mode == CLT_TOPK_GLOBAL)
      return run_tokentopk<bf16_t, true>((const bf16_t *)pre, T, F, L, pre_layer_stride, kk, mean, denom, row_ptr, col, (bf16_t *)val, ws, s);
    return run_tokentopk<bf16_t, false>((const bf16_t *)pre, T, F, L, pre_layer_stride, kk, mean, denom, row_ptr, col, (bf16_t *)val, ws, s);
  }
  if (dtype == CLT_F16) {
    if (mode == CLT_TOPK_GLOBAL)
      return run_tokentopk<f16_t, true>((const f16_t *)pre, T, F, L, pre_layer_stride, kk, mean, denom, row_ptr, col, (f16_t *)val, ws, s);
    return run_tokentopk<f16_t, false>((const f16_t *)pre, T, F, L, pre_layer_stride, kk, mean, denom, row_ptr, col, (f16_t *)val, ws, s);
  }
  if (mode == CLT_TOPK_GLOBAL)
    return run_tokentopk<float, true>((const float *)pre, T, F, L, pre_layer_stride, kk, mean, denom, row_ptr, col, (float *)val, ws, s);
  return run_tokentopk<float, false>((const float *)pre, T, F, L, pre_layer_stride, kk, mean, denom, row_ptr, col, (float *)val, ws, s);
}
