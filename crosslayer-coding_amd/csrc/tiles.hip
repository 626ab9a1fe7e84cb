// Decoder weight gradient + Adam over COLUMN TILES, for untied decoders.
//
// The row-at-a-time kernel (backward.hip, k_feature_outer) sums a gradient row by gathering one row of
// d loss / d reconstruction per list entry through the vector memory path: at the sizes this library is
// built for that is ~40 KB of L2 reads per row beside the 7.5 KB of moments and parameters the Adam step
// streams, and both compete for the same miss queue of the compute unit.  Here the roles are turned round:
// a workgroup parks ONE column slice of one target's d loss / d reconstruction -- [T tokens][32 bytes] --
// in its LDS and then runs over every (source <= target, feature) row for that slice, so that the gather
// is LDS traffic and the vector memory path carries only what must come from memory once: the token /
// coefficient lists and the moments and parameters of the slice.
//
// For that the optimiser keeps the decoder weights and both moments in a tiled layout
//   [n_dec][NS = d / CS][F][CS]      CS = 32 bytes of the model dtype (16 bf16 / 8 fp32 columns)
// in which the slice of consecutive features is contiguous: a wavefront (32 rows, two lanes per row, 16 bytes
// of parameters per lane) reads and writes whole cache lines.  clt_tile_decoders / clt_untile_decoders
// convert between this layout and the feature-major slab [n_dec][F][pitch] (+ the checkpoint layout [d][F]).
//
// Arithmetic: one fused multiply-add per (entry, column) in ascending token order (fp32 fmaf; for bf16
// v_dot2_f32_bf16 with the partner factor zero, whose product is exact) and the same adam_update as the row
// kernel; the sum of a list that the kernel cuts between two lane pairs is associated differently (see
// k_tile_outer_adam), so results agree with clt_decoder_weight_grad + clt_adam_step_decoders to fp32 rounding
// of the gradient, not bit for bit, and repeat bit for bit from run to run.
// (reference: loss.backward() and optimizer.step() of clt/training/trainer.py:663-778 for the decoder weights.)
#include <type_traits>

#include "adam.h"
#include "clt_common.h"

namespace {

constexpr int TL_THREADS = 768;             // 12 wavefronts; the slice takes most of the LDS: one workgroup per CU
constexpr int TL_WAVES = TL_THREADS / 64;
constexpr int TL_ROWS = 32;                 // rows per wavefront step: two lanes per row in the Adam phase
constexpr int TL_SLICE_BYTES = 32;          // bytes of one token in the parked slice
constexpr int TL_STAGE_BYTES = TL_ROWS * 16 * 4;                              // per wavefront: 32 rows x 16 fp32
constexpr int64_t TL_LDS_MAX = 160 * 1024 - TL_WAVES * TL_STAGE_BYTES - 64;   // what the slice may take
constexpr int64_t TL_CHUNK = 2048;          // features per work unit (a multiple of TL_ROWS)
constexpr int TL_PRE = 8;                   // groups of four entries of a range asked for at once
constexpr int TL_PAD = 192;                 // entries the regrouped lists are padded with (read, never used)

__device__ __forceinline__ int64_t tl_slot(int64_t s, int64_t t, int64_t L) { return s * L - (s * (s - 1)) / 2 + (t - s); }

// list entries as the kernel wants them: token and coefficient side by side ...
template <typename T> struct TlPair;
template <> struct TlPair<bf16_t> {
  typedef uint32_t type;    // token | coefficient bits << 16
  __device__ static __forceinline__ type make(int32_t tok, bf16_t c) { return (uint32_t)tok | ((uint32_t)c << 16); }
  __device__ static __forceinline__ int tok(type p) { return (int)(p & 0xFFFFu); }
  __device__ static __forceinline__ float coef(type p) { return __uint_as_float(p & 0xFFFF0000u); }
};
template <> struct TlPair<float> {
  typedef uint2 type;
  __device__ static __forceinline__ type make(int32_t tok, float c) { return make_uint2((uint32_t)tok, __float_as_uint(c)); }
  __device__ static __forceinline__ int tok(type p) { return (int)p.x; }
  __device__ static __forceinline__ float coef(type p) { return __uint_as_float(p.y); }
};

// ... and one byte per entry: the feature's place in its block of 32 (bits 0-4), bit 7 on the last entry of a list.
// Eight lanes per list.
template <typename T>
__global__ __launch_bounds__(256) void k_tile_pairs(const int32_t *__restrict__ ptr, int64_t nlist, int64_t F,
                                                     const int32_t *__restrict__ tok, const int32_t *__restrict__ src,
                                                     const T *__restrict__ val, typename TlPair<T>::type *__restrict__ pairs,
                                                     uint8_t *__restrict__ rowb, uint32_t *ticket) {
  if (blockIdx.x == 0 && threadIdx.x == 0) *ticket = 0u;
  const int sub = threadIdx.x & 7;
  for (int64_t q = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 3; q < nlist; q += ((int64_t)gridDim.x * blockDim.x) >> 3) {
    const int32_t b = ptr[q], e = ptr[q + 1];
    const uint8_t place = (uint8_t)((q % F) & (TL_ROWS - 1));
    for (int32_t i0 = b + sub; i0 < e; i0 += 32) {
      // four entries per lane with their loads in flight together (token and position, then the value)
      int32_t tk[4], sr[4];
      T vl[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int32_t i = i0 + 8 * u < e ? i0 + 8 * u : e - 1;
        tk[u] = tok[i]; sr[u] = src[i];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) vl[u] = val[sr[u]];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int32_t i = i0 + 8 * u;
        if (i < e) {
          pairs[i] = TlPair<T>::make(tk[u], vl[u]);
          rowb[i] = place | (i == e - 1 ? 0x80 : 0);
        }
      }
    }
  }
}

typedef float tl_f4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t tl_u4 __attribute__((ext_vector_type(4)));

template <typename T> __device__ __forceinline__ void tl_unpack(const uint4 &v, float *x) {
  if constexpr (sizeof(T) == 2) {
    x[0] = __uint_as_float(v.x << 16); x[1] = __uint_as_float(v.x & 0xFFFF0000u);
    x[2] = __uint_as_float(v.y << 16); x[3] = __uint_as_float(v.y & 0xFFFF0000u);
    x[4] = __uint_as_float(v.z << 16); x[5] = __uint_as_float(v.z & 0xFFFF0000u);
    x[6] = __uint_as_float(v.w << 16); x[7] = __uint_as_float(v.w & 0xFFFF0000u);
  } else {
    x[0] = __uint_as_float(v.x); x[1] = __uint_as_float(v.y); x[2] = __uint_as_float(v.z); x[3] = __uint_as_float(v.w);
  }
}

// Work unit = (target t, column slice cs, feature chunk k): all rows (source s <= t, feature in the chunk) of
// that slice.  Units are handed out by a ticket counter, large targets first, so the last ones are small.
//
// A wavefront step takes 32 consecutive rows of one source.  Their lists are one contiguous run of entries, and
// list lengths are very uneven (a few features fire on many tokens), so the ENTRIES, not the rows, are dealt
// out: the run is cut into 32 equal ranges, one per lane pair (the two lanes of a pair hold the two 16-byte
// halves of the slice).  A lane pair sums along its range; at the last entry of a list it writes the sum to the
// row's place in a staging area in LDS and starts again from zero; what it holds when its range ends in the
// middle of a list stays in its registers.  Then the step turns to rows: lane pair r owns row r, adds the
// leftovers of the ranges that ended inside its list, in range order, then the staged sum, and applies Adam.
// The order of the additions is fixed, so results repeat bit for bit; a list that lies within one range is
// summed exactly as k_feature_outer sums it, one cut by a range boundary in a different (fixed) association.
template <typename T>
__global__ __launch_bounds__(TL_THREADS) void k_tile_outer_adam(
    const int32_t *__restrict__ ptr, const typename TlPair<T>::type *__restrict__ pairs, const uint8_t *__restrict__ rowb,
    const T *__restrict__ g, T *__restrict__ w_t, float *__restrict__ m_t, float *__restrict__ v_t, int64_t Tn, int64_t d,
    int64_t F, int64_t L, int NS, int NK, AdamCoef c, uint32_t *ticket) {
  extern __shared__ uint4 tl_lds[];        // slice [Tn][2] 16-byte pieces, then the staging areas of the wavefronts
  __shared__ uint32_t unit_sh;
  constexpr int EL = 16 / (int)sizeof(T), CS = 2 * EL, NQ = EL / 4;   // NQ: 16-byte pieces of a lane's fp32 values
  typedef typename TlPair<T>::type pair_t;
  const int lane = lane_id(), wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), h = lane & 1, rl = lane >> 1;
  uint4 *slice = tl_lds;
  const char *slice_h = reinterpret_cast<const char *>(tl_lds) + h * 16;    // this lane's half of every token
  // staging: [32 rows][2 halves][NQ pieces]; a bf16 half is 8 fp32 = 2 pieces, an fp32 half 4 fp32 = 1 piece
  uint4 *stage = tl_lds + Tn * 2 + (int64_t)wv * (TL_STAGE_BYTES / 16);
  const uint32_t total = (uint32_t)(L * NS * NK);
  for (;;) {
    __syncthreads();      // all wavefronts have left the slice and have read unit_sh
    if (threadIdx.x == 0) unit_sh = atomicAdd(ticket, 1u);
    __syncthreads();
    const uint32_t u = unit_sh;
    if (u >= total) break;
    const int64_t t = L - 1 - (int64_t)(u / (uint32_t)(NS * NK));
    const uint32_t rest = u % (uint32_t)(NS * NK);
    const int64_t k = rest / (uint32_t)NS, cs = rest % (uint32_t)NS;
    {
      // six loads in flight per thread (one at a time would cost a memory latency per 384 tokens)
      const T *gt = g + t * Tn * d + cs * CS + (threadIdx.x & 1) * EL;
      constexpr int FB = 6, STEP = TL_THREADS / 2;
      for (int64_t base = threadIdx.x >> 1; base < Tn; base += FB * STEP) {
        uint4 tmp[FB];
#pragma unroll
        for (int u2 = 0; u2 < FB; ++u2) {      // (past the end: the last token again, not stored)
          const int64_t tk = base + u2 * STEP < Tn ? base + u2 * STEP : Tn - 1;
          tmp[u2] = *reinterpret_cast<const uint4 *>(gt + tk * d);
        }
#pragma unroll
        for (int u2 = 0; u2 < FB; ++u2)
          if (base + u2 * STEP < Tn) slice[(base + u2 * STEP) * 2 + (threadIdx.x & 1)] = tmp[u2];
      }
    }
    __syncthreads();
    const int64_t f_begin = k * TL_CHUNK, f_end = f_begin + TL_CHUNK < F ? f_begin + TL_CHUNK : F;
    const int64_t nblk = (f_end - f_begin + TL_ROWS - 1) / TL_ROWS;
    // row blocks wv, wv + 12, ... of the (t + 1) * nblk blocks of the unit, as (source, block) without a division;
    // everything derived from them is the same for the whole wavefront and stays in scalar registers
    int sb = 0, blk = wv;
    for (;; blk += TL_WAVES) {
      while (blk >= (int)nblk) { blk -= (int)nblk; ++sb; }
      if (sb > (int)t) break;
      const int64_t s = sb, f0 = f_begin + (int64_t)blk * TL_ROWS, f = f0 + rl;
      const int nrows = (int)(f_end - f0 < TL_ROWS ? f_end - f0 : TL_ROWS);
      const int64_t q0 = s * F + f0;
      // this lane pair's row as a list: [p_lo, p_hi) (empty beyond the chunk)
      const int32_t p_lo = ptr[q0 + (rl < nrows ? rl : nrows)], p_hi = ptr[q0 + (rl + 1 < nrows ? rl + 1 : nrows)];
      const int32_t B = __builtin_amdgcn_readfirstlane(p_lo), E = __builtin_amdgcn_readlane(p_hi, 63);
      const int32_t A0 = B & ~3;
      const int32_t n_per = (((E - A0 + 31) >> 5) + 3) & ~3;    // entries per lane pair, a multiple of four
      const uint32_t start = (uint32_t)(A0 + rl * n_per);    // 32-bit offsets from uniform bases: one address add per load
      // The whole range is asked for first (up to TL_PRE groups of four entries stay in registers), then the
      // moments and the parameters, which come from memory and take longest: loads return in order, so the
      // gather runs on the entries while the Adam operands are still on their way, and nothing is asked for
      // behind them.  (Ranges longer than that -- 32 rows with more than 1024 entries -- load as they go.)
      pair_t pq[TL_PRE][4];
      uint32_t rq[TL_PRE];
#pragma unroll
      for (int gq = 0; gq < TL_PRE; ++gq) {
        if (gq * 4 < n_per) {
#pragma unroll
          for (int j = 0; j < 4; ++j) pq[gq][j] = pairs[start + gq * 4 + j];
          rq[gq] = *reinterpret_cast<const uint32_t *>(rowb + start + gq * 4);
        }
      }
      const bool live = rl < nrows;
      const int64_t at_row0 = ((tl_slot(s, t, L) * NS + cs) * F + f0) * CS;     // uniform
      const uint32_t at_lane = (uint32_t)((live ? rl : 0) * CS + h * EL);
      float *const m_at = m_t + at_row0 + at_lane, *const v_at = v_t + at_row0 + at_lane;
      T *const w_at = w_t + at_row0 + at_lane;
      // (asked for by every lane, rows beyond the chunk read row f0 again: a branch here would make the
      // compiler wait for these loads wherever it now waits for the entries)
      tl_f4 am[NQ], av[NQ];
#pragma unroll
      for (int j = 0; j < NQ; ++j) {
        am[j] = __builtin_nontemporal_load(reinterpret_cast<const tl_f4 *>(m_at) + j);
        av[j] = __builtin_nontemporal_load(reinterpret_cast<const tl_f4 *>(v_at) + j);
      }
      const tl_u4 aw = __builtin_nontemporal_load(reinterpret_cast<const tl_u4 *>(w_at));
      // empty lists have no last entry: their staged sum is the zero written here
#pragma unroll
      for (int j = 0; j < NQ; ++j) stage[(rl * 2 + h) * NQ + j] = make_uint4(0, 0, 0, 0);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      float acc[EL];
#pragma unroll
      for (int j = 0; j < EL; ++j) acc[j] = 0.0f;
      // one entry: gather its piece of the slice, multiply, and at the end of a list park the sum
      auto fetch = [&](const pair_t &pr) {
        return *reinterpret_cast<const uint4 *>(slice_h + (uint32_t)TlPair<T>::tok(pr) * TL_SLICE_BYTES);
      };
      auto entry = [&](const pair_t &pr, const uint4 &piece, uint32_t rbyte) {
        if constexpr (sizeof(T) == 2) {
          // bf16 x bf16 products are exact in fp32, and with the partner factor zero v_dot2 is one fused
          // multiply-add per column without unpacking: (x_lo, x_hi) . (c, 0) and (x_lo, x_hi) . (0, c)
          const bf16x2_t c_lo = __builtin_bit_cast(bf16x2_t, (uint32_t)(pr >> 16)), c_hi = __builtin_bit_cast(bf16x2_t, (uint32_t)(pr & 0xFFFF0000u));
          const uint32_t w4[4] = {piece.x, piece.y, piece.z, piece.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            acc[2 * e] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w4[e]), c_lo, acc[2 * e], false);
            acc[2 * e + 1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, w4[e]), c_hi, acc[2 * e + 1], false);
          }
        } else {
          const float cf = TlPair<T>::coef(pr);
          float x[EL];
          tl_unpack<T>(piece, x);
#pragma unroll
          for (int e = 0; e < EL; ++e) acc[e] = fmaf(cf, x[e], acc[e]);
        }
        if (rbyte & 0x80u) {
          uint4 *dst = stage + ((rbyte & 31u) * 2 + h) * NQ;
#pragma unroll
          for (int qd = 0; qd < NQ; ++qd) {
            dst[qd] = make_uint4(__float_as_uint(acc[4 * qd]), __float_as_uint(acc[4 * qd + 1]), __float_as_uint(acc[4 * qd + 2]),
                                 __float_as_uint(acc[4 * qd + 3]));
            acc[4 * qd] = acc[4 * qd + 1] = acc[4 * qd + 2] = acc[4 * qd + 3] = 0.0f;
          }
        }
      };
      // a group of four: normally every lane's group lies wholly inside [B, E) or wholly outside, and the
      // wavefront takes the branch without per-entry bounds tests (a uniform branch: one of the two bodies
      // runs); only the groups at the two ends of the run have lanes with part of a group inside
      auto group = [&](const pair_t *pr, uint32_t rw, int32_t i) {
        const int32_t i0 = (int32_t)start + i;
        const bool whole = i0 >= B && i0 + 4 <= E, some = i0 + 4 > B && i0 < E;
        if (__builtin_amdgcn_ballot_w64(some && !whole) == 0) {
          if (whole) {
            uint4 pc[4];      // the four LDS reads go out together: their latency is paid once per group
#pragma unroll
            for (int j = 0; j < 4; ++j) pc[j] = fetch(pr[j]);
#pragma unroll
            for (int j = 0; j < 4; ++j) entry(pr[j], pc[j], (rw >> (8 * j)) & 0xFFu);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if ((uint32_t)(i0 + j - B) < (uint32_t)(E - B)) entry(pr[j], fetch(pr[j]), (rw >> (8 * j)) & 0xFFu);
        }
      };
#pragma unroll
      for (int gq = 0; gq < TL_PRE; ++gq)
        if (gq * 4 < n_per) group(pq[gq], rq[gq], gq * 4);
      for (int32_t i = TL_PRE * 4; i < n_per; i += 4) {
        pair_t pr[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) pr[j] = pairs[start + i + j];
        group(pr, *reinterpret_cast<const uint32_t *>(rowb + start + i), i);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      // rows: the leftovers of the ranges m = first .. last whose end A0 + m * n_per lies strictly inside this list
      float tot[EL];
#pragma unroll
      for (int e = 0; e < EL; ++e) tot[e] = 0.0f;
      int m_first = 1, m_last = 0;
      if (n_per) {
        // x / n_per for 0 <= x < 2^22 through the reciprocal: the estimate is off by at most one
        const float rn = 1.0f / (float)n_per;
        auto quot = [&](int32_t x) {
          int32_t qv = (int32_t)((float)x * rn);
          qv -= qv * n_per > x ? 1 : 0;
          qv += (qv + 1) * n_per <= x ? 1 : 0;
          return qv;
        };
        m_first = quot(p_lo - A0) + 1;
        m_last = quot(p_hi - A0 + n_per - 1) - 1;
      }
      // every lane takes part in every exchange (the source lane differs per row: lane pair m - 1 holds the
      // leftover of range m); the trip count is that of the list cut most often, normally one or two
      bool any = false;
      for (int m = m_first; __builtin_amdgcn_ballot_w64(m <= m_last) != 0; ++m) {
        const bool mine = m <= m_last;
        const int srcl = mine ? (m - 1) * 2 + h : lane;
#pragma unroll
        for (int e = 0; e < EL; ++e) {
          const float part = __shfl(acc[e], srcl);
          if (mine) tot[e] = any ? tot[e] + part : part;
        }
        any = any || mine;
      }
      {
        const uint4 *srcp = stage + (rl * 2 + h) * NQ;
#pragma unroll
        for (int qd = 0; qd < NQ; ++qd) {
          const uint4 sv = srcp[qd];
          const float st[4] = {__uint_as_float(sv.x), __uint_as_float(sv.y), __uint_as_float(sv.z), __uint_as_float(sv.w)};
#pragma unroll
          for (int e = 0; e < 4; ++e) tot[4 * qd + e] = any ? tot[4 * qd + e] + st[e] : st[e];
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");    // the staging area is read before the next step clears it
      if (!live) continue;
      float mm[EL], vv[EL], pp[EL];
#pragma unroll
      for (int j = 0; j < NQ; ++j) {
        mm[4 * j] = am[j].x; mm[4 * j + 1] = am[j].y; mm[4 * j + 2] = am[j].z; mm[4 * j + 3] = am[j].w;
        vv[4 * j] = av[j].x; vv[4 * j + 1] = av[j].y; vv[4 * j + 2] = av[j].z; vv[4 * j + 3] = av[j].w;
      }
      tl_unpack<T>(make_uint4(aw.x, aw.y, aw.z, aw.w), pp);
      T np[EL];
#pragma unroll
      for (int e = 0; e < EL; ++e) np[e] = Elem<T>::from_f32(adam_update(pp[e], tot[e], mm[e], vv[e], c));
#pragma unroll
      for (int j = 0; j < NQ; ++j) {
        tl_f4 mo = {mm[4 * j], mm[4 * j + 1], mm[4 * j + 2], mm[4 * j + 3]}, vo = {vv[4 * j], vv[4 * j + 1], vv[4 * j + 2], vv[4 * j + 3]};
        __builtin_nontemporal_store(mo, reinterpret_cast<tl_f4 *>(m_at) + j);
        __builtin_nontemporal_store(vo, reinterpret_cast<tl_f4 *>(v_at) + j);
      }
      tl_u4 wo;
      if constexpr (sizeof(T) == 2) {
        wo.x = (uint32_t)np[0] | ((uint32_t)np[1] << 16); wo.y = (uint32_t)np[2] | ((uint32_t)np[3] << 16);
        wo.z = (uint32_t)np[4] | ((uint32_t)np[5] << 16); wo.w = (uint32_t)np[6] | ((uint32_t)np[7] << 16);
      } else {
        wo.x = __float_as_uint(np[0]); wo.y = __float_as_uint(np[1]); wo.z = __float_as_uint(np[2]); wo.w = __float_as_uint(np[3]);
      }
      __builtin_nontemporal_store(wo, reinterpret_cast<tl_u4 *>(w_at));
    }
  }
}

// ---- layout conversions: 64 features x 64 columns per workgroup through LDS, whole lines on both sides ----
// TO_TILES: slab [n_dec][F][pitch] -> tiles.  Otherwise tiles -> slab and, when w_refs is given, -> the
// checkpoint layout [d][F] of every decoder.
template <typename T, bool TO_TILES>
__global__ __launch_bounds__(256) void k_tile_convert(T *__restrict__ slab, T *__restrict__ tiles, T *const *__restrict__ w_refs,
                                                       int64_t d, int64_t F, int64_t pitch, int NS) {
  constexpr int EL = 16 / (int)sizeof(T), CS = 2 * EL, PPR = 64 / EL;   // 16-byte pieces per 64-column row
  __shared__ __attribute__((aligned(16))) T tile[64][64 + EL];
  const int64_t dec = blockIdx.z, f0 = (int64_t)blockIdx.x * 64, d0 = (int64_t)blockIdx.y * 64;
  T *sl = slab + dec * F * pitch;
  T *tl = tiles + dec * NS * F * CS;
  // row-major pieces: p -> (feature p / PPR, piece p % PPR); tile-major pieces: p -> (slice, feature, half)
  auto slab_piece = [&](int p, bool store) {
    const int fl = p / PPR, pc = p % PPR;
    const int64_t f = f0 + fl, dd = d0 + pc * EL;
    if (f >= F || dd >= d) return;
    uint4 *mem = reinterpret_cast<uint4 *>(sl + f * pitch + dd), *lds = reinterpret_cast<uint4 *>(&tile[fl][pc * EL]);
    if (store) *mem = *lds; else *lds = *mem;
  };
  auto tile_piece = [&](int p, bool store) {
    const int cl = p / 128, fl = (p % 128) >> 1, hh = p & 1;
    const int64_t f = f0 + fl, dd = d0 + cl * CS + hh * EL;
    if (f >= F || dd >= d) return;
    uint4 *mem = reinterpret_cast<uint4 *>(tl + ((dd / CS) * F + f) * CS + hh * EL), *lds = reinterpret_cast<uint4 *>(&tile[fl][cl * CS + hh * EL]);
    if (store) *mem = *lds; else *lds = *mem;
  };
  constexpr int NP = 64 * PPR;
  for (int p = threadIdx.x; p < NP; p += 256) { if (TO_TILES) slab_piece(p, false); else tile_piece(p, false); }
  __syncthreads();
  for (int p = threadIdx.x; p < NP; p += 256) { if (TO_TILES) tile_piece(p, true); else slab_piece(p, true); }
  if (!TO_TILES && w_refs) {
    T *o = w_refs[dec];
    typedef typename std::conditional<sizeof(T) == 2, uint2, uint4>::type quad_t;
    const int qd = threadIdx.x & 15, r = threadIdx.x >> 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dl = r + 16 * i;
      const int64_t dd = d0 + dl, f = f0 + qd * 4;
      if (dd < d && f < F) {       // F % 4 == 0
        T t4[4];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) t4[kk] = tile[qd * 4 + kk][dl];
        *reinterpret_cast<quad_t *>(o + dd * F + f) = *reinterpret_cast<const quad_t *>(t4);
      }
    }
  }
}

static int tl_width(int dtype) { return TL_SLICE_BYTES / (dtype == CLT_BF16 ? 2 : 4); }

}  // namespace

extern "C" int clt_decoder_tile_width(int64_t T, int64_t d, int64_t F, int dtype) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return 0;
  const int cs = tl_width(dtype);
  if (T <= 0 || d <= 0 || F <= 0 || d % cs != 0 || F % 4 != 0) return 0;
  if (T > 65536 || T * TL_SLICE_BYTES > TL_LDS_MAX) return 0;
  // ... and the device must grant a workgroup that much LDS (160 KB per compute unit on gfx950)
  int dev = 0, lds_max = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&lds_max, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  if (T * TL_SLICE_BYTES + (int64_t)TL_WAVES * TL_STAGE_BYTES + 64 > (int64_t)lds_max) return 0;
  if ((d / cs) * clt_ceil_div(F, TL_CHUNK) > (1 << 24)) return 0;
  return cs;
}

static size_t tl_pairs_bytes(int64_t capacity, int dtype) {
  return ((((size_t)capacity + TL_PAD) * (dtype == CLT_BF16 ? 4 : 8)) + 255) & ~(size_t)255;
}

extern "C" size_t clt_decoder_tiles_workspace_bytes(int64_t capacity, int dtype) {
  if (capacity < 0) capacity = 0;
  return 256 + tl_pairs_bytes(capacity, dtype) + (((size_t)capacity + TL_PAD + 255) & ~(size_t)255);
}

extern "C" int clt_tile_decoders(const void *w_packed, void *w_tiles, int64_t n_dec, int64_t d, int64_t F, int dtype,
                                 void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (n_dec <= 0 || d <= 0 || F <= 0 || n_dec > 65535 || !w_packed || !w_tiles) return CLT_ERR_ARG;
  const int cs = tl_width(dtype);
  if (d % cs != 0 || F % 4 != 0) return CLT_ERR_RANGE;
  if (!clt_aligned16(w_packed) || !clt_aligned16(w_tiles)) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)clt_ceil_div(d, 64), (unsigned)n_dec);
  if (dtype == CLT_BF16)
    k_tile_convert<bf16_t, true><<<grid, 256, 0, s>>>((bf16_t *)w_packed, (bf16_t *)w_tiles, nullptr, d, F, clt_pitch(d, 2), (int)(d / cs));
  else
    k_tile_convert<float, true><<<grid, 256, 0, s>>>((float *)w_packed, (float *)w_tiles, nullptr, d, F, clt_pitch(d, 4), (int)(d / cs));
  return clt_check_launch();
}

extern "C" int clt_untile_decoders(const void *w_tiles, void *w_packed, void *const *w_refs_dev, void *const *w_refs_host,
                                   int64_t n_dec, int64_t d, int64_t F, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (n_dec <= 0 || d <= 0 || F <= 0 || n_dec > 65535 || !w_packed || !w_tiles) return CLT_ERR_ARG;
  if ((w_refs_dev == nullptr) != (w_refs_host == nullptr)) return CLT_ERR_ARG;
  const int cs = tl_width(dtype);
  if (d % cs != 0 || F % 4 != 0) return CLT_ERR_RANGE;
  if (!clt_aligned16(w_packed) || !clt_aligned16(w_tiles)) return CLT_ERR_ALIGN;
  for (int64_t i = 0; w_refs_host && i < n_dec; ++i)
    if (!w_refs_host[i] || (((uintptr_t)w_refs_host[i]) & (dtype == CLT_BF16 ? 7u : 15u)) != 0) return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)clt_ceil_div(F, 64), (unsigned)clt_ceil_div(d, 64), (unsigned)n_dec);
  if (dtype == CLT_BF16)
    k_tile_convert<bf16_t, false><<<grid, 256, 0, s>>>((bf16_t *)w_packed, (bf16_t *)w_tiles, (bf16_t *const *)w_refs_dev, d, F, clt_pitch(d, 2), (int)(d / cs));
  else
    k_tile_convert<float, false><<<grid, 256, 0, s>>>((float *)w_packed, (float *)w_tiles, (float *const *)w_refs_dev, d, F, clt_pitch(d, 4), (int)(d / cs));
  return clt_check_launch();
}

extern "C" int clt_decoder_weight_grad_adam_tiled(const int32_t *list_ptr, const int32_t *list_tok, const int32_t *list_src,
                                                  const void *val, const void *g_model, void *w_tiles, float *m_tiles,
                                                  float *v_tiles, int64_t T, int64_t d, int64_t F, int64_t L, int64_t capacity,
                                                  double lr, double beta1, double beta2, double eps, int64_t step, int dtype,
                                                  void *workspace, size_t workspace_bytes, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T <= 0 || F <= 0 || L <= 0 || L > 64 || capacity < 0 || step < 1 || !(beta1 >= 0 && beta1 < 1) || !(beta2 >= 0 && beta2 < 1) ||
      !list_ptr || !list_tok || !list_src || !val || !g_model || !w_tiles || !m_tiles || !v_tiles || !workspace)
    return CLT_ERR_ARG;
  const int cs = clt_decoder_tile_width(T, d, F, dtype);
  if (cs == 0) return CLT_ERR_RANGE;
  if (workspace_bytes < clt_decoder_tiles_workspace_bytes(capacity, dtype)) return CLT_ERR_WORKSPACE;
  if ((((uintptr_t)workspace) & 255u) != 0 || !clt_aligned16(g_model) || !clt_aligned16(w_tiles) || !clt_aligned16(m_tiles) ||
      !clt_aligned16(v_tiles))
    return CLT_ERR_ALIGN;
  hipStream_t s = (hipStream_t)stream;
  uint32_t *ticket = (uint32_t *)workspace;
  void *pairs = (char *)workspace + 256;
  uint8_t *rowb = (uint8_t *)pairs + tl_pairs_bytes(capacity, dtype);
  const int NS = (int)(d / cs), NK = (int)clt_ceil_div(F, TL_CHUNK);
  const size_t lds = (size_t)T * TL_SLICE_BYTES + (size_t)TL_WAVES * TL_STAGE_BYTES;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) {
    (void)hipGetLastError();
    cus = 256;
  }
  const AdamCoef c = adam_coef(lr, beta1, beta2, eps, step);
#define CLT_TILE(CT)                                                                                                        \
  do {                                                                                                                      \
    typedef TlPair<CT>::type pair_t;                                                                                        \
    k_tile_pairs<CT><<<2048, 256, 0, s>>>(list_ptr, L * F, F, list_tok, list_src, (const CT *)val, (pair_t *)pairs, rowb, ticket); \
    if (lds > 64 * 1024 &&                                                                                                  \
        hipFuncSetAttribute((const void *)k_tile_outer_adam<CT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) { \
      (void)hipGetLastError();                                                                                              \
      return CLT_ERR_LAUNCH;                                                                                                \
    }                                                                                                                       \
    k_tile_outer_adam<CT><<<(unsigned)cus, TL_THREADS, lds, s>>>(list_ptr, (const pair_t *)pairs, rowb, (const CT *)g_model, \
                                                                  (CT *)w_tiles, m_tiles, v_tiles, T, d, F, L, NS, NK, c, ticket); \
  } while (0)
  if (dtype == CLT_BF16) CLT_TILE(bf16_t); else CLT_TILE(float);
#undef CLT_TILE
  return clt_check_launch();
}
