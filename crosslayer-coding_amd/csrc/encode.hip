// Encoder projection  pre[l] = x[l] . W[l]^T + b[l]   (reference clt/models/parallel.py:286)
//
// MFMA kernel for gfx950.  Both operands are K-contiguous (x is [T][d], W is [F][d]), so
// one loader serves both.
//
//   block tile  256 tokens x 256 features, 4 wavefronts (2 x 2), wave tile 128 x 128:
//               256 fp32 accumulators per lane, one wavefront per SIMD, one block per CU
//   k step      128 bytes of K per LDS stage (64 bf16 / 32 fp32), two stages of 64 KB
//   loads       global_load_lds_dwordx4: 16 bytes per lane straight into LDS, no staging
//               registers.  LDS rows are 128 bytes; chunk c of row r lives at chunk position
//               c ^ ((r >> 1) & 7), which the loader realises by permuting which global chunk
//               each lane fetches, so the 16-byte fragment reads of a wavefront spread over
//               all banks
//   math        the matrix-core "A" operand is the W tile and "B" the x tile, so a lane ends
//               up with 4 consecutive features of one token per accumulator group
//   bias        the accumulators start from the bias, so it is added in fp32 before the one rounding
//   epilogue    rounding, then the tile goes through LDS so that the stores are 16 bytes per lane
//               and 256 contiguous bytes per token
//   bf16        v_mfma_f32_32x32x16_bf16, fp32 accumulate, one rounding (v_cvt_pk_bf16_f32)
//   fp32        v_mfma_f32_32x32x2_f32
#include <type_traits>
#include "select_state.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int BM = 256;   // tokens per block
constexpr int BN = 256;   // features per block
constexpr int ROWB = 128; // bytes of K per LDS row
constexpr int STAGE = (BM + BN) * ROWB;  // bytes of one LDS stage
constexpr int NWAVES = 8;                // wavefronts per block (4 x 2, wave tile 64 tokens x 128 features): two per SIMD
constexpr int NTHREADS = NWAVES * 64;
constexpr int CAND_LIST = 512;           // candidates of one 32-token piece the collecting epilogue lists in LDS
constexpr int ENC_SN = 8;  // feature tiles x token tiles that one XCD works on at a time
constexpr int ENC_SM = 4;


template <typename T> struct Mma;
template <> struct Mma<bf16_t> {
  __device__ static __forceinline__ void run(f32x16_t &acc, const uint4 &a, const uint4 &b) {
    bf16x8_t av = __builtin_bit_cast(bf16x8_t, a), bv = __builtin_bit_cast(bf16x8_t, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
  }
};
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
template <> struct Mma<f16_t> {
  __device__ static __forceinline__ void run(f32x16_t &acc, const uint4 &a, const uint4 &b) {
    f16x8_t av = __builtin_bit_cast(f16x8_t, a), bv = __builtin_bit_cast(f16x8_t, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
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

// 16 bytes per lane from global memory straight into LDS: lane i of the wavefront lands at
// lds_base + 16 * i (lds_base must be wave-uniform).
__device__ __forceinline__ void load16_to_lds(const void *gsrc, void *lds_base) {
  __builtin_amdgcn_global_load_lds(gsrc, (__attribute__((address_space(3))) void *)lds_base, 16, 0, 0);
}

typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

// two fp32 -> packed 16-bit elements (round to nearest even; bf16: one v_cvt_pk_bf16_f32)
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
template <typename T> __device__ __forceinline__ uint32_t pack16x2(float a, float b) {
  f32x2_t v = {a, b};
  if constexpr (IsHalf<T>::value) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// element j of a 16-byte slot as a float / as raw bits
template <typename T> __device__ __forceinline__ float slot_elem(const uint4 &w, int j);
template <> __device__ __forceinline__ float slot_elem<float>(const uint4 &w, int j) {
  return __uint_as_float(j == 0 ? w.x : j == 1 ? w.y : j == 2 ? w.z : w.w);
}
template <> __device__ __forceinline__ float slot_elem<bf16_t>(const uint4 &w, int j) {
  const uint32_t u = (j >> 1) == 0 ? w.x : (j >> 1) == 1 ? w.y : (j >> 1) == 2 ? w.z : w.w;
  return __uint_as_float((j & 1) ? (u & 0xFFFF0000u) : (u << 16));
}
template <> __device__ __forceinline__ float slot_elem<f16_t>(const uint4 &w, int j) {
  const uint32_t u = (j >> 1) == 0 ? w.x : (j >> 1) == 1 ? w.y : (j >> 1) == 2 ? w.z : w.w;
  return f16_bits_to_f32((j & 1) ? (u >> 16) : (u & 0xFFFFu));
}
template <typename T> __device__ __forceinline__ uint32_t slot_raw(const uint4 &w, int j);
template <> __device__ __forceinline__ uint32_t slot_raw<float>(const uint4 &w, int j) {
  return j == 0 ? w.x : j == 1 ? w.y : j == 2 ? w.z : w.w;
}
template <> __device__ __forceinline__ uint32_t slot_raw<bf16_t>(const uint4 &w, int j) {
  const uint32_t u = (j >> 1) == 0 ? w.x : (j >> 1) == 1 ? w.y : (j >> 1) == 2 ? w.z : w.w;
  return (j & 1) ? (u >> 16) : (u & 0xFFFFu);
}

template <> __device__ __forceinline__ uint32_t slot_raw<f16_t>(const uint4 &w, int j) { return slot_raw<bf16_t>(w, j); }

// packed 16-bit helpers (two elements per 32-bit word)
typedef short i16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_sub_sat16(uint32_t a, uint32_t b) {   // signed saturating a - b
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_sub_sat(__builtin_bit_cast(i16x2_t, a), __builtin_bit_cast(i16x2_t, b)));
}
__device__ __forceinline__ uint32_t pk_sign16(uint32_t a) {                 // 0xFFFF where the half is negative
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(i16x2_t, a) >> (short)15);
}
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, a), __builtin_bit_cast(u16x2_t, b)));
}

// inclusive prefix sums with DPP row shifts: inside each row of 16 lanes / over the wavefront
__device__ __forceinline__ uint32_t row16_inclusive_scan(uint32_t v) {
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);  // row_shr:8
  return v;
}
__device__ __forceinline__ uint32_t wave_inclusive_scan32(uint32_t v) {
  v = row16_inclusive_scan(v);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);  // row_bcast:31
  return v;
}

// Requires K % (128 / sizeof(T)) == 0 (whole LDS stages), M >= BM and N >= BN.  A tile that
// would stick out of the matrix is shifted back inside (its overlap with the neighbour is
// computed twice and stored by the neighbour only), so no load is predicated.
//
// Block -> tile map: workgroups go to the 8 XCDs round-robin, so block b runs on XCD b % 8.
// When the feature tiles split evenly, XCD x takes the feature tiles n = x, x+8, ... in groups
// (see the map below): a W tile is fetched by one XCD only.
//
// COLLECT 0 stores the tile.  COLLECT 1 / 2 store nothing: the epilogue compares every element
// with the layer's cut value (1) or its feature's threshold (2) and appends the ones that reach
// it, as (feature, raw value) entries ordered by (token, feature), to one extent of the layer's
// candidate pool per wavefront and feature segment (see CollectArgs).  A tile that was shifted
// back, in either direction, reports only the tokens and features its neighbour does not own.
// SEG (storing mode only): K is made of segments of `sps` stages each; segment q of a row starts
// q * xss (x) / q * wss (W) elements after the row's first segment and rows are xrs / wrs elements apart,
// so both operands may be gathered from several matrices side by side (see clt_encode_segmented).
struct SegArgs {
  int sps;           // stages per segment
  uint32_t magic;    // ceil(2^32 / sps): segment of stage i = (i * magic) >> 32 for i < 2^16
  int64_t xss, wss;  // segment strides, elements
  int xrs, wrs;      // row strides, elements
};

template <typename T, int COLLECT, bool SEG, bool ODD>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_encode_mfma(
    const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias, T *__restrict__ pre,
    int M, int K, int N, int tiles_m, int tiles_n, int total_tiles, int64_t xs, int64_t wstr, int64_t bs,
    int64_t ps, const SelState *__restrict__ gate, CollectArgs ca, SegArgs sg, int by_tokens) {
  static_assert(!SEG || COLLECT == 0, "segmented operands only in the storing mode");
  static_assert(!SEG || !ODD, "segmented operands come in an even number of stages");
  constexpr int CE = 16 / (int)sizeof(T);  // elements per 16-byte chunk
  constexpr int BK = ROWB / (int)sizeof(T);
  // Persistent workgroups (the grid is one block per CU, block b takes the tiles b, b + gridDim.x, ...)
  // that overlap the start of the next tile with the end of this one: the epilogue parks only in the
  // second stage buffer, 32 tokens of a wave tile at a time, so the first stage of the next tile is asked
  // for two stages before this tile's K loop ends and has landed when the epilogue is over.
  // Two separate stage buffers (not one array with an offset): the compiler can then tell that
  // a fragment read of one stage does not depend on the direct-to-LDS loads in flight into the
  // other, and does not wait for them.
  __shared__ __attribute__((aligned(16))) unsigned char stage0[STAGE];
  __shared__ __attribute__((aligned(16))) unsigned char stage1[STAGE];
  __shared__ uint16_t cand_list[COLLECT ? NWAVES : 1][COLLECT ? CAND_LIST : 1];   // per wavefront, see the emission
  __shared__ __attribute__((aligned(16))) T bias_lds[NWAVES][128];                // per wavefront: the bias of its features
  __shared__ __attribute__((aligned(16))) T theta_lds[COLLECT == 2 ? NWAVES : 1][COLLECT == 2 ? 128 : 8];   // and their thresholds
  __shared__ __attribute__((aligned(16))) uint32_t cut_lds[COLLECT == 1 ? NWAVES : 1][4];                   // the layer's cut key

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 3, wn = wave >> 2;   // wave tile: tokens [64 wm, +64) x features [128 wn, +128)
  const int per_layer = tiles_m * tiles_n;
  // The K loop walks its stages in pairs.  An odd number of stages (ODD, a separate instantiation so that the
  // even case pays nothing for it) gets a repeat of the last one appended, which is loaded like any other (every
  // count the pipeline's waits rely on stays the same) and multiplied by nothing.
  const int nk_real = K / BK;
  constexpr bool odd = ODD;
  const int nk = nk_real + (odd ? 1 : 0);

  struct TileAt { int layer, tm, tn, m0, n0, om0, on0, rot; };
  auto locate = [&](int bid) {
    TileAt t;
    t.layer = bid / per_layer;
    bid -= t.layer * per_layer;
    if (by_tokens) {
      // The mirror image, for products whose token operand is the larger one (the dense decoder product
      // summed [T, F] x W[t] [d, F]: few feature tiles, many token tiles): XCD x owns the TOKEN tiles
      // m = x, x+8, ..., so the large operand is fetched by one XCD only and the small one by all.
      const int xcd = bid & 7, idx = bid >> 3, mloc = tiles_m >> 3;
      const int g = idx / (ENC_SN * tiles_n), r = idx - g * ENC_SN * tiles_n;
      const int cnt = (mloc - g * ENC_SN) < ENC_SN ? (mloc - g * ENC_SN) : ENC_SN;
      const int ng = r / (cnt * ENC_SM), r2 = r - ng * cnt * ENC_SM;
      t.tn = ng * ENC_SM + r2 / cnt;
      t.tm = (g * ENC_SN + r2 % cnt) * 8 + xcd;
    } else if ((tiles_n & 7) == 0) {
      // XCD x owns the feature tiles n = x, x+8, ...  Its tiles run in groups of ENC_SN feature tiles
      // x ENC_SM token tiles (about one tile per CU of the XCD): the group's W tiles stay in the L2
      // while the token groups sweep past, so W is fetched once and the x slab once per ENC_SN tiles.
      const int xcd = bid & 7, idx = bid >> 3, nloc = tiles_n >> 3;
      const int g = idx / (ENC_SN * tiles_m), r = idx - g * ENC_SN * tiles_m;
      const int cnt = (nloc - g * ENC_SN) < ENC_SN ? (nloc - g * ENC_SN) : ENC_SN;
      const int mg = r / (cnt * ENC_SM), r2 = r - mg * cnt * ENC_SM;
      t.tm = mg * ENC_SM + r2 / cnt;
      t.tn = (g * ENC_SN + r2 % cnt) * 8 + xcd;
    } else {
      t.tn = bid / tiles_m; t.tm = bid - t.tn * tiles_m;
    }
    t.m0 = t.tm * BM; t.n0 = t.tn * BN;
    t.om0 = t.m0; t.on0 = t.n0;       // what the tile owns: it stores nothing before these
    if (t.m0 + BM > M) t.m0 = M - BM;
    if (t.n0 + BN > N) t.n0 = N - BN;
    // K is walked from a tile-dependent starting stage, wrapping around: the CUs of an XCD that share an
    // x tile or a W tile then ask for different lines of it at any one time, so one of them takes the
    // L2 miss and the others find the line there later, instead of all of them queueing behind the miss.
    // (no rotation with an appended stage: that one must come last)
    t.rot = odd ? 0 : (by_tokens ? 3 * t.tn + (t.tm >> 3) : (tiles_n & 7) == 0 ? 3 * t.tm + (t.tn >> 3) : t.tm + t.tn) % nk;
    return t;
  };
  // the storing mode computes only the layers that asked for it when a gate is given; the states of up to
  // 64 layers are fetched with one load
  const int nlayer = total_tiles / per_layer;
  unsigned long long want_mask = ~0ull;
  if (COLLECT == 0 && gate && nlayer <= 64)
    want_mask = __ballot(lane < nlayer && gate[lane < nlayer ? lane : 0].status == ST_RETRY);
  auto wanted = [&](int bid) {
    if (COLLECT != 0 || !gate) return true;
    const int l = bid / per_layer;
    return nlayer <= 64 ? ((want_mask >> l) & 1ull) != 0ull : gate[l].status == ST_RETRY;
  };
  if (COLLECT == 0 && gate && nlayer <= 64 && want_mask == 0ull) return;
  int bid = blockIdx.x;
  while (bid < total_tiles && !wanted(bid)) bid += gridDim.x;
  if (bid >= total_tiles) return;

  // ---- loader: wave `wave` brings in rows [32*wave, 32*wave+32) of both tiles, 8 rows (1 KB)
  // per instruction.  Lane l lands at row l>>3, chunk position l&7 of its 8-row group and
  // therefore fetches global chunk (l&7) ^ ((row >> 1) & 7).
  const int lr = lane >> 3, lp = lane & 7;
  const int xrs = SEG ? sg.xrs : K, wrs = SEG ? sg.wrs : K;     // row strides
  const int chE = (lp ^ (lane >> 4)) * CE;                      // 8-row groups starting at a multiple of 16
  const int chO = (lp ^ ((lane >> 4) | 4)) * CE;                // ... at 8 mod 16
  const int offE = lr * xrs + chE, offO = lr * xrs + chO;
  const int woffE = SEG ? lr * wrs + chE : offE, woffO = SEG ? lr * wrs + chO : offO;
  auto x_rows = [&](const TileAt &t) { return x + (int64_t)t.layer * xs + (int64_t)(t.m0 + wave * 32) * xrs; };
  auto w_rows = [&](const TileAt &t) { return w + (int64_t)t.layer * wstr + (int64_t)(t.n0 + wave * 32) * wrs; };
  // the stage walked kt-th by a tile (an index into K / BK)
  auto stage_k0 = [&](const TileAt &t, int kt) {
    int q = kt + t.rot;
    if (q >= nk) q -= nk;
    if constexpr (ODD) return q < nk_real ? q : nk_real - 1;
    return q;
  };
  auto issue_stage = [&](unsigned char *stage, const T *xt, const T *wt, int kst) {
    unsigned char *xs_l = stage + wave * 32 * ROWB;
    unsigned char *ws_l = xs_l + BM * ROWB;
    int64_t xk = (int64_t)kst * BK, wk = xk;
    if constexpr (SEG) {
      const int q = sg.sps == 1 ? kst : (int)__umulhi((uint32_t)kst, sg.magic);
      const int kin = (kst - q * sg.sps) * BK;
      xk = q * sg.xss + kin;
      wk = q * sg.wss + kin;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      load16_to_lds(xt + (int64_t)t * 8 * xrs + xk + ((t & 1) ? offO : offE), xs_l + t * 8 * ROWB);
      load16_to_lds(wt + (int64_t)t * 8 * wrs + wk + ((t & 1) ? woffO : woffE), ws_l + t * 8 * ROWB);
    }
  };

  // ---- fragment reader: row l31 of each 32-row group; chunk (kk*2 + lh) at its swizzled position
  const int l31 = lane & 31, lh = lane >> 5;
  const int xrow = (wm * 64 + l31) * ROWB;              // + i * 32 * ROWB
  const int wrow = BM * ROWB + (wn * 128 + l31) * ROWB; // + j * 32 * ROWB
  int koff[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) koff[kk] = ((kk * 2 + lh) ^ ((l31 >> 1) & 7)) << 4;

  // The accumulators start from the bias (the matrix core adds its products onto them in fp32), so
  // the epilogue has no bias loads or adds: accumulator (j, rg*4+q) of a lane belongs to feature
  // j*32 + rg*8 + (lane>>5)*4 + q of the wave tile, whatever the token group i.  Each wavefront brings
  // the bias of its 128 features into LDS with one direct load ahead of the tile's stages - no register
  // holds it while the previous tile's epilogue runs - and reads it from there when the first stage has
  // landed.
  f32x16_t acc[2][4];
  constexpr int BIAS_LANES = 128 * (int)sizeof(T) / 16;   // lanes of the one 16-byte-per-lane load
  auto load_bias = [&](const TileAt &t) {
    if (bias && lane < BIAS_LANES)
      load16_to_lds(bias + (int64_t)t.layer * bs + t.n0 + wn * 128 + lane * CE, bias_lds[wave]);
    if constexpr (COLLECT == 2) {
      if (lane < BIAS_LANES)
        load16_to_lds((const T *)ca.theta + (int64_t)t.layer * ca.theta_stride + t.n0 + wn * 128 + lane * CE, theta_lds[wave]);
    }
    // the layer's cut travels the same way: four bytes into the wavefront's slot, read in the epilogue
    if constexpr (COLLECT == 1) {
      if (lane == 0)
        __builtin_amdgcn_global_load_lds(&ca.st[t.layer].cut_key, (__attribute__((address_space(3))) void *)cut_lds[wave], 4, 0, 0);
    }
  };
  if (!bias && lane < BIAS_LANES)   // no bias: the slot holds zeros for good
    *reinterpret_cast<uint4 *>(reinterpret_cast<unsigned char *>(bias_lds[wave]) + lane * 16) = make_uint4(0u, 0u, 0u, 0u);
  // The bias is read with hand-written LDS loads and a hand-placed wait: the compiler, which cannot tell how
  // many of the outstanding direct loads are older than the one into the bias slot, would otherwise wait for
  // all of them (the stage just asked for included) before the first read.
  const uint32_t bias_at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)
                               reinterpret_cast<unsigned char *>(bias_lds[wave]) + (uint32_t)(lane >> 5) * 4u * (uint32_t)sizeof(T);
  auto init_acc = [&]() {
    typedef typename std::conditional<sizeof(T) == 4, uint4, uint2>::type braw_t;
    braw_t raw[16];
    // raw[4 j + rg] = the 4 values at feature j * 32 + rg * 8 of this lane's half.  All sixteen reads and their
    // wait are one statement, so no register is looked at before its value has arrived.
    if constexpr (sizeof(T) == 4) {
        asm volatile(
                     "ds_read_b128 %0, %16\n\t"
                     "ds_read_b128 %1, %16 offset:32\n\t"
                     "ds_read_b128 %2, %16 offset:64\n\t"
                     "ds_read_b128 %3, %16 offset:96\n\t"
                     "ds_read_b128 %4, %16 offset:128\n\t"
                     "ds_read_b128 %5, %16 offset:160\n\t"
                     "ds_read_b128 %6, %16 offset:192\n\t"
                     "ds_read_b128 %7, %16 offset:224\n\t"
                     "ds_read_b128 %8, %16 offset:256\n\t"
                     "ds_read_b128 %9, %16 offset:288\n\t"
                     "ds_read_b128 %10, %16 offset:320\n\t"
                     "ds_read_b128 %11, %16 offset:352\n\t"
                     "ds_read_b128 %12, %16 offset:384\n\t"
                     "ds_read_b128 %13, %16 offset:416\n\t"
                     "ds_read_b128 %14, %16 offset:448\n\t"
                     "ds_read_b128 %15, %16 offset:480\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(raw[0]), "=&v"(raw[1]), "=&v"(raw[2]), "=&v"(raw[3]), "=&v"(raw[4]), "=&v"(raw[5]), "=&v"(raw[6]), "=&v"(raw[7]), "=&v"(raw[8]), "=&v"(raw[9]), "=&v"(raw[10]), "=&v"(raw[11]), "=&v"(raw[12]), "=&v"(raw[13]), "=&v"(raw[14]), "=&v"(raw[15])
                     : "v"(bias_at));
    } else {
        asm volatile(
                     "ds_read_b64 %0, %16\n\t"
                     "ds_read_b64 %1, %16 offset:16\n\t"
                     "ds_read_b64 %2, %16 offset:32\n\t"
                     "ds_read_b64 %3, %16 offset:48\n\t"
                     "ds_read_b64 %4, %16 offset:64\n\t"
                     "ds_read_b64 %5, %16 offset:80\n\t"
                     "ds_read_b64 %6, %16 offset:96\n\t"
                     "ds_read_b64 %7, %16 offset:112\n\t"
                     "ds_read_b64 %8, %16 offset:128\n\t"
                     "ds_read_b64 %9, %16 offset:144\n\t"
                     "ds_read_b64 %10, %16 offset:160\n\t"
                     "ds_read_b64 %11, %16 offset:176\n\t"
                     "ds_read_b64 %12, %16 offset:192\n\t"
                     "ds_read_b64 %13, %16 offset:208\n\t"
                     "ds_read_b64 %14, %16 offset:224\n\t"
                     "ds_read_b64 %15, %16 offset:240\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(raw[0]), "=&v"(raw[1]), "=&v"(raw[2]), "=&v"(raw[3]), "=&v"(raw[4]), "=&v"(raw[5]), "=&v"(raw[6]), "=&v"(raw[7]), "=&v"(raw[8]), "=&v"(raw[9]), "=&v"(raw[10]), "=&v"(raw[11]), "=&v"(raw[12]), "=&v"(raw[13]), "=&v"(raw[14]), "=&v"(raw[15])
                     : "v"(bias_at));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        float bv[4];
        if constexpr (sizeof(T) == 4) {
          const uint4 r = raw[j * 4 + rg];
          bv[0] = __uint_as_float(r.x); bv[1] = __uint_as_float(r.y); bv[2] = __uint_as_float(r.z); bv[3] = __uint_as_float(r.w);
        } else {
          const uint2 r = raw[j * 4 + rg];
          unpack_pair<T>(r.x, bv[0], bv[1]);
          unpack_pair<T>(r.y, bv[2], bv[3]);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[i][j][rg * 4 + q] = bv[q];
      }
  };

  // Software pipeline over the K stages.  Fragments are double-buffered in registers (fa/fb)
  // and read one k-step ahead of the matrix ops that use them.  There is one barrier per
  // stage, placed before the LAST k-step of a stage: at that point this wavefront's loads of
  // the next stage have landed and its LDS reads of the current stage are complete, so after
  // the barrier the next stage may be read (its first fragments are fetched under the last
  // k-step's matrix ops) and the current one may be overwritten by the stage after next.
  uint4 fa[6], fb[6];   // [0..1] x fragments, [2..5] W fragments
  auto load_frags = [&](uint4 (&f)[6], const unsigned char *sb, int kk) {
    // in the order the matrix ops of the next k-step want them: x0 and all of W first
    f[0] = *reinterpret_cast<const uint4 *>(sb + xrow + koff[kk]);
#pragma unroll
    for (int j = 0; j < 4; ++j) f[2 + j] = *reinterpret_cast<const uint4 *>(sb + wrow + j * 32 * ROWB + koff[kk]);
    f[1] = *reinterpret_cast<const uint4 *>(sb + xrow + 32 * ROWB + koff[kk]);
  };
  auto mma8 = [&](const uint4 (&f)[6]) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) Mma<T>::run(acc[i][j], f[2 + j], f[i]);
  };
  constexpr int MPI = sizeof(T) == 2 ? 1 : 4;   // matrix instructions per Mma::run
  // interleave hint: the six LDS reads go out behind the first matrix ops of the k-step, one apiece
  auto mix_ds = [&]() {
#pragma unroll
    for (int g = 0; g < 6; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPI, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 2 * MPI, 0);
  };
  // one stage except its last k-step, the barrier, then the last k-step overlapped with the loads that
  // `refill` asks for (the stage after next, into `cur`) and, unless this is the tile's last stage,
  // the first fragments of `nxt`
  // `cm` / `nm`: AND masks for the fragments read from `cur` / `nxt` (all ones, or zero for the appended stage,
  // whose products must add nothing: both operands are cleared, so that an infinity in the repeated data cannot
  // turn into a NaN)
  auto mask_frags = [&](uint4 (&f)[6], uint32_t m) {
#pragma unroll
    for (int i = 0; i < 6; ++i) { f[i].x &= m; f[i].y &= m; f[i].z &= m; f[i].w &= m; }
  };
  auto body = [&](unsigned char *cur, unsigned char *nxt, bool last, auto refill, uint32_t cm, uint32_t nm) {
    load_frags(fb, cur, 1); mask_frags(fb, cm); mma8(fa); mix_ds();
    load_frags(fa, cur, 2); mask_frags(fa, cm); mma8(fb); mix_ds();
    load_frags(fb, cur, 3); mask_frags(fb, cm); mma8(fa); mix_ds();
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    refill();
    if (!last) { load_frags(fa, nxt, 0); mask_frags(fa, nm); }
    mma8(fb);
#pragma unroll
    for (int g = 0; g < 8; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPI, 0);
      if (g < 6) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
  };

  TileAt cur = locate(bid);
  // both stage buffers are free at this point: the bias, then the first stage, then the second
  load_bias(cur);
  __builtin_amdgcn_sched_barrier(0);
  issue_stage(stage0, x_rows(cur), w_rows(cur), stage_k0(cur, 0));
  issue_stage(stage1, x_rows(cur), w_rows(cur), stage_k0(cur, 1));

  for (;;) {
    int nbid = bid + (int)gridDim.x;
    while (nbid < total_tiles && !wanted(nbid)) nbid += gridDim.x;
    const bool has_next = nbid < total_tiles;
    const TileAt nxt_tile = locate(has_next ? nbid : bid);
    const T *xt = x_rows(cur), *wt = w_rows(cur);
    const int m0 = cur.m0, n0 = cur.n0, layer = cur.layer;

    // only the first stage (this wavefront's 8 older loads, and the bias load before them) is waited for:
    // at most the 8 loads of the second stage stay outstanding
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F78);   // vmcnt(8)
    // a bare barrier between two compiler-only fences: the fences of __syncthreads() would wait for the
    // second stage too
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);    // nothing that reads the bias may move above the wait
    init_acc();
    load_frags(fa, stage0, 0);
    // nk is even
    for (int kt = 0; kt < nk - 2; kt += 2) {
      body(stage0, stage1, false, [&]() { issue_stage(stage0, xt, wt, stage_k0(cur, kt + 2)); }, ~0u, ~0u);
      body(stage1, stage0, false, [&]() { issue_stage(stage1, xt, wt, stage_k0(cur, kt + 3)); }, ~0u, ~0u);
    }
    // the last two stages: the first buffer is free after the first of them and takes the next tile's
    // first stage; nothing may be in flight into the second one, which is parked in
    constexpr uint32_t last_mask = odd ? 0u : ~0u;
    body(stage0, stage1, false, [&]() {
      if (has_next) issue_stage(stage0, x_rows(nxt_tile), w_rows(nxt_tile), stage_k0(nxt_tile, 0));
    }, ~0u, last_mask);
    body(stage1, stage0, true, [&]() {}, last_mask, ~0u);
    // past the barrier of the last stage no wavefront reads either buffer any more

    // ---- epilogue.  The accumulator layout gives a lane 4 consecutive features of one token,
    // i.e. 8-byte pieces scattered over 32 rows per store - slow to write.  Each wavefront
    // therefore parks its tile in LDS, 32 tokens at a time (8 KB; two passes of 64 features for fp32) in its
    // eighth of the second stage buffer, and works on it row by row from there.
    T *pl = pre + (int64_t)layer * ps;
    // The epilogue's addresses are rebuilt from the lane number for every tile.  Left visible as loop
    // invariants they would be computed once ahead of the tile loop and live across the K loop.
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int l31 = lane_e & 31, lh = lane_e >> 5;
    unsigned char *park = stage1 + wave * (STAGE / 8);
    constexpr int NPASS = sizeof(T) == 2 ? 1 : 2;           // feature halves per pass
    constexpr int JP = 4 / NPASS;                            // 32-feature groups per pass
    // token groups [i0, i0 + ni) of feature pass `pass` -> rows (i - i0) * 32 + l31 of 256 bytes
    // (128 bf16 / 64 fp32), 16-byte slots XOR-swizzled with the row
    auto park_rows = [&](int pass, int i0, int ni) {
#pragma unroll
      for (int jj = 0; jj < JP; ++jj) {
        const int j = pass * JP + jj;
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const int nl = jj * 32 + rg * 8 + lh * 4;          // feature inside this pass
#pragma unroll
          for (int ii = 0; ii < ni; ++ii) {
            const int i = i0 + ii;
            const int ml = ii * 32 + l31;                    // row inside the parked piece
            float y[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) y[q] = acc[i][j][rg * 4 + q];
            if (sizeof(T) == 4) {
              const int slot = (nl >> 2) ^ (ml & 15);
              *reinterpret_cast<float4 *>(park + ml * 256 + slot * 16) = make_float4(y[0], y[1], y[2], y[3]);
            } else {
              const int slot = (nl >> 3) ^ (ml & 15);
              uint2 o;
              o.x = pack16x2<T>(y[0], y[1]);
              o.y = pack16x2<T>(y[2], y[3]);
              *reinterpret_cast<uint2 *>(park + ml * 256 + slot * 16 + (nl & 4) * 2) = o;
            }
          }
        }
      }
    };
    constexpr int EPS = 16 / (int)sizeof(T);               // elements per 16-byte slot
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
      if constexpr (COLLECT == 0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
        park_rows(pass, h, 1);
        // the wavefront reads its own piece back: lane -> (row = it*4 + lane/16, slot = lane%16)
#pragma unroll 4
        for (int it = 0; it < 8; ++it) {
          const int ml = it * 4 + (lane_e >> 4), sl = lane_e & 15;
          const uint4 v = *reinterpret_cast<const uint4 *>(park + ml * 256 + ((sl ^ (ml & 15)) * 16));
          const int m = m0 + wm * 64 + h * 32 + ml;
          const int n = n0 + wn * 128 + pass * (128 / NPASS) + sl * EPS;
          // the part of a shifted tile that its neighbour owns is left to the neighbour: the two walk K
          // from different stages, so their sums may differ in the last bit
          // (N is a multiple of 4, so a 16-byte piece of bf16 may straddle the line by half)
          if (m >= cur.om0) {
            if (n >= cur.on0) *reinterpret_cast<uint4 *>(pl + (int64_t)m * N + n) = v;
            else if (sizeof(T) == 2 && n + 4 >= cur.on0) *reinterpret_cast<uint2 *>(pl + (int64_t)m * N + n + 4) = make_uint2(v.z, v.w);
          }
        }
        }
      } else {
        // Two lanes per token row of the parked piece: lane -> row lane % 32, slots [8 hs, 8 hs + 8) with
        // hs = lane / 32.  Counting and ordering inside a half row need no cross-lane work; the two halves
        // of a row meet through one lane exchange.
        constexpr int KB = Elem<T>::KEYBITS;
        constexpr int SEGW = 128 / NPASS;                    // features per segment (16 slots)
        constexpr int NWL = SEGW / 64;                       // 32-bit mask words per lane (half a row)
        const int ncol0 = n0 + wn * 128 + pass * SEGW;       // first feature of the segment
        uint32_t cut_bits = 0;
        if constexpr (COLLECT == 1) {
          // The cut came in with the bias, ahead of the tile's stages, and has long landed.  Read by hand, with
          // its own wait inside the statement: the compiler, which cannot tell the direct-to-LDS loads in flight
          // (the next tile's first stage) from the one into this slot, would wait for all of them first.
          uint32_t cut_key_v;
          const uint32_t cut_at = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t *)cut_lds[wave];
          asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(cut_key_v) : "v"(cut_at) : "memory");
          cut_bits = key_value_bits<T>((uint32_t)__builtin_amdgcn_readfirstlane((int)cut_key_v));
        }
        const bool cut_nan = (cut_bits & 0x7FFFFFFFu) > 0x7F800000u;   // only NaNs reach such a cut
        const float cutf = __uint_as_float(cut_bits);
        const int hs = lh, rsw = l31 & 15;
        const unsigned char *myrow = park + l31 * 256;
        uint32_t W[2][NWL];
        uint32_t cnt[2], part[2], incl[2], tot[2];           // own half row, the other half, rows up to this one
        // generic: float compares, element by element; bit c of a lane's mask = column 64 hs + c
        auto scan_generic = [&](uint32_t (&Wh)[NWL]) {
#pragma unroll
          for (int i = 0; i < NWL; ++i) Wh[i] = 0;
#pragma unroll
          for (int s8 = 0; s8 < 8; ++s8) {
            const int sl = hs * 8 + s8;
            const uint4 v = *reinterpret_cast<const uint4 *>(myrow + ((sl ^ rsw) * 16));
            uint4 tv = make_uint4(0, 0, 0, 0);
            if constexpr (COLLECT == 2)
              tv = *reinterpret_cast<const uint4 *>(theta_lds[wave] + pass * SEGW + sl * EPS);
            uint32_t m = 0;
#pragma unroll
            for (int j = 0; j < EPS; ++j) {
              const float xv = slot_elem<T>(v, j);
              bool c;
              if constexpr (COLLECT == 1) c = cut_nan ? (xv != xv) : !(xv < cutf);
              else c = xv >= slot_elem<T>(tv, j);
              m |= (c ? 1u : 0u) << j;
            }
            Wh[(s8 * EPS) >> 5] |= m << ((s8 * EPS) & 31);
          }
        };
        // bf16 and a positive cut / threshold: x >= c  <=>  bits(x) >= bits(c) as signed 16-bit
        // integers (negative values have the sign bit), two elements per operation: the sign of
        // the saturated difference (c - 1) - x marks a candidate.  NaNs would be treated wrongly
        // (a top-k cut must take them all, also those with the sign bit set; a threshold must take
        // none), so the unsigned maximum of the raw values is tracked and the piece is redone with
        // float compares if it shows one.
        bool fast_ok = false;
        uint32_t cm1 = 0;
        const T *theta_seg = nullptr;
        if constexpr (sizeof(T) == 2) {
          if constexpr (COLLECT == 1) {
            const uint32_t cb = Elem<T>::raw(Elem<T>::from_f32(cutf));   // the cut is a value of T
            fast_ok = cb >= 1u && cb <= Elem<T>::INF16;
            cm1 = (cb - 1u) | ((cb - 1u) << 16);
          } else {
            theta_seg = theta_lds[wave] + pass * SEGW;
            bool bad = false;
            if (lane_e < 16) {   // every threshold of the segment must be a positive number
              const uint4 tv = *reinterpret_cast<const uint4 *>(theta_seg + lane_e * 8);
              const uint32_t t4[4] = {tv.x, tv.y, tv.z, tv.w};
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                const uint32_t lo = t4[k] & 0xFFFFu, hi = t4[k] >> 16;
                bad = bad || lo < 1u || lo > Elem<T>::INF16 || hi < 1u || hi > Elem<T>::INF16;
              }
            }
            fast_ok = __ballot(bad) == 0;
          }
        }
        auto scan_piece = [&](uint32_t (&Wh)[NWL]) {
          bool done = false;
          if constexpr (sizeof(T) == 2) {
            if (fast_ok) {
              uint32_t mx = 0;
#pragma unroll
              for (int i = 0; i < NWL; ++i) Wh[i] = 0;
#pragma unroll
              for (int s8 = 0; s8 < 8; ++s8) {
                const int sl = hs * 8 + s8;
                const uint4 v = *reinterpret_cast<const uint4 *>(myrow + ((sl ^ rsw) * 16));
                const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
                uint32_t c4[4] = {cm1, cm1, cm1, cm1};
                if constexpr (COLLECT == 2) {
                  const uint4 tv = *reinterpret_cast<const uint4 *>(theta_seg + sl * 8);   // one address per half wave
                  c4[0] = tv.x - 0x00010001u; c4[1] = tv.y - 0x00010001u; c4[2] = tv.z - 0x00010001u; c4[3] = tv.w - 0x00010001u;
                }
                uint32_t a = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                  const uint32_t sg = pk_sign16(pk_sub_sat16(c4[k], w4[k]));   // 0xFFFF per candidate half
                  a |= sg & ((1u << (2 * k)) | (0x20000u << (2 * k)));         // element 2k -> bit 2k, 2k+1 -> bit 16+2k+1
                  mx = pk_max_u16(mx, COLLECT == 1 ? w4[k] : (w4[k] & 0x7FFF7FFFu));
                }
                const uint32_t m = (a | (a >> 16)) & 0xFFu;
                Wh[s8 >> 2] |= m << ((s8 & 3) * 8);
              }
              const uint32_t nan_above = COLLECT == 1 ? (0x8000u | Elem<T>::INF16) : Elem<T>::INF16;
              const bool nan_seen = (mx & 0xFFFFu) > nan_above || (mx >> 16) > nan_above;
              done = __ballot(nan_seen) == 0;
            }
          }
          if (!done) scan_generic(Wh);
        };
        uint2 *mypool = ca.pool + (unsigned long long)layer * ca.pool_cap;
        // Emission of the parked piece: `n` candidates, this lane's starting at position `first` of
        // the piece, to dst[0 .. n).  Each lane first drops a 16-bit code (row, column) for every
        // candidate of its half row into the wavefront's list, at the candidate's ordered position; then
        // the lanes take one candidate each: 64 consecutive pool entries per store instruction, and the
        // number of rounds is the piece's count / 64 instead of the fullest row's count.
        auto emit_piece = [&](const uint32_t (&Wh)[NWL], uint32_t first, uint32_t n, uint2 *dst) {
          if (n <= (uint32_t)CAND_LIST) {
            uint16_t *lst = cand_list[wave];
            const uint32_t rowcode = ((uint32_t)l31 << 8) | (uint32_t)(hs * (SEGW / 2));
            uint32_t p = first;
#pragma unroll
            for (int i = 0; i < NWL; ++i) {
              uint32_t wd = Wh[i];
              while (wd) {
                lst[p++] = (uint16_t)(rowcode + (uint32_t)(i * 32 + (__ffs(wd) - 1)));
                wd &= wd - 1u;
              }
            }
#pragma unroll 2
            for (uint32_t idx = lane_e; idx < n; idx += 64) {
              const uint32_t code = lst[idx];
              const int ml = (int)(code >> 8), c = (int)(code & 255u);
              const int sl = c / EPS, j = c % EPS;
              const T rawv = *reinterpret_cast<const T *>(park + ml * 256 + ((sl ^ (ml & 15)) * 16) + j * (int)sizeof(T));
              dst[idx] = make_uint2((uint32_t)(ncol0 + c), Elem<T>::raw(rawv));
            }
          } else {
            // more candidates than the list holds: every lane walks its own half row
            uint32_t pos = first;
#pragma unroll
            for (int i = 0; i < NWL; ++i) {
              uint32_t wd = Wh[i];
              while (wd) {
                const int c = hs * (SEGW / 2) + i * 32 + (__ffs(wd) - 1);   // column inside the segment
                wd &= wd - 1u;
                const int sl = c / EPS, j = c % EPS;
                const T rawv = *reinterpret_cast<const T *>(myrow + ((sl ^ rsw) * 16) + j * (int)sizeof(T));
                dst[pos++] = make_uint2((uint32_t)(ncol0 + c), Elem<T>::raw(rawv));
              }
            }
          }
        };
        // the books are kept on the grid of whole tiles, in both directions: this wave tile's rows start at grid
        // row om0 + 64 wm, its segment is the one at feature on0 + 128 wn (+ the pass's half) of the grid
        const int nseg = tiles_n * BN / SEGW;
        const int seg = (cur.on0 + wn * 128 + pass * SEGW) / SEGW;
        const int Mp = tiles_m * BM, grow0 = cur.om0 + wm * 64;
        const int nrb = Mp / COLLECT_ROWS, rowblk = grow0 / COLLECT_ROWS;
        const int shift = cur.om0 - m0;                      // > 0: the tile was shifted back inside the matrix
        const int cshift = cur.on0 - ncol0;                  // > 0: the segment's first cshift features are the neighbour's
        const uint32_t tile = (uint32_t)seg * (uint32_t)nrb + (uint32_t)rowblk;
        uint32_t off = tile * ca.caps;                       // the tile's fixed slot
        // Each piece of 32 tokens is emitted into the fixed slot as soon as it is scanned, while it is
        // parked; the rare tile whose two pieces do not fit the slot takes an extent behind the slots (one
        // atomic) and parks and emits both again.
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          park_rows(pass, h, 1);
          scan_piece(W[h]);
          // the first `shift` tokens of a shifted tile belong to its neighbour, which reports them, and so do the
          // features in front of on0 (bit b of word i of a lane = feature hs * SEGW / 2 + 32 i + b of the segment)
          if (shift > 0 && wm * 64 + h * 32 + l31 < shift) {
#pragma unroll
            for (int i = 0; i < NWL; ++i) W[h][i] = 0;
          }
          if (cshift > 0) {
#pragma unroll
            for (int i = 0; i < NWL; ++i) {
              const int low = cshift - hs * (SEGW / 2) - i * 32;     // bits below `low` go
              W[h][i] &= low <= 0 ? ~0u : low >= 32 ? 0u : ~0u << low;
            }
          }
          cnt[h] = 0;
#pragma unroll
          for (int i = 0; i < NWL; ++i) cnt[h] += __popc(W[h][i]);
          part[h] = (uint32_t)__shfl_xor((int)cnt[h], 32);
          // rows up to and including this one, inside each half of the wavefront
          uint32_t v = row16_inclusive_scan(cnt[h] + part[h]);
          v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);  // row_bcast:15
          incl[h] = v;
          tot[h] = __builtin_amdgcn_readlane(v, 31);
          const uint32_t before = h ? tot[0] : 0u;
          const uint32_t first = incl[h] - cnt[h] - (hs ? 0u : part[h]);
          if (before + tot[h] <= ca.caps) emit_piece(W[h], first, tot[h], mypool + off + before);
        }
        const uint32_t total = tot[0] + tot[1];
        bool ok = true;
        if (total > ca.caps) {
          const unsigned long long fixed = (unsigned long long)nseg * nrb * ca.caps;
          uint32_t a = 0;
          if (lane_e == 0) a = atomicAdd(&ca.pool_count[layer], total);
          a = __builtin_amdgcn_readfirstlane(a);
          ok = fixed + a + total <= ca.pool_cap;
          off = (uint32_t)(fixed + a);
          if (!ok && lane_e == 0) atomicOr(&ca.st[layer].overflow, 1u);
          if (ok) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              park_rows(pass, h, 1);
              emit_piece(W[h], incl[h] - cnt[h] - (hs ? 0u : part[h]), tot[h], mypool + off + (h ? tot[0] : 0u));
            }
          }
        }
        if (lane_e == 0) ca.tile_meta[(int64_t)layer * nseg * nrb + tile] = make_uint2(off, ok ? total : 0u);
        uint2 *meta = ca.seg_meta + ((int64_t)layer * nseg + seg) * Mp + grow0;
        if (hs == 0) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const uint32_t rowtot = cnt[h] + part[h];
            const uint32_t rel = (h ? tot[0] : 0u) + incl[h] - rowtot;
            meta[h * 32 + l31] = ok ? make_uint2(off + rel, rowtot) : make_uint2(0u, 0u);
          }
        }
      }
    }
    if (!has_next) break;
    // Every wavefront is done with its parked rows before the next tile's loads overwrite them.  The wait
    // covers the epilogue's stores as well (and the next tile's first stage, long since landed): with only
    // loads outstanding afterwards, the counted wait at the top of the tile is exact.
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    bid = nbid;
    cur = nxt_tile;
    load_bias(cur);
    __builtin_amdgcn_sched_barrier(0);   // the bias stays ahead of the stage loads: the wait above counts on it
    issue_stage(stage1, x_rows(cur), w_rows(cur), stage_k0(cur, 1));
  }
  __builtin_amdgcn_s_waitcnt(0);   // no direct-to-LDS load may be in flight when the block retires
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
static bool encode_fast_ok(const void *x, const void *w, const void *b, const void *pre, int64_t T_, int64_t d,
                           int64_t F, int64_t xs, int64_t wstr, int64_t bs, int64_t ps) {
  constexpr int CE = 16 / (int)sizeof(T);
  return (d % (ROWB / (int)sizeof(T)) == 0) && (F % 4 == 0) && T_ >= BM && F >= BN && clt_aligned16(x) &&
         clt_aligned16(w) && clt_aligned16(pre) && (xs % CE == 0) && (wstr % CE == 0) && (ps % 4 == 0) &&
         (ps * (int64_t)sizeof(T)) % 16 == 0 && (F * (int64_t)sizeof(T)) % 8 == 0 && T_ < (1 << 30) &&
         F < (1 << 30) && d < (1 << 30) && (!b || (((uintptr_t)b) % 16 == 0 && bs % 8 == 0));
}

// One persistent workgroup per CU (a whole number of rounds over the 8 XCDs, so that block b stays on XCD
// b % 8 for all of its tiles), or one per tile when there are fewer tiles; 0 when the device cannot be asked.
static int64_t persistent_grid(int64_t tiles) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8)
    return 0;
  cus -= cus % 8;
  return tiles < cus ? tiles : cus;
}

template <typename T>
static int launch_encode(const void *x, const void *w, const void *b, void *pre, int64_t T_, int64_t d, int64_t F,
                         int64_t L, int64_t xs, int64_t wstr, int64_t bs, int64_t ps, int collect,
                         const SelState *gate, const CollectArgs *ca, hipStream_t stream) {
  const bool fast = encode_fast_ok<T>(x, w, b, collect ? nullptr : pre, T_, d, F, xs, wstr, bs, collect ? 16 : ps);
  if (collect && !fast) return CLT_ERR_ARG;
  if (fast) {
    const int64_t tm = clt_ceil_div(T_, BM), tn = clt_ceil_div(F, BN);
    const int64_t nblk = tm * tn * L;
    if (nblk > 2147483647LL) return CLT_ERR_RANGE;
    CollectArgs none = {};
    const CollectArgs a = ca ? *ca : none;
    const int64_t grid = persistent_grid(nblk);
    if (grid <= 0) return CLT_ERR_LAUNCH;
    const SegArgs noseg = {};
    // which operand an XCD keeps to itself: the feature tiles (W, the larger one in the encoder), or the token
    // tiles when there are more of those and they split evenly over the XCDs
    const int by_tokens = (tm % 8 == 0 && tm > tn) ? 1 : 0;
#define CLT_ENC(C, O)                                                                                               \
  k_encode_mfma<T, C, false, O><<<(unsigned)grid, NTHREADS, 0, stream>>>((const T *)x, (const T *)w, (const T *)b,  \
                                                                     (T *)pre, (int)T_, (int)d, (int)F, (int)tm,  \
                                                                     (int)tn, (int)nblk, xs, wstr, bs, ps, gate,  \
                                                                     a, noseg, by_tokens)
    const bool odd_stages = ((d / (ROWB / (int64_t)sizeof(T))) & 1) != 0;
    if (odd_stages) {
      if (collect == 0) CLT_ENC(0, true);
      else if (collect == 1) CLT_ENC(1, true);
      else CLT_ENC(2, true);
    } else {
      if (collect == 0) CLT_ENC(0, false);
      else if (collect == 1) CLT_ENC(1, false);
      else CLT_ENC(2, false);
    }
#undef CLT_ENC
  } else {
    // the gate is ignored here: recomputing a layer that did not ask for it is harmless
    k_encode_generic<T><<<256 * 8, 256, 0, stream>>>((const T *)x, (const T *)w, (const T *)b, (T *)pre, T_, d, F, L,
                                                     xs, wstr, bs, ps);
  }
  return clt_check_launch();
}

// pre[T][F] = sum over segments q of x_q[T][dseg] . w_q[F][dseg]^T on the matrix-core kernel
template <typename T>
static int launch_encode_segmented(const void *x, const void *w, void *pre, int64_t T_, int64_t dseg, int64_t nseg,
                                   int64_t F, int64_t xss, int64_t xrs, int64_t wss, int64_t wrs, hipStream_t stream) {
  constexpr int CE = 16 / (int)sizeof(T);
  constexpr int BK = ROWB / (int)sizeof(T);
  const int64_t K = dseg * nseg;
  const bool ok = dseg % BK == 0 && (K / BK) % 2 == 0 && K / BK < 65536 && T_ >= BM && F >= BN && F % 4 == 0 &&
                  clt_aligned16(x) && clt_aligned16(w) && clt_aligned16(pre) && xss % CE == 0 && wss % CE == 0 &&
                  xrs % CE == 0 && wrs % CE == 0 && xrs < (1 << 24) && wrs < (1 << 24) && T_ < (1 << 30) &&
                  F < (1 << 30) && (F * (int64_t)sizeof(T)) % 8 == 0;
  if (!ok) return CLT_ERR_ARG;
  const int64_t tm = clt_ceil_div(T_, BM), tn = clt_ceil_div(F, BN), nblk = tm * tn;
  if (nblk > 2147483647LL) return CLT_ERR_RANGE;
  SegArgs sg;
  sg.sps = (int)(dseg / BK);
  sg.magic = (uint32_t)((0x100000000ull + (uint64_t)sg.sps - 1ull) / (uint64_t)sg.sps);
  sg.xss = xss; sg.wss = wss; sg.xrs = (int)xrs; sg.wrs = (int)wrs;
  const CollectArgs none = {};
  const int64_t grid = persistent_grid(nblk);
  if (grid <= 0) return CLT_ERR_LAUNCH;
  k_encode_mfma<T, 0, true, false><<<(unsigned)grid, NTHREADS, 0, stream>>>((const T *)x, (const T *)w, nullptr, (T *)pre, (int)T_,
                                                                    (int)K, (int)F, (int)tm, (int)tn, (int)nblk, 0, 0, 0,
                                                                    0, nullptr, none, sg, (tm % 8 == 0 && tm > tn) ? 1 : 0);
  return clt_check_launch();
}

}  // namespace

extern "C" int clt_encode_segmented(const void *x, const void *w, void *pre, int64_t T, int64_t d_seg, int64_t n_seg,
                                    int64_t F, int64_t x_seg_stride, int64_t x_row_stride, int64_t w_seg_stride,
                                    int64_t w_row_stride, int dtype, void *stream) {
  if (dtype != CLT_F32 && dtype != CLT_BF16) return CLT_ERR_DTYPE;
  if (T < 0 || d_seg <= 0 || n_seg <= 0 || F <= 0 || x_row_stride < d_seg || w_row_stride < d_seg || x_seg_stride < 0 ||
      w_seg_stride < 0)
    return CLT_ERR_ARG;
  if (T == 0) return CLT_OK;
  if (!x || !w || !pre) return CLT_ERR_ARG;
  if (dtype == CLT_BF16)
    return launch_encode_segmented<bf16_t>(x, w, pre, T, d_seg, n_seg, F, x_seg_stride, x_row_stride, w_seg_stride,
                                           w_row_stride, (hipStream_t)stream);
  return launch_encode_segmented<float>(x, w, pre, T, d_seg, n_seg, F, x_seg_stride, x_row_stride, w_seg_stride,
                                        w_row_stride, (hipStream_t)stream);
}

int clt_launch_encode(const void *x, const void *w, const void *b, void *pre, int64_t T, int64_t d, int64_t F,
                      int64_t L, int64_t xs, int64_t wstr, int64_t bs, int64_t ps, int dtype, int collect,
                      const SelState *gate, const CollectArgs *ca, hipStream_t stream) {
  if (dtype == CLT_BF16) return launch_encode<bf16_t>(x, w, b, pre, T, d, F, L, xs, wstr, bs, ps, collect, gate, ca, stream);
  if (dtype == CLT_F16) return launch_encode<f16_t>(x, w, b, pre, T, d, F, L, xs, wstr, bs, ps, collect, gate, ca, stream);
  return launch_encode<float>(x, w, b, pre, T, d, F, L, xs, wstr, bs, ps, collect, gate, ca, stream);
}

bool clt_encode_can_collect(const void *x, const void *w, const void *b, int64_t T, int64_t d, int64_t F,
                            int64_t xs, int64_t wstr, int64_t bs, int dtype) {
  const bool fast = dtype != CLT_F32 ? encode_fast_ok<bf16_t>(x, w, b, nullptr, T, d, F, xs, wstr, bs, 16)   // any 16-bit type
                                     : encode_fast_ok<float>(x, w, b, nullptr, T, d, F, xs, wstr, bs, 16);
  return fast;
}

extern "C" int clt_encode_fast_path(const void *x, const void *w, const void *b, const void *pre, int64_t T, int64_t d,
                                    int64_t F, int64_t L, int64_t x_layer_stride, int64_t w_layer_stride,
                                    int64_t b_layer_stride, int64_t pre_layer_stride, int dtype) {
  if (!clt_model_dtype(dtype) || T <= 0 || d <= 0 || F <= 0 || L <= 0 || !x || !w || !pre) return 0;
  if (clt_ceil_div(T, BM) * clt_ceil_div(F, BN) * L > 2147483647LL) return 0;
  const bool fast = dtype != CLT_F32
                        ? encode_fast_ok<bf16_t>(x, w, b, pre, T, d, F, x_layer_stride, w_layer_stride, b_layer_stride, pre_layer_stride)
                        : encode_fast_ok<float>(x, w, b, pre, T, d, F, x_layer_stride, w_layer_stride, b_layer_stride, pre_layer_stride);
  return fast ? 1 : 0;
}

extern "C" int clt_encode(const void *x, const void *w, const void *b, void *pre, int64_t T, int64_t d, int64_t F,
                          int64_t L, int64_t x_layer_stride, int64_t w_layer_stride, int64_t b_layer_stride,
                          int64_t pre_layer_stride, int dtype, void *stream) {
  if (!clt_model_dtype(dtype)) return CLT_ERR_DTYPE;
  if (T < 0 || d <= 0 || F <= 0 || L <= 0) return CLT_ERR_ARG;
  if (T == 0) return CLT_OK;
  if (!x || !w || !pre) return CLT_ERR_ARG;
  return clt_launch_encode(x, w, b, pre, T, d, F, L, x_layer_stride, w_layer_stride, b_layer_stride,
                           pre_layer_stride, dtype, 0, nullptr, nullptr, (hipStream_t)stream);
}

