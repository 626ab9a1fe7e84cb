// State shared between the selection kernels (select.hip) and the encoder kernel that collects
// candidates in its epilogue (encode.hip).
#pragma once
#include "clt_common.h"

enum : uint32_t { ST_RUN = 0, ST_RETRY = 1, ST_DONE = 2 };

// where the candidates of a problem live
enum : uint32_t {
  PATH_ROWS = 0,   // per-row chains of extents written by the streaming pass
  PATH_TILES = 1,  // per-(row, feature segment) runs written by the encoder epilogue
};

struct SelState {
  uint32_t cut_key;   // candidates have key >= cut_key
  uint32_t status;    // ST_*
  uint32_t level;     // level whose histogram is being accumulated
  uint32_t flo, fhi;  // levels >= 1: inclusive range of (key - cut_key) still in play
  uint32_t bbase;     // levels >= 1: bin = (diff - bbase) >> shift
  uint32_t shift;
  uint32_t thr_key;   // result: key of the K-th largest element
  unsigned long long k_rem;       // still to take from the active range
  unsigned long long tie_budget;  // result: how many elements equal to thr_key survive
  uint32_t path;      // PATH_*
  uint32_t overflow;  // the encoder epilogue ran out of pool space (set with atomicOr)
};

// tokens of one wave tile of the collecting encoder epilogue
constexpr int COLLECT_ROWS = 64;
// tokens of one workgroup tile of the encoder kernel
constexpr int COLLECT_TILE_ROWS = 256;

// The collecting epilogue keeps its books on a grid of whole workgroup tiles: Tp = T rounded up to a multiple
// of COLLECT_TILE_ROWS token rows.  When T is not such a multiple the last token tile is shifted back inside
// the matrix (it covers the tokens [T - 256, T)), reports only the tokens its neighbour does not own, and
// files them where it computed them: token t of the last tile sits at row t + (Tp - T) of the grid, the
// Tp - T rows in front of them are empty.
__host__ __device__ inline int64_t collect_grid_rows(int64_t T) {
  return (T + COLLECT_TILE_ROWS - 1) / COLLECT_TILE_ROWS * COLLECT_TILE_ROWS;
}
__device__ __forceinline__ int64_t collect_grid_row(int64_t token, int64_t T, int64_t Tp) {
  return token + (token >= Tp - COLLECT_TILE_ROWS ? Tp - T : 0);
}

// What the collecting encoder epilogue writes.  A wavefront's 64-token tile of one feature
// segment (128 features for 16-bit elements, 64 for 32-bit) becomes ONE extent of the layer's
// pool, ordered by (token, feature).  Tile number i = segment * (Tp / 64) + token block owns
// the fixed slot [i * caps, (i + 1) * caps) of the pool; only a tile with more than `caps`
// candidates takes an extent behind the slots instead, handed out by an atomic counter (one
// same-address atomic per tile from every CU at once would cost more than the whole epilogue).
//   tile_meta[layer * ntile + i]                           = (offset of the extent, entries)
//   seg_meta[(layer * nseg + segment) * Tp + grid row]     = (offset of the token's run, length)
struct CollectArgs {
  SelState *st;              // [L]
  uint32_t *pool_count;      // [L] entries handed out behind the fixed slots
  uint2 *pool;               // [L][pool_cap] entries (feature, raw value bits)
  unsigned long long pool_cap;
  uint2 *tile_meta;          // [L][ntile]
  uint2 *seg_meta;           // [L][nseg][Tp]
  uint32_t caps;             // entries per fixed slot
  const void *theta;         // COLLECT == 2: [L][F] thresholds in the model dtype
  int64_t theta_stride;
};

// Launchers that live in encode.hip and are used by the fused entry points in select.hip.
//   collect 0: plain store of the pre-activations; with `gate` only the layers whose state is
//              ST_RETRY are computed
//   collect 1: no store; elements whose value reaches the layer's cut go to the pool
//   collect 2: no store; elements with value >= theta[layer][feature] go to the pool
// Returns CLT_ERR_ARG when the shape does not qualify for the matrix-core kernel in a
// collecting mode (the caller then runs the separate encode + select path).
int clt_launch_encode(const void *x, const void *w, const void *b, void *pre, int64_t T, int64_t d, int64_t F,
                      int64_t L, int64_t xs, int64_t wstr, int64_t bs, int64_t ps, int dtype, int collect,
                      const SelState *gate, const CollectArgs *ca, hipStream_t stream);
bool clt_encode_can_collect(const void *x, const void *w, const void *b, int64_t T, int64_t d, int64_t F,
                            int64_t xs, int64_t wstr, int64_t bs, int dtype);
