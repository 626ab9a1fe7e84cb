/*
 * clt_hip.h - C ABI of libclt_hip.so, the gfx950 (MI355X) implementation of the
 * cross-layer-transcoder forward path: encoder projection, BatchTopK / TokenTopK /
 * JumpReLU selection into a compact survivor list, and sparse cross-layer decode.
 *
 * The reference (curt-tigges/crosslayer-coding) has no native boundary for this
 * path: it issues stock ATen ops from Python.  Each entry point below names the
 * reference call site (file:line, relative to the reference checkout) whose work
 * it replaces.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - sizes and strides are int64 element counts (strides between layers);
 *   - `dtype` is CLT_F32, CLT_BF16 or CLT_F16 and names the model dtype (inputs, weights,
 *     pre-activations, survivor values, outputs unless said otherwise).  CLT_F16 (IEEE half,
 *     fp32 accumulation, one rounding per product) is taken by the forward-path entry points -
 *     encoder, column statistics, selection, thresholds, the theta-estimation minimum, packing,
 *     decode, densify, decoder norms, the dense accumulation of per-target tying, the evaluator
 *     reductions and the store feed;
 *     the gradient, optimiser and tile entry points (and clt_encode_segmented, which serves the
 *     threshold gradient) return CLT_ERR_DTYPE for it;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - functions launch asynchronously on `stream` and return CLT_OK or a negative
 *     error code; nothing is allocated or freed inside;
 *   - rows of the survivor list ("CSR") are numbered r = layer * T + token;
 *     row_ptr has L*T+1 int32 entries, col holds feature indices in ascending
 *     order inside a row, val the raw pre-activation values in the model dtype.
 */
#ifndef CLT_HIP_H
#define CLT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CLT_F32 0
#define CLT_BF16 1
#define CLT_F16 2 /* forward-path entry points only, see above */

#define CLT_OK 0
#define CLT_ERR_ARG (-1)       /* null pointer, negative size, unsupported combination */
#define CLT_ERR_DTYPE (-2)     /* dtype is not one this entry point takes */
#define CLT_ERR_WORKSPACE (-3) /* workspace smaller than clt_*_workspace_bytes() says */
#define CLT_ERR_LAUNCH (-4)    /* HIP reported an error when launching */
#define CLT_ERR_ALIGN (-5)     /* a pointer or row pitch is not 16-byte aligned */
#define CLT_ERR_RANGE (-6)     /* a size exceeds what the kernels index (see each call) */

/* decoder tying, reference clt/config/clt_config.py:41 */
#define CLT_TYING_NONE 0
#define CLT_TYING_PER_SOURCE 1
#define CLT_TYING_PER_TARGET 2

/* selection scope, reference clt/config/clt_config.py:31 */
#define CLT_TOPK_PER_LAYER 0
#define CLT_TOPK_GLOBAL 1

/* predicates of clt_threshold_count / clt_threshold_emit */
#define CLT_PRED_GE_THETA 0 /* x >= theta[layer][feature]   (JumpReLU) */
#define CLT_PRED_GT_ZERO 1  /* x > 0                        (ReLU)     */
#define CLT_PRED_NONZERO 2  /* x != 0                       (compaction of a dense tensor) */

/* de-normalisation applied by clt_reconstruction_stats (reference clt/training/evaluator.py:279-292) */
#define CLT_DENORM_NONE 0
#define CLT_DENORM_MEAN_STD 1 /* x * std[layer][column] + mean[layer][column] */
#define CLT_DENORM_SCALE 2    /* x / scale   (scale = sqrt(d_model)) */

/* Library version (major*10000 + minor*100 + patch). */
int clt_version(void);

/* Static text for an error code. */
const char *clt_error_string(int code);

/*
 * Encoder projection for L layers in one launch:
 *   pre[l][t][f] = sum_k x[l][t][k] * w[l][f][k] + b[l][f]
 * x [L][T][d], w [L][F][d] (nn.Linear layout), b [L][F] or NULL, pre [L][T][F].
 * fp32 accumulation, one rounding to the model dtype.
 * Replaces F.linear in ColumnParallelLinear.forward (clt/models/parallel.py:286)
 * as called by Encoder.get_preactivations (clt/models/encoder.py:101), for every
 * layer that Encoder.encode_all_layers walks (clt/models/encoder.py:151-162).
 */
int clt_encode(const void *x, const void *w, const void *b, void *pre,
               int64_t T, int64_t d, int64_t F, int64_t L,
               int64_t x_layer_stride, int64_t w_layer_stride,
               int64_t b_layer_stride, int64_t pre_layer_stride,
               int dtype, void *stream);

/*
 * 1 when clt_encode runs these operands on the matrix cores: T >= 256, F >= 256, F % 4 == 0,
 * d a whole number of 128-byte stages (64 elements of 16 bits, 32 of fp32), 16-byte aligned
 * pointers, layer strides that keep every layer 16-byte aligned (the bias stride a multiple
 * of 8 elements).  0: the call is served by a generic kernel with one thread per output,
 * two to three orders of magnitude slower on large shapes; a caller with such a shape does
 * better to hand over zero-padded copies (the host mirror does, crosslayer_coding_amd.engine.encode).
 * No counterpart in the reference (its F.linear takes any shape at one speed).
 */
int clt_encode_fast_path(const void *x, const void *w, const void *b, const void *pre,
                         int64_t T, int64_t d, int64_t F, int64_t L,
                         int64_t x_layer_stride, int64_t w_layer_stride,
                         int64_t b_layer_stride, int64_t pre_layer_stride, int dtype);

/*
 * The same product with both operands cut into n_seg segments of d_seg along K, each segment
 * in a matrix of its own:
 *   pre[t][f] = sum_q sum_k x[q * x_seg_stride + t * x_row_stride + k] * w[q * w_seg_stride + f * w_row_stride + k]
 * (k < d_seg; strides in elements, a segment stride of 0 repeats the matrix).  No bias, one layer.
 * It is the product of the stacked loss gradients [T][(L-s) d] with the stacked decoders
 * [F][(L-s) d] that autograd forms per source layer behind JumpReLU.backward
 * (clt/models/activations.py:183-220 reached through Decoder.decode, clt/models/decoder.py:176-340),
 * taken from the gradient slab and the packed decoder slab where they lie, without copying them
 * side by side.  Needs T >= 256, F >= 256, d_seg a multiple of 64 (bf16) / 32 (fp32) elements with an
 * even number of such pieces over all segments, 16-byte aligned rows; CLT_ERR_ARG otherwise.
 */
int clt_encode_segmented(const void *x, const void *w, void *pre,
                         int64_t T, int64_t d_seg, int64_t n_seg, int64_t F,
                         int64_t x_seg_stride, int64_t x_row_stride,
                         int64_t w_seg_stride, int64_t w_row_stride,
                         int dtype, void *stream);

/*
 * Per-feature ranking statistics of the global BatchTopK / TokenTopK helper:
 *   mean[l][f]  = mean over tokens of pre[l][:, f]
 *   denom[l][f] = unbiased std over tokens + 1e-6
 * both rounded to the model dtype as the reference's tensors are, stored as fp32.
 * Replaces preact.mean(dim=0) / preact.std(dim=0) (clt/models/activations.py:281-283).
 */
int clt_colstats(const void *pre, float *mean, float *denom,
                 int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                 int dtype, void *stream);

/*
 * As clt_colstats, and also stdv[l][f] = the unbiased std itself (rounded to the model dtype,
 * stored as fp32), which the post-hoc threshold estimation averages over batches
 * (clt/models/theta.py:305-318).
 */
int clt_colstats_full(const void *pre, float *mean, float *stdv, float *denom,
                      int64_t T, int64_t F, int64_t L, int64_t pre_layer_stride,
                      int dtype, void *stream);

/*
 * One batch of the post-hoc threshold estimation
 * (ThetaManager._update_min_selected_preactivations, clt/models/theta.py:82-173): for every
 * (layer, feature), the minimum over the survivors with a positive value of their z-score
 * (x - mean) / denom evaluated in the model dtype; where that minimum is finite,
 * sum[l][f] += min and count[l][f] += 1 (both [L][F] in the model dtype, each addition
 * rounded to it).  workspace: L*F*4 bytes.
 */
int clt_selected_min_accumulate(const int32_t *row_ptr, const int32_t *col, const void *val,
                                const float *mean, const float *denom,
                                int64_t T, int64_t F, int64_t L, int dtype,
                                void *sum, void *count,
                                void *workspace, size_t workspace_bytes, void *stream);

/*
 * BatchTopK selection into a survivor list.
 *   mode CLT_TOPK_PER_LAYER: for each layer, the min(k*T, T*F) largest of its T*F
 *     pre-activations (ranking on the raw value), i.e. BatchTopK._compute_mask
 *     (clt/models/activations.py:11-36) as applied per layer by
 *     batchtopk_per_layer_activation (clt/activations/registry.py:43-72).
 *   mode CLT_TOPK_GLOBAL: the min(k*T, T*L*F) largest over all layers, ranked on
 *     (x - mean[l][f]) / denom[l][f] evaluated in the model dtype; the raw value
 *     is what is kept: _apply_batch_topk_helper (clt/models/activations.py:261-357).
 * Ties at the threshold go to the lowest flat index of the [T, F] (per layer) or
 * [T, L*F] (global) block; -0.0 == +0.0; NaN ranks above +inf.
 * Outputs: row_ptr [L*T+1], col / val with room for the survivor total
 * (L * min(k*T, T*F) per-layer, min(k*T, T*L*F) global).
 * Limits: T*F*L < 2^32, F % 8 == 0 for bf16 / F % 4 == 0 for fp32 on the fast
 * path (other F take a scalar path), pre rows 16-byte aligned on the fast path.
 */
size_t clt_batchtopk_workspace_bytes(int64_t T, int64_t F, int64_t L, int64_t k,
                                     int mode, int dtype);
int clt_batchtopk_select(const void *pre, int64_t T, int64_t F, int64_t L,
                         int64_t pre_layer_stride, int64_t k, int mode,
                         const float *mean, const float *denom, int dtype,
                         int32_t *row_ptr, int32_t *col, void *val,
                         void *workspace, size_t workspace_bytes, void *stream);

/*
 * Encoder projection and per-layer BatchTopK in one path, without writing the dense
 * pre-activations: the encoder's epilogue compares every value with a per-layer cut found
 * from a small sample beforehand and appends the ones that reach it to a candidate pool; the
 * exact selection (same result as clt_encode followed by clt_batchtopk_select with
 * CLT_TOPK_PER_LAYER, same tie rule) then runs on the pool only.
 *   clt_encode_collect   sample, cut, encoder with the collecting epilogue, first histogram
 *   clt_collect_select   threshold, tie allotment, ordered write of row_ptr / col / val
 * Both calls take the same workspace (clt_encode_collect_workspace_bytes) and must run on
 * the same stream, clt_collect_select after clt_encode_collect.
 * `pre` [L][T][F] is scratch: it is written only for a layer whose cut turned out unusable
 * (fewer than k*T candidates, or no pool space left), which then takes the streaming route.
 * clt_encode_collect_supported returns 1 when the shapes qualify (T >= 256 and F >= 256 with
 * any remainder: a last tile is shifted back inside the matrix and reports only the tokens
 * and features its neighbour does not own; F % 8 == 0, d % 64 == 0 for 16-bit elements /
 * d % 32 == 0 for fp32, 16-byte aligned rows, k > 0), else 0; callers then use clt_encode +
 * clt_batchtopk_select.
 * Replaces the same reference calls as clt_encode and clt_batchtopk_select
 * (clt/models/encoder.py:151-162, clt/activations/registry.py:43-72,
 * clt/models/activations.py:11-36).
 */
int clt_encode_collect_supported(const void *x, const void *w, const void *b,
                                 int64_t T, int64_t d, int64_t F, int64_t L,
                                 int64_t x_layer_stride, int64_t w_layer_stride,
                                 int64_t b_layer_stride, int64_t k, int dtype);
size_t clt_encode_collect_workspace_bytes(int64_t T, int64_t d, int64_t F, int64_t L,
                                          int64_t k, int dtype);
int clt_encode_collect(const void *x, const void *w, const void *b, void *pre,
                       int64_t T, int64_t d, int64_t F, int64_t L,
                       int64_t x_layer_stride, int64_t w_layer_stride,
                       int64_t b_layer_stride, int64_t pre_layer_stride,
                       int64_t k, int dtype, void *workspace, size_t workspace_bytes,
                       void *stream);
int clt_collect_select(const void *pre, int64_t T, int64_t F, int64_t L,
                       int64_t pre_layer_stride, int64_t k, int dtype,
                       int32_t *row_ptr, int32_t *col, void *val,
                       void *workspace, size_t workspace_bytes, void *stream);

/*
 * TokenTopK selection: per token row, the kk largest of its F (per layer) or L*F
 * (global, ranked on the z-score as above) entries.  kk is the already resolved
 * integer count (fraction/ceil rule of clt/models/activations.py:108-116).
 * Replaces TokenTopK._compute_mask (clt/models/activations.py:99-128) and
 * _apply_token_topk_helper (clt/models/activations.py:391-491).
 */
size_t clt_tokentopk_workspace_bytes(int64_t T, int64_t F, int64_t L, int64_t kk,
                                     int mode, int dtype);
int clt_tokentopk_select(const void *pre, int64_t T, int64_t F, int64_t L,
                         int64_t pre_layer_stride, int64_t kk, int mode,
                         const float *mean, const float *denom, int dtype,
                         int32_t *row_ptr, int32_t *col, void *val,
                         void *workspace, size_t workspace_bytes, void *stream);

/*
 * Threshold activations (JumpReLU, ReLU) and compaction of a dense activation
 * tensor, in two calls because the survivor total is data dependent:
 *   clt_threshold_count fills row_ptr [L*T+1] (row_ptr[L*T] = total);
 *   the caller sizes col/val from the total and calls clt_threshold_emit.
 * theta [L][F] in the model dtype (already exp()'d and rounded), used by
 * CLT_PRED_GE_THETA only.  Replaces JumpReLU.forward
 * (clt/models/activations.py:177-180) as called by ThetaManager.jumprelu
 * (clt/models/theta.py:70-79), F.relu (clt/activations/registry.py:30-33), and
 * the `activation_tensor != 0` scans of Decoder.decode (clt/models/decoder.py:230, 270).
 * workspace: (L*T) * 4 bytes.
 */
int clt_threshold_count(const void *pre, int64_t T, int64_t F, int64_t L,
                        int64_t pre_layer_stride, const void *theta, int pred,
                        int dtype, int32_t *row_ptr, void *workspace,
                        size_t workspace_bytes, void *stream);
int clt_threshold_emit(const void *pre, int64_t T, int64_t F, int64_t L,
                       int64_t pre_layer_stride, const void *theta, int pred,
                       int dtype, const int32_t *row_ptr, int32_t *col, void *val,
                       const int32_t *skip, void *stream);

/*
 * The same activations kept dense, for densities at which a survivor list is the larger object
 * (a ReLU model, JumpReLU thresholds at the start of a training run): x [L][T][F] is gated in
 * place - x where the predicate holds (CLT_PRED_GE_THETA or CLT_PRED_GT_ZERO), else 0 - and
 * *total (device memory) receives the number of elements kept.  The result is the dense
 * activation tensor the reference itself works on (clt/models/activations.py:177-180,
 * clt/activations/registry.py:30-33 as called from clt/models/clt.py:271-277), ready for the
 * dense decode products.
 */
int clt_threshold_dense(void *x, int64_t T, int64_t F, int64_t L, int64_t layer_stride,
                        const void *theta, int pred, int dtype, uint64_t *total, void *stream);

/*
 * For callers that do not read the survivor total back between a count call and its emit call (no
 * host synchronisation in the forward).  Such a caller gives col / val a capacity that no batch it can
 * represent exceeds - min(L*T*F, 2^31 - 1) entries, the most an int32 row pointer addresses - and runs
 * this check on the device in between.  If the total row_ptr[R] (R = L*T) is negative (a count beyond
 * 2^31 - 1 is stored as -2) or exceeds `capacity`, *status = 1 and the list is emptied (row_ptr := 0
 * everywhere, so every later kernel sees rows without survivors); otherwise *status = 0.  The emit
 * calls take `status` as their `skip` argument and write nothing when it is set (NULL: no check).  A
 * batch with *status = 1 has NO valid survivor list: the caller must not hand results computed from it
 * on (see clt_poison_if).  No counterpart in the reference, where the dense mask has a fixed size.
 */
int clt_survivors_fit(int32_t *row_ptr, int64_t R, int64_t capacity, int32_t *status, void *stream);

/*
 * Fills `buf` (`bytes` of it, 4-byte aligned) with NaN bit patterns (all bits set:
 * NaN as float32, bfloat16 and float16 alike) when *flag != 0, and does nothing otherwise; the decision
 * is taken on the device.  For results computed from a survivor list that clt_survivors_fit or
 * clt_encode_threshold_recover had to give up on: they become unmistakably invalid instead of looking
 * like reconstructions without active features.  No counterpart in the reference.
 */
int clt_poison_if(void *buf, int64_t bytes, const int32_t *flag, void *stream);

/*
 * clt_threshold_count for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments and result as clt_threshold_count without the workspace: the per-row counters live
 * in a device array inside the library (4 MiB per GPU, held until the process ends), so the call
 * allocates and frees nothing.  Limit: L*T <= 1048576 rows, else CLT_ERR_RANGE.  The device that
 * owns `stream` must be current.  All calls on one GPU share the array: calls that overlap on one
 * GPU (different streams or threads) race; calls on one stream are ordered and safe.  The first call
 * on a device looks the array's address up (hipGetSymbolAddress); make that call outside a capture.
 */
int clt_threshold_count_static(const void *pre, int64_t T, int64_t F, int64_t L,
                               int64_t pre_layer_stride, const void *theta, int pred,
                               int dtype, int32_t *row_ptr, void *stream);

/*
 * Encoder projection and JumpReLU in one path, without writing the dense pre-activations:
 * the encoder's epilogue compares every value with its feature's threshold and appends the
 * survivors to a pool; the survivor list is then laid out from the pool.  Same result as
 * clt_encode followed by clt_threshold_count / clt_threshold_emit with CLT_PRED_GE_THETA.
 *   clt_encode_threshold_count  projection + collection, fills row_ptr [L*T+1];
 *                               row_ptr[L*T] = survivor total, or -1 when the pool was too
 *                               small (then use the separate calls)
 *   clt_encode_threshold_emit   writes col / val (sized from the total) from the pool
 * theta [L][F] in the model dtype (already exp()'d and rounded).  density_ppm is the caller's
 * estimate of the survivor density in parts per million; it sizes the pool (three times that
 * per 128 x 128 tile plus twice that overall) and must be the same in all three calls.
 * clt_encode_threshold_supported: same shape conditions as clt_encode_collect_supported.
 * Replaces F.linear (clt/models/parallel.py:286) + ThetaManager.jumprelu
 * (clt/models/theta.py:70-79, clt/models/activations.py:177-180) for all layers.
 */
int clt_encode_threshold_supported(const void *x, const void *w, const void *b, const void *theta,
                                   int64_t T, int64_t d, int64_t F, int64_t L,
                                   int64_t x_layer_stride, int64_t w_layer_stride,
                                   int64_t b_layer_stride, int64_t theta_layer_stride,
                                   int64_t density_ppm, int dtype);
size_t clt_encode_threshold_workspace_bytes(int64_t T, int64_t d, int64_t F, int64_t L,
                                            int64_t density_ppm, int dtype);
int clt_encode_threshold_count(const void *x, const void *w, const void *b, const void *theta,
                               int64_t T, int64_t d, int64_t F, int64_t L,
                               int64_t x_layer_stride, int64_t w_layer_stride,
                               int64_t b_layer_stride, int64_t theta_layer_stride,
                               int64_t density_ppm, int dtype, int32_t *row_ptr,
                               void *workspace, size_t workspace_bytes, void *stream);
int clt_encode_threshold_emit(int64_t T, int64_t F, int64_t L, int64_t density_ppm, int dtype,
                              const int32_t *row_ptr, int32_t *col, void *val, const int32_t *skip,
                              void *workspace, size_t workspace_bytes, void *stream);

/*
 * The fused route's fallback, decided and run on the device: call it between
 * clt_encode_threshold_count and the emit calls, on the same stream, with the same workspace and
 * density_ppm.  If the pool of clt_encode_threshold_count was too small (row_ptr[L*T] == -1), the
 * projection is repeated with the dense store into `pre` [L][T][F] (scratch, written only then),
 * compared with the thresholds and row_ptr is rebuilt from the dense counts - the route of
 * clt_encode + clt_threshold_count, launched behind a device flag so that the host never has to
 * look.  status is int32[3] on the device:
 *   status[0]  pass as `skip` to clt_encode_threshold_emit (set when the pool list is not the one to emit)
 *   status[1]  pass as `skip` to clt_threshold_emit on `pre` with CLT_PRED_GE_THETA (set when the dense
 *              route was not needed)
 *   status[2]  set when the batch has more than `capacity` survivors (or more than 2^31 - 1): the list
 *              was emptied as by clt_survivors_fit, both emits skip; cannot happen with
 *              capacity = min(L*T*F, 2^31 - 1) unless the total exceeds 2^31 - 1
 * After both emit calls the list in row_ptr / col / val is the exact one whichever route produced it.
 * theta_layer_stride must be F.  Replaces the same reference calls as clt_encode_threshold_count
 * (clt/models/parallel.py:286, clt/models/theta.py:70-79), for a batch of any density.
 */
int clt_encode_threshold_recover(const void *x, const void *w, const void *b, const void *theta, void *pre,
                                 int64_t T, int64_t d, int64_t F, int64_t L,
                                 int64_t x_layer_stride, int64_t w_layer_stride,
                                 int64_t b_layer_stride, int64_t theta_layer_stride,
                                 int64_t pre_layer_stride, int64_t density_ppm, int dtype,
                                 int32_t *row_ptr, int64_t capacity, int32_t *status,
                                 void *workspace, size_t workspace_bytes, void *stream);

/*
 * Repack decoder weights from the checkpoint layout [d][F] (nn.Linear weight of
 * RowParallelLinear, clt/models/parallel.py:66-70) to feature-major [F][pitch] (pitch =
 * clt_decoder_pitch(d, dtype); the padding columns are not written), so a feature's decoder vector is
 * one contiguous run.  n_dec matrices; in_stride / out_stride are the element strides between matrices
 * (out_stride = F * pitch for a slab).
 */
int clt_pack_decoder(const void *w_ref, void *w_packed, int64_t d, int64_t F,
                     int64_t n_dec, int64_t in_stride, int64_t out_stride,
                     int dtype, void *stream);

/*
 * Sparse cross-layer decode for targets t in [t_begin, t_end):
 *   out[t][tok][:] = sum over sources s <= t with bit s of src_mask set,
 *                    over survivors (f, v) of row s*T+tok:
 *                        v' * w_packed[slot(s,t)][f][:]
 *                    + bias_sum[t][:] (+ skip_add[t][tok][:])
 *   v' = v, or (v + feat_offset[t][f]) * feat_scale[t][f] (model-dtype rounding
 *   after each step, zeros left untouched) when those arrays are given.
 *   slot(s,t): CLT_TYING_NONE       s*L - s*(s-1)/2 + (t-s)  (order of "s->t" keys)
 *              CLT_TYING_PER_SOURCE s
 *              CLT_TYING_PER_TARGET t
 * fp32 accumulation; out [L][T][d] in the model dtype (out_f32 = 0) or fp32.
 * bias_sum [L][d] fp32 or NULL, feat_offset / feat_scale [L][F] model dtype or
 * NULL, skip_add [L][T][d] fp32 or NULL.
 * Replaces Decoder.decode (clt/models/decoder.py:176-340) and the
 * RowParallelLinear.forward calls inside it (clt/models/parallel.py:366, 380-381),
 * for all targets that CrossLayerTranscoder.forward loops over
 * (clt/models/clt.py:192-199).
 * Limits: L <= 64; d % 8 == 0 (bf16) / d % 4 == 0 (fp32) on the fast path.
 * workspace: NULL runs one wavefront per (target, token) over all features and sources.
 * With a workspace of clt_decode_workspace_bytes() each of the 8 XCDs works on one eighth of a
 * decoder matrix at a time - 2 feature slices x 4 column quarters when d is a multiple of 256 and
 * the decoders are not tied per target, 8 feature slices of whole rows otherwise - with one
 * launch per source layer, so that the eighth stays in one L2 while all tokens pass; partial
 * sums live as fp32 rows per (slice, target, token) in the workspace and are added in a fixed
 * order at the end.  All routes give the same result up to fp32 summation order.
 */
size_t clt_decode_workspace_bytes(int64_t T, int64_t d, int64_t F, int64_t L);
int clt_decode_sparse(const int32_t *row_ptr, const int32_t *col, const void *val,
                      const void *w_packed, const float *bias_sum,
                      const void *feat_offset, const void *feat_scale,
                      const float *skip_add, void *out,
                      int64_t T, int64_t d, int64_t F, int64_t L,
                      int tying, int64_t t_begin, int64_t t_end, uint64_t src_mask,
                      int dtype, int out_f32, void *workspace, size_t workspace_bytes,
                      void *stream);

/*
 * Which schedule clt_decode_sparse takes for these shapes when it is given a workspace of
 * `workspace_bytes` (16-byte aligned weights assumed): one of CLT_ROUTE_*, or a negative error code.
 * A query for callers and tests; it launches nothing.
 */
#define CLT_ROUTE_GENERIC 0            /* any d: lanes stride over the output row */
#define CLT_ROUTE_SINGLE 1             /* one wavefront per (target, token), all sources */
#define CLT_ROUTE_SLICED 2             /* 8 feature slices, one launch per source layer */
#define CLT_ROUTE_SLICED_ALL_SOURCES 3 /* 8 feature slices, decoders tied per target: one launch */
#define CLT_ROUTE_QUARTER 4            /* 2 feature slices x 4 column quarters, one launch per source */
#define CLT_ROUTE_LINE 5               /* column parts of one cache line, one launch per source */
int clt_decode_route(int64_t T, int64_t d, int64_t F, int64_t L, int tying, int dtype,
                     size_t workspace_bytes);

/*
 * Keeping the packed copy true to its parameters without the host looking at them.  The reference reads
 * its decoder parameters in place in every forward (clt/models/parallel.py:335-383), so any write to
 * them - also one that bypasses autograd's version counters, like `weight.data.copy_(...)` - shows in the
 * next result.  clt_decoder_fingerprint hashes a sample of every decoder parameter (w_refs_dev[i] = address
 * of matrix i, [d][F]; all of a matrix up to 1 MiB, of a larger one a 256-byte run per row on a diagonal, so
 * that every row is looked at and every column in several rows):
 * changed[i] = 1 where the hash differs from the one kept in state, and state is brought up to date.
 * store_only != 0 only records (after the caller itself wrote the parameters).  `state` holds 16 * n_dec
 * 64-bit words (one 128-byte line per matrix, 128-byte aligned), zeroed by the caller before the first
 * call - made with store_only - and left alone afterwards.
 * clt_pack_decoders_if repacks the matrices whose flag is set (clt_pack_decoder otherwise) - a launch that
 * costs microseconds when no flag is set.  Both run on the stream; nothing is read back.  A write to the
 * whole matrix, a whole row or a whole column of it is always seen; one that touches a few scattered elements
 * of a large matrix may miss the sample.
 */
int clt_decoder_fingerprint(void *const *w_refs_dev, int64_t n_dec, int64_t d, int64_t F, int dtype,
                            uint64_t *state, int32_t *changed, int store_only, void *stream);
int clt_pack_decoders_if(void *const *w_refs_dev, void *w_packed, int64_t n_dec, int64_t d, int64_t F,
                         int dtype, const int32_t *changed, void *stream);

/*
 * bias_sum[t][c] (fp32 [L][d]) = sum of the biases of the decoders that run for target t: one per source
 * s <= t whose bit is set in src_mask, in ascending order (clt/models/decoder.py:294-295 through
 * parallel.py:380-381), or the target's own decoder for per-target tying (decoder.py:250-251).
 * b_refs_dev[slot] = address of the bias of decoder `slot` (n_dec of them, d elements each).
 */
int clt_bias_sum(void *const *b_refs_dev, int64_t n_dec, int64_t d, int64_t L, int tying, uint64_t src_mask,
                 int dtype, float *out, void *stream);

/*
 * Layout of the packed (feature-major) decoder slab that every entry point taking `w_packed` assumes:
 *   w_packed[slot][f][c],  0 <= c < d,  rows clt_decoder_pitch(d, dtype) elements apart,
 *   matrices F * pitch elements apart.
 * pitch = d, except that a row of a whole, EVEN number of 128-byte cache lines gets one line more
 * (d + 64 in bf16, d + 32 in fp32): with an even line pitch one column part of all rows falls on a
 * fraction of the 16 L2 channels, and the schedules of clt_decode_sparse that give each XCD one column
 * part would use only that fraction of its L2.  clt_pack_decoder writes this layout.
 * clt_decoder_slab_elems: the number of elements such a slab has, n_dec * F * pitch with n_dec =
 * L(L+1)/2 untied and L tied, formed in 64 bits as every kernel forms slot * F * pitch + f * pitch + c
 * (the Pythia-410m shape has 1.1e10 elements); callers check their allocation against it.  Both return
 * -1 on bad arguments.
 */
int64_t clt_decoder_pitch(int64_t d, int dtype);
int64_t clt_decoder_slab_elems(int64_t d, int64_t F, int64_t L, int tying, int dtype);

/*
 * Running dense sum of activations over source layers, the operand of a decoder tied per target
 * (`summed_activation += activation_tensor`, clt/models/decoder.py:208-246):
 *   acc[tok][f] = round(acc[tok][f] + v')   for the survivors (f, v) of rows layer*T .. layer*T+T-1
 *   v' = v, or round(round(v + feat_offset[f]) * feat_scale[f]) on non-zero v when those rows
 *   ([F], the target layer's, model dtype) are given (decoder.py:228-244).
 * acc [T][F] in the model dtype, every addition rounded to it as the reference's tensor is; init != 0
 * clears acc first (layer < 0 with init != 0: clear only).  The decode of target t is then one dense product of acc with the target's
 * decoder in its checkpoint layout [d][F], which clt_encode computes (x = acc, w = decoder weight,
 * b = decoder bias): the route for targets whose summed activations are dense enough that the matrix
 * cores beat the row gather of clt_decode_sparse.
 */
int clt_accumulate_dense(const int32_t *row_ptr, const int32_t *col, const void *val,
                         const void *feat_offset, const void *feat_scale, void *acc,
                         int64_t T, int64_t F, int64_t layer, int init, int dtype, void *stream);

/*
 * Dense materialisation of a survivor list: out[l][t][f] = value or 0.
 * out_f32 selects fp32 output (JumpReLU returns fp32, activations.py:180).
 * Replaces `x * mask.to(x.dtype)` (clt/models/activations.py:65, 347).
 */
int clt_densify(const int32_t *row_ptr, const int32_t *col, const void *val,
                void *out, int64_t T, int64_t F, int64_t L, int64_t out_layer_stride,
                int dtype, int out_f32, void *stream);

/*
 * Per-feature decoder norms from packed weights:
 *   norms[s][f] = sqrt(sum over decoders fed by source s of ||w[f][:]||^2)
 * fp32 accumulation, rounded to the model dtype.
 * Replaces Decoder.get_decoder_norms (clt/models/decoder.py:374-485).
 */
int clt_decoder_norms(const void *w_packed, void *norms, int64_t d, int64_t F,
                      int64_t L, int tying, int dtype, void *stream);

/*
 * ---- backward pass for the MSE reconstruction loss ---------------------------------------
 * The reference trains through torch autograd (clt/training/trainer.py:663-751); these entry
 * points compute the same gradients from the survivor list, without dense activations.
 *
 * clt_mse_loss_grad: loss_per_layer[l] = mean((rec'[l] - target'[l])^2) as nn.MSELoss gives per
 *   layer (clt/training/losses.py:45-92, summed over layers by the caller), where ' is the
 *   de-normalisation LossManager applies first (losses.py:70-86): CLT_DENORM_NONE nothing,
 *   CLT_DENORM_MEAN_STD x * std[l][c] + mean[l][c] (the store's target statistics, [L][d] in the model
 *   dtype), CLT_DENORM_SCALE x / denorm_scale (sqrt(d_model)), each step rounded to the model dtype.
 *   g[l][t][:] = d loss / d rec = 2 (rec' - target') / (T d) * std (or / denorm_scale) in fp32 (and,
 *   when g_model != NULL, the same rounded to the model dtype: what clt_decoder_weight_grad reads), and
 *   (when bias_grad != NULL) bias_grad[l][:] = sum over tokens of g[l] - the gradient of every decoder
 *   bias that feeds target l.
 *   rec / target [L][T][d] in the model dtype; workspace clt_mse_workspace_bytes().
 * clt_decode_backward_values: dval[j] = sum over targets t >= s of g[t][token] . w[slot(s,t)][f]
 *   for survivor j = (s, token, f): the gradient of the loss with respect to the kept
 *   activation, which the straight-through gate passes on to the pre-activation
 *   (clt/models/activations.py:66-96).  With feat_scale ([L][F] model dtype, tied decoders,
 *   clt/models/decoder.py:228-285) target t's share carries the factor feat_scale[t][f] for a non-zero
 *   activation (val is needed then; both may be NULL otherwise).  dval [nnz] fp32; nnz = row_ptr[L*T]; workspace
 *   clt_decode_backward_workspace_bytes() (slice pointers and one partial per target and survivor,
 *   summed in target order); `nnz` is the stride of those partials: any value >= row_ptr[L*T], e.g. the
 *   number of entries col holds, so that no total has to be read back.
 * clt_feature_lists: the survivor list regrouped by (layer, feature): list_ptr [L*F+1],
 *   list_tok [nnz] token of each entry, list_src [nnz] its position in col / val.  Every
 *   list is in ascending token order, so sums over a list always run in the same order (T <= 262144).
 *   Pass list_tok = list_src = NULL to get the counts only.
 * clt_decoder_weight_grad: dw_packed[slot(s,t)][f][:] = sum over the list of (s, f) of
 *   val * g_model[t][token][:] (fp32 sums, feature-major, dense rows of d elements); with tied decoders the
 *   slot collects every pair that shares it (CLT_TYING_PER_SOURCE: all t >= s; CLT_TYING_PER_TARGET:
 *   all s <= t), so dw_packed has L matrices instead of L(L+1)/2.  One launch per target layer,
 *   in ascending order on `stream`.
 *   With feat_offset / feat_scale ([L][F] model dtype or NULL) the values are first transformed as the
 *   forward transforms them for target t: (val + feat_offset[t][f]) * feat_scale[t][f] on non-zero val.
 * clt_feature_affine_grad: gradients of feat_offset / feat_scale, fp32 [L][F] (either may be NULL):
 *   d_offset[t][f] = feat_scale[t][f] * sum h, d_scale[t][f] = sum h * (val + feat_offset[t][f]), over the
 *   non-zero survivors of feature f in the sources s <= t, h = g[t][token] . w[slot(s,t)][f].  Call it after
 *   clt_decode_backward_values with the SAME workspace and nnz: it reads the per-target dot products that
 *   call left there.
 * clt_skip_weight_grad: gradient of one skip-connection matrix (rec[t] += x[s] @ W_skip.T,
 *   clt/models/decoder.py:297-338): out[i][j] (+)= sum over tokens of g[token][i] * x[token][j];
 *   g [T][d] fp32 (the loss gradient of the target), x [T][d] model dtype (the source's input),
 *   out [d][d] fp32, accumulate != 0 adds to out.
 * clt_encoder_weight_grad: dw_enc[s][f][:] = sum over the list of dval * x[s][token][:],
 *   db_enc[s][f] = sum of dval (fp32; x [L][T][d] in the model dtype).
 * Limits: d % 8 == 0 (bf16) / d % 4 == 0 (fp32) and d <= 4096.
 */
size_t clt_mse_workspace_bytes(int64_t T, int64_t d, int64_t L);
int clt_mse_loss_grad(const void *rec, const void *target, int64_t T, int64_t d, int64_t L,
                      int dtype, int denorm_mode, const void *mean, const void *stdv,
                      double denorm_scale, float *loss_per_layer, float *g, void *g_model,
                      float *bias_grad, void *workspace, size_t workspace_bytes, void *stream);
size_t clt_decode_backward_workspace_bytes(int64_t T, int64_t L, int64_t nnz);
int clt_decode_backward_values(const int32_t *row_ptr, const int32_t *col, const void *val,
                               const void *w_packed, const void *feat_scale, const float *g,
                               int64_t T, int64_t d, int64_t F, int64_t L, int tying,
                               uint64_t src_mask, int64_t nnz, int dtype, float *dval,
                               void *workspace, size_t workspace_bytes, void *stream);
int clt_feature_affine_grad(const int32_t *list_ptr, const int32_t *list_src, const void *val,
                            const void *feat_offset, const void *feat_scale, int64_t T, int64_t F,
                            int64_t L, uint64_t src_mask, int64_t nnz, int dtype, float *d_offset,
                            float *d_scale, const void *workspace, size_t workspace_bytes, void *stream);
int clt_skip_weight_grad(const float *g, const void *x, float *out, int64_t T, int64_t d,
                         int accumulate, int dtype, void *stream);
size_t clt_feature_lists_workspace_bytes(int64_t F, int64_t L);
int clt_feature_lists(const int32_t *row_ptr, const int32_t *col, int64_t T, int64_t F, int64_t L,
                      int32_t *list_ptr, int32_t *list_tok, int32_t *list_src,
                      void *workspace, size_t workspace_bytes, void *stream);
int clt_decoder_weight_grad(const int32_t *list_ptr, const int32_t *list_tok, const int32_t *list_src,
                            const void *val, const void *g_model, const void *feat_offset,
                            const void *feat_scale, float *dw_packed,
                            int64_t T, int64_t d, int64_t F, int64_t L, int tying, int dtype,
                            void *stream);
int clt_encoder_weight_grad(const int32_t *list_ptr, const int32_t *list_tok, const int32_t *list_src,
                            const float *dval, const void *x, float *dw_enc, float *db_enc,
                            int64_t T, int64_t d, int64_t F, int64_t L, int dtype, void *stream);

/*
 * Adam update with fp32 moments and fp32 gradients on parameters in the model dtype
 * (torch.optim.Adam semantics without weight decay / amsgrad; the reference builds its
 * optimizer in clt/training/trainer.py:290-312).  `step` counts from 1.
 * clt_adam_step: param, grad, m, v share one layout (n elements).
 * clt_adam_step_decoder: one decoder matrix; w_ref is the parameter in the checkpoint layout
 *   [d][F], w_packed its feature-major working copy [F][pitch]; grad_packed, m, v are dense [F][d].  Both
 *   copies receive the same new values.
 * clt_adam_step_decoders: n_dec decoder matrices in one launch.  w_packed is the [n_dec][F][pitch] slab,
 *   grad_packed, m, v are [n_dec][F][d] slabs; the parameters are separate tensors (one per nn.Linear of the reference's
 *   Decoder.decoders, clt/models/decoder.py:57-99), given as a device array of pointers for the kernel and
 *   the same pointers in a host array for checking.
 * clt_adam_step_many: `count` small parameters of n elements each (the decoder biases), gradient and
 *   moments as [count][n] slabs, parameters as a device array of pointers.
 */
int clt_adam_step(void *param, const float *grad, float *m, float *v, int64_t n,
                  double lr, double beta1, double beta2, double eps, int64_t step,
                  int dtype, void *stream);

/*
 * Decoder weight gradient and its Adam step in one pass, for untied decoders: what
 * clt_decoder_weight_grad followed by clt_adam_step_decoders computes (loss.backward() and
 * optimizer.step() of clt/training/trainer.py:663-778 for the decoder weights), without the fp32
 * gradient [n_dec][F][d] ever reaching memory: every gradient row goes from the registers that
 * summed it straight into the update of the moments m, v [n_dec][F][d] and of the feature-major
 * working copy w_packed [n_dec][F][pitch].  Bit-identical to the two-call sequence.  The
 * checkpoint-layout parameters [d][F] are NOT written: clt_unpack_decoders brings them up to date
 * from the working copy (w_refs_dev: device array of n_dec parameter addresses, w_refs_host: the
 * same addresses in host memory or NULL, as for clt_adam_step_decoders).  Everything that reads the decoders of the step being differentiated
 * (clt_decode_backward_values, clt_feature_affine_grad, the threshold-gradient product) must have
 * run before.
 */
int clt_decoder_weight_grad_adam(const int32_t *list_ptr, const int32_t *list_tok,
                                 const int32_t *list_src, const void *val, const void *g_model,
                                 void *w_packed, float *m, float *v,
                                 int64_t T, int64_t d, int64_t F, int64_t L,
                                 double lr, double beta1, double beta2, double eps, int64_t step,
                                 int dtype, void *stream);
int clt_unpack_decoders(const void *w_packed, void *const *w_refs_dev, void *const *w_refs_host,
                        int64_t n_dec, int64_t d, int64_t F, int dtype, void *stream);
/*
 * The same step over COLUMN TILES (same reference lines; the gradient sums of lists that the kernel
 * cuts between two lane pairs are associated differently, so results agree with the call above to
 * fp32 rounding of the gradient and repeat bit for bit from run to run).
 * clt_decoder_weight_grad_adam gathers one row of d loss / d reconstruction per list entry through
 * the L2; here a workgroup parks one 32-byte column slice of one target's g_model [T][d] in its LDS
 * and runs over every (source <= target, feature) row of that slice, so that only the lists, the
 * moments and the parameters pass through the vector memory path.  For that the decoder weights and
 * both moments are kept tiled,
 *     [n_dec][d / CS][F][CS],   CS = clt_decoder_tile_width(...) = 16 bf16 / 8 fp32 columns,
 * so that one slice of consecutive features is contiguous.  clt_decoder_tile_width returns 0 when
 * the shape cannot take this route (d % CS != 0, F % 4 != 0, or T * 32 bytes beyond the LDS of a
 * compute unit, T <= 4350): callers then use clt_decoder_weight_grad_adam with feature-major moments.
 * clt_tile_decoders fills the tiled weights from the feature-major slab [n_dec][F][pitch];
 * clt_untile_decoders writes the slab back from the tiles and, when w_refs_dev / w_refs_host (both
 * or neither) are given, the checkpoint-layout parameters [d][F] too.
 * workspace: clt_decoder_tiles_workspace_bytes(capacity of the lists, dtype) bytes, 256-byte
 * aligned (the list entries regrouped as token|coefficient pairs, and a work counter).
 */
int clt_decoder_tile_width(int64_t T, int64_t d, int64_t F, int dtype);
size_t clt_decoder_tiles_workspace_bytes(int64_t capacity, int dtype);
int clt_tile_decoders(const void *w_packed, void *w_tiles, int64_t n_dec, int64_t d, int64_t F,
                      int dtype, void *stream);
int clt_untile_decoders(const void *w_tiles, void *w_packed, void *const *w_refs_dev,
                        void *const *w_refs_host, int64_t n_dec, int64_t d, int64_t F, int dtype,
                        void *stream);
int clt_decoder_weight_grad_adam_tiled(const int32_t *list_ptr, const int32_t *list_tok,
                                       const int32_t *list_src, const void *val, const void *g_model,
                                       void *w_tiles, float *m_tiles, float *v_tiles,
                                       int64_t T, int64_t d, int64_t F, int64_t L, int64_t capacity,
                                       double lr, double beta1, double beta2, double eps,
                                       int64_t step, int dtype, void *workspace,
                                       size_t workspace_bytes, void *stream);
int clt_adam_step_decoder(void *w_ref, void *w_packed, const float *grad_packed, float *m, float *v,
                          int64_t d, int64_t F, double lr, double beta1, double beta2, double eps,
                          int64_t step, int dtype, void *stream);
int clt_adam_step_decoders(void *const *w_refs_dev, void *const *w_refs_host, int64_t n_dec,
                           void *w_packed, const float *grad_packed, float *m, float *v,
                           int64_t d, int64_t F, double lr, double beta1, double beta2, double eps,
                           int64_t step, int dtype, void *stream);
int clt_adam_step_many(void *const *params_dev, const float *grad, float *m, float *v, int64_t count,
                       int64_t n, double lr, double beta1, double beta2, double eps, int64_t step,
                       int dtype, void *stream);

/*
 * dense[tok][col[j]] = src[j], rounded to the model dtype, for every survivor j of layer `layer`
 * (rows layer*T .. layer*T + T - 1 of the list); the other elements of dense [T][F] are left as they
 * are.  Used for the JumpReLU threshold gradient behind a per-target feature scale: at the kept
 * activations d loss / d activation carries the scale of every target (the values of
 * clt_decode_backward_values), elsewhere it is the plain product (clt/models/decoder.py:228-245,
 * 268-285: the scale is applied to the non-zero activations only; clt/models/activations.py:183-220).
 */
int clt_scatter_survivor_values(const int32_t *row_ptr, const int32_t *col, const float *src,
                                int64_t layer, int64_t T, int64_t F, int64_t L, int dtype,
                                void *dense, void *stream);

/* clt_jumprelu_theta_grad: gradient of the JumpReLU thresholds of one layer (JumpReLU.backward,
 *   clt/models/activations.py:196-199; bandwidth is 1.0 in ThetaManager, clt/models/theta.py:41):
 *     grad_theta[f] = sum over tokens of grad_out[tok][f] * (-pre[tok][f] / bandwidth)
 *                     over the elements with |pre - theta[f]| <= bandwidth / 2
 *   pre, grad_out [T][F] and theta [F] in the model dtype (each arithmetic step is rounded to it,
 *   as the reference's tensor arithmetic is), grad_theta [F] fp32.  The band holds elements on
 *   both sides of the threshold, so pre and grad_out are dense: the caller gets grad_out of a
 *   source layer as one product of the stacked loss gradients with the stacked decoders (clt_encode
 *   serves as that product).  workspace: clt_jumprelu_theta_grad_workspace_bytes(F).
 */
size_t clt_jumprelu_theta_grad_workspace_bytes(int64_t F);
int clt_jumprelu_theta_grad(const void *pre, const void *grad_out, const void *theta, int64_t T,
                            int64_t F, double bandwidth, int dtype, float *grad_theta,
                            void *workspace, size_t workspace_bytes, void *stream);

/* ---- evaluation reductions ---------------------------------------------------
 * clt_survivor_metrics: from a survivor list, per layer the number of entries whose value is
 *   != 0 (nonzero_per_layer [L]; divided by T it is the layer's mean L0 of
 *   CLTEvaluator._compute_sparsity, clt/training/evaluator.py:194-244) and per (layer, feature)
 *   the number of tokens whose value is > fired_eps (fired_count [L][F]; the reference's
 *   `act_bool.sum(dim=0)` of _compute_feature_density, evaluator.py:350-405, which uses 1e-6,
 *   and the `fired_mask_per_token.any(dim=0)` of the trainer's dead-feature update,
 *   clt/training/trainer.py:701-707).  Both outputs are cleared by the call.  col / val may be
 *   NULL for an empty list.
 * clt_dead_feature_update: passes_since_fired[i] = fired_count[i] ? 0 : passes_since_fired[i] + 1
 *   over n = L*F counters (int64, the dtype of Trainer.n_forward_passes_since_fired,
 *   trainer.py:342-347, 711-712).
 * clt_reconstruction_stats: for rec, target [L][T][d] in the model dtype, per layer
 *   stats[l] = { MSE, mean over columns of the population variance of the target, the same of
 *   (target - rec) }, after de-normalising both in the model dtype (mean / std [L][d] in the model
 *   dtype for CLT_DENORM_MEAN_STD); the quantities CLTEvaluator._compute_reconstruction_metrics
 *   (evaluator.py:246-345) turns into explained variance and normalised MSE.
 *   workspace: clt_reconstruction_stats_workspace_bytes(d, L), 8-byte aligned.
 */
int clt_survivor_metrics(const int32_t *row_ptr, const int32_t *col, const void *val, int64_t T,
                         int64_t F, int64_t L, int dtype, float fired_eps,
                         uint64_t *nonzero_per_layer, uint32_t *fired_count, void *stream);
int clt_dead_feature_update(const uint32_t *fired_count, int64_t *passes_since_fired, int64_t n,
                            void *stream);
size_t clt_reconstruction_stats_workspace_bytes(int64_t d, int64_t L);
int clt_reconstruction_stats(const void *rec, const void *target, int64_t T, int64_t d, int64_t L,
                             int dtype, int denorm_mode, const void *mean, const void *stdv,
                             double scale, double *stats, void *workspace, size_t workspace_bytes,
                             void *stream);

/* ---- calibration ------------------------------------------------------------------
 * clt_probe_gather: no counterpart in the reference.  A bare row gather with the access pattern of
 *   clt_decode_sparse (16 bytes per lane, six rows in flight per wavefront): every wavefront of
 *   `blocks` workgroups (4 wavefronts each) sums its share of the rows idx[0..n_idx) of table
 *   [n_rows][row_bytes] (row_bytes % 16 == 0, <= 2048; idx values outside [0, n_rows) are clamped).
 *   to_lds != 0 issues the same loads as direct-to-LDS loads (the encoder's way of bringing its
 *   tiles in; row_bytes >= 1024, the bytes moved are then 2 KB per row).
 *   out: blocks * 256 floats.  Timed with a table that fits an L2, the memory-side cache, or neither,
 *   it gives the rate such a gather can reach on the GPU at hand - the yardstick bench.py prints
 *   next to the decode stage.
 */
int clt_probe_gather(const void *table, int64_t n_rows, int64_t row_bytes, const int32_t *idx,
                     int64_t n_idx, int64_t blocks, int to_lds, float *out, void *stream);

/* ---- activation-store feed -----------------------------------------------------
 * clt_feed_gather: rows of one stored chunk -> rows [out_row0, out_row0 + n) of the batch slabs
 *   x_out, tgt_out [L][T][d] (out_dtype CLT_F32 / CLT_BF16 / CLT_F16), for all layers, inputs and targets.
 *     out[l][out_row0 + j][:] = cast(norm(float(src_l[row_index[j]][:])))
 *   src is the chunk (or a fetched slice of it) in the store's layout
 *   Layer0_Inputs | Layer0_Targets | Layer1_Inputs | ... (ManifestActivationStore._fetch_slice,
 *   clt/training/data/manifest_activation_store.py:555-560): [src_rows][d] elements of src_dtype
 *   (CLT_F32 / CLT_BF16 / CLT_F16) per tensor, a layer's targets src_target_offset elements after
 *   its inputs, layers src_layer_stride elements apart (the packed wire format has
 *   src_target_offset = src_rows*d, src_layer_stride = 2*src_rows*d).  src may be device memory or
 *   pinned (hipHostMalloc) host memory; anything else returns CLT_ERR_ARG.  row_index [n] int32
 *   (device): for a fetched slice, the position of each batch row among the sorted rows that were
 *   fetched (the `reorder_idx` of manifest_activation_store.py:868-872); for a resident chunk,
 *   the row numbers themselves.  An index outside [0, src_rows) is not read: its row becomes NaN.
 *   norm_mode: CLT_DENORM_NONE cast only; CLT_DENORM_MEAN_STD (x - mean) / std with mean / std
 *   [L][d] fp32 per tensor kind (std already holds the store's + 1e-6; a NULL pair leaves that
 *   kind as it is); CLT_DENORM_SCALE x * scale (scale = sqrt(d_model)).  fp32 arithmetic, one
 *   rounding to out_dtype.  Replaces the parse / re-order / cat / normalise / cast tail of
 *   ManifestActivationStore._fetch_and_parse_batch (manifest_activation_store.py:859-934).
 */
int clt_feed_gather(const void *src, int src_dtype, int64_t src_rows, int64_t src_layer_stride,
                    int64_t src_target_offset, const int32_t *row_index, int64_t n, int64_t d,
                    int64_t L, int norm_mode, const float *mean_in, const float *std_in,
                    const float *mean_tg, const float *std_tg, double scale, void *x_out,
                    void *tgt_out, int64_t out_row0, int64_t T, int out_dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CLT_HIP_H */
