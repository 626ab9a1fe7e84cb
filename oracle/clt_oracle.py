"""CPU oracle for the cross-layer-transcoder forward path.

TEST INFRASTRUCTURE ONLY.  This module restates, with plain torch-CPU / numpy
operations, the algorithm the reference runs on its forward path.  It exists so
that the HIP kernels can be checked against it; nothing that ships (the package,
its C-ABI library) may import or call it.  Only ``tests/``, the smoke check and
the ``cpu_baseline`` leg of the benchmark use it, and there only as the checker
or as the timed CPU baseline.

Every function cites the reference lines it follows (paths relative to the
reference checkout).

How each function is pinned (see ``tests/test_oracle_*.py``):

* ``batchtopk_mask`` / ``batchtopk_forward``  - the reference's known-answer
  vectors (tests/unit/models/test_activations.py:10-25, 28-63, 66-111) plus a
  brute-force full-sort selector on small random inputs with forced ties.
* ``tokentopk_mask``  - known answers (test_activations.py:158-283).
* ``jumprelu_forward``  - known answer (test_activations.py:304-315) and the
  ``where(x >= theta, x, 0)`` identity (tests/unit/models/test_theta.py:79-92).
* ``encoder_preactivations``  - affine map checked against a float64 numpy
  contraction (the reference pins it against nn.Linear,
  tests/integration/test_tp_equivalence.py:316-343).
* ``decode``  - additivity over sources (tests/unit/models/test_decoder.py:62-81),
  zero weights give zero output (tests/unit/models/test_tied_decoders.py:138-166),
  and a float64 numpy per-element loop on tiny shapes.
* ``global_batchtopk`` / ``global_tokentopk``  - closed form of the z-score on hand-computable
  columns, and the reference's own outputs on seeded tiny models (the forward cases of
  tests/golden/reference_fixtures.json, written by tests/golden/make_reference_fixtures.py).
* ``theta_estimate_posthoc`` / ``theta_convert``  - a hand-computed two-feature case and the
  properties the reference's own test asserts (tests/unit/models/test_theta.py:110-175:
  thresholds finite and positive, higher for the features that were selected); the
  reference holds no golden numbers for them; pinned by the reference's own run on seeded tiny
  models (theta_estimation cases of tests/golden/reference_fixtures.json).
* ``JumpReLUFunction``  - the reference's table of input / threshold gradients
  (tests/unit/models/test_activations.py:318-381, 16 cases).
* ``mse_loss_and_gradients``  - torch autograd itself computes the gradients; a central
  finite-difference check in float64 on a tiny model pins the loss / gradient pairing, and the
  reference's backward tables (test_activations.py:114-152: grad * mask) pin the gate; the
  reference's own loss and autograd gradients on seeded tiny models (gradients cases of
  tests/golden/reference_fixtures.json: global BatchTopK, JumpReLU with its threshold gradient,
  decoders tied per source and per target) pin the whole function.
* ``sparsity_metrics`` / ``feature_density_metrics`` / ``reconstruction_metrics`` /
  ``dead_feature_update``  - hand-computed small cases, numpy's ``var`` in float64, and the
  closed forms (a perfect reconstruction has explained variance 1 and NMSE 0; an all-zero
  reconstruction of a zero-mean target has NMSE 1); the reference has no test of its evaluator, so
  ``sparsity_metrics`` / ``feature_density_metrics`` / ``reconstruction_metrics`` are also checked
  against the reference's own methods run on a seeded case (evaluator section of
  tests/golden/reference_fixtures.json); ``dead_feature_update`` restates trainer code that cannot be
  imported here (it needs wandb): PARITY UNPINNED beyond the hand-computed case.
* ``store_parse_batch``  - a hand-written two-chunk case with every expected row spelled out, the
  ordering property of the reference's own test (tests/unit/data/test_data_integrity.py:215-294:
  every row once, identified by a value that encodes its position) and its normalisation test
  (:137-213: statistics of the normalised batch, same generator and seed); the reference's store
  tests need h5py files, which this image cannot write: PARITY UNPINNED beyond that.
* ``forward``  - composition of the above; pinned by the reference's own reconstructions and
  activations on six seeded tiny models (global BatchTopK / TokenTopK, JumpReLU, ReLU; untied,
  per-source and per-target decoders; skip connections; feature offset / scale) in
  tests/golden/reference_fixtures.json.

Tie rule.  ``torch.topk(sorted=False)`` leaves the choice among equal ranking
values unspecified (reference activations.py:28).  This oracle fixes it the way
the HIP kernels do: among equal ranking values the lowest flat index wins, where
-0.0 and +0.0 are equal and every NaN ranks above +inf (as torch.topk orders them).
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F


# ---------------------------------------------------------------------------
# ranking keys
# ---------------------------------------------------------------------------

def ranking_key_u32(x: torch.Tensor) -> np.ndarray:
    """Order-preserving unsigned key of a float tensor (flattened).

    key(a) > key(b)  <=>  a ranks above b under torch.topk's ordering
    (activations.py:28): ascending float order, -0.0 == +0.0, NaN above +inf.
    bf16/fp16 inputs are widened to fp32 first (exact), so one 32-bit key law
    covers every dtype.
    """
    xf = x.detach().to(torch.float32).reshape(-1).contiguous()
    bits = xf.numpy().view(np.uint32).copy()
    nan = np.isnan(xf.numpy())
    bits[bits == np.uint32(0x80000000)] = np.uint32(0)  # -0.0 -> +0.0
    neg = (bits >> np.uint32(31)).astype(bool)
    key = np.where(neg, ~bits, bits | np.uint32(0x80000000)).astype(np.uint32)
    key[nan] = np.uint32(0xFFFFFFFF)
    return key


def _select_flat(key: np.ndarray, k_total: int) -> np.ndarray:
    """Flat indices of the k_total largest keys, ties to the lowest index."""
    if k_total <= 0:
        return np.zeros(0, dtype=np.int64)
    # stable ascending sort of the inverted key = descending key, ties by index
    order = np.argsort(~key, kind="stable")
    return order[:k_total]


# ---------------------------------------------------------------------------
# activations  (reference clt/models/activations.py)
# ---------------------------------------------------------------------------

def batchtopk_mask(x: torch.Tensor, k_per_token: int,
                   x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
    """BatchTopK._compute_mask (activations.py:11-36).

    k_total = min(k * B, numel) survivors over the whole flattened block,
    ranked on ``x_for_ranking`` when given, else on ``x``; k <= 0 or an empty
    tensor gives an all-False mask.
    """
    B = x.size(0)
    if k_per_token <= 0 or x.numel() == 0:
        return torch.zeros_like(x, dtype=torch.bool)
    k_total = min(int(k_per_token) * B, x.numel())
    rank = x_for_ranking if x_for_ranking is not None else x
    idx = _select_flat(ranking_key_u32(rank), k_total)
    mask = np.zeros(x.numel(), dtype=bool)
    mask[idx] = True
    return torch.from_numpy(mask).view(x.shape)


def batchtopk_mask_topk(x: torch.Tensor, k_per_token: int,
                        x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The same mask through the reference's own op sequence - torch.topk(sorted=False)
    then an index write (activations.py:21-32).  Ties fall wherever torch.topk puts them,
    so this variant is used for the timed CPU baseline only, never as the parity checker."""
    B = x.size(0)
    if k_per_token <= 0 or x.numel() == 0:
        return torch.zeros_like(x, dtype=torch.bool)
    k_total = min(int(k_per_token) * B, x.numel())
    rank = x_for_ranking if x_for_ranking is not None else x
    _, idx = torch.topk(rank.reshape(-1), k_total, sorted=False)
    mask = torch.zeros(x.numel(), dtype=torch.bool)
    mask[idx] = True
    return mask.view_as(x)


def batchtopk_forward(x: torch.Tensor, k: float, x_for_ranking: Optional[torch.Tensor] = None,
                      timed_baseline: bool = False) -> torch.Tensor:
    """BatchTopK.forward (activations.py:39-65): x * mask, negatives kept."""
    fn = batchtopk_mask_topk if timed_baseline else batchtopk_mask
    mask = fn(x, int(k), x_for_ranking)
    return x * mask.to(x.dtype)


def tokentopk_k(k_float: float, f_total: int) -> int:
    """k rule of TokenTopK._compute_mask (activations.py:108-116).

    0 < k < 1 is a fraction of the row (rounded up, computed in fp32 like the
    reference's torch.tensor(k * F)), k >= 1 is an integer count, k <= 0 keeps
    nothing; always capped at the row length.
    """
    if f_total == 0 or k_float <= 0:
        return 0
    if k_float < 1:
        kk = int(math.ceil(float(np.float32(k_float * f_total))))
    else:
        kk = int(k_float)
    return min(kk, f_total)


def tokentopk_mask(x: torch.Tensor, k_float: float,
                   x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
    """TokenTopK._compute_mask (activations.py:99-128): row-wise top-k."""
    if x.numel() == 0:
        return torch.zeros_like(x, dtype=torch.bool)
    n_rows, f_total = x.shape
    kk = tokentopk_k(k_float, f_total)
    if kk <= 0:
        return torch.zeros_like(x, dtype=torch.bool)
    rank = x_for_ranking if x_for_ranking is not None else x
    key = ranking_key_u32(rank).reshape(n_rows, f_total)
    mask = np.zeros((n_rows, f_total), dtype=bool)
    for r in range(n_rows):
        mask[r, _select_flat(key[r], kk)] = True
    return torch.from_numpy(mask)


def tokentopk_forward(x: torch.Tensor, k: float,
                      x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
    """TokenTopK.forward (activations.py:131-156)."""
    return x * tokentopk_mask(x, k, x_for_ranking).to(x.dtype)


def jumprelu_forward(x: torch.Tensor, threshold: torch.Tensor) -> torch.Tensor:
    """JumpReLU.forward (activations.py:177-180): (x >= theta).float() * x.

    The product is fp32 whatever the input dtype, as in the reference.
    """
    return (x >= threshold).float() * x


class JumpReLUFunction(torch.autograd.Function):
    """JumpReLU with the reference's backward (activations.py:175-220): the input gradient passes
    where input >= threshold; the threshold gradient is grad_output * (-input / bandwidth) on the
    elements with |input - threshold| <= bandwidth / 2, summed over the leading dimensions that the
    threshold does not have."""

    @staticmethod
    def forward(ctx, x, threshold, bandwidth):
        ctx.save_for_backward(x, threshold)
        ctx.bandwidth = bandwidth
        return (x >= threshold).to(x.dtype) * x

    @staticmethod
    def backward(ctx, grad_output):
        x, threshold = ctx.saved_tensors
        grad_x = grad_output * (x >= threshold).type_as(grad_output)
        near = torch.abs(x - threshold) <= (ctx.bandwidth / 2.0)
        per_element = grad_output * ((-x / ctx.bandwidth) * near.type_as(x))
        extra = per_element.dim() - threshold.dim()
        grad_t = per_element.sum(dim=tuple(range(extra))) if extra > 0 else per_element
        return grad_x, grad_t.reshape(threshold.shape), None


def theta_from_log(log_threshold_row: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """ThetaManager.jumprelu's threshold (theta.py:78): exp, then cast to the
    model dtype *before* the comparison."""
    return torch.exp(log_threshold_row).to(dtype)


# ---------------------------------------------------------------------------
# encoder  (reference clt/models/encoder.py:54-131, parallel.py:282-294)
# ---------------------------------------------------------------------------

def encoder_preactivations(x: torch.Tensor, weight: torch.Tensor,
                           bias: Optional[torch.Tensor]) -> torch.Tensor:
    """pre = x . W^T + b with W [F, d_model] (parallel.py:286); a 3-D input is
    flattened to [B*S, d_model] first (encoder.py:67-75)."""
    if x.dim() == 3:
        x = x.reshape(-1, x.shape[-1])
    return F.linear(x, weight, bias)


# ---------------------------------------------------------------------------
# global BatchTopK / TokenTopK helper  (activations.py:229-357, 360-491)
# ---------------------------------------------------------------------------

def zscore_for_ranking(pre: torch.Tensor) -> torch.Tensor:
    """Per-feature z-score used for ranking only (activations.py:281-283):
    (x - mean_0) / (std_0 + 1e-6) with the unbiased std over the batch axis,
    every intermediate kept in the tensor's own dtype."""
    mean = pre.mean(dim=0, keepdim=True)
    std = pre.std(dim=0, keepdim=True)
    return (pre - mean) / (std + 1e-6)


def global_batchtopk(preacts: Dict[int, torch.Tensor], num_layers: int,
                     k: int, timed_baseline: bool = False) -> Dict[int, torch.Tensor]:
    """_apply_batch_topk_helper at world_size 1 (activations.py:261-357).

    Layers are concatenated in range(num_layers) order to [T, sum F], the
    ranking tensor is the per-layer z-score, k*T survivors are taken over the
    whole block, the mask multiplies the raw values.
    """
    layers = [l for l in range(num_layers) if l in preacts]
    if not layers:
        return {}
    orig = torch.cat([preacts[l] for l in layers], dim=1)
    norm = torch.cat([zscore_for_ranking(preacts[l]) for l in layers], dim=1)
    mask = (batchtopk_mask_topk if timed_baseline else batchtopk_mask)(orig, int(k), norm)
    act = orig * mask.to(orig.dtype)
    out, off = {}, 0
    for l in layers:
        f = preacts[l].shape[1]
        out[l] = act[:, off:off + f]
        off += f
    return out


def global_tokentopk(preacts: Dict[int, torch.Tensor], num_layers: int,
                     k: float) -> Dict[int, torch.Tensor]:
    """_apply_token_topk_helper at world_size 1 (activations.py:391-491)."""
    layers = [l for l in range(num_layers) if l in preacts]
    if not layers:
        return {}
    orig = torch.cat([preacts[l] for l in layers], dim=1)
    norm = torch.cat([zscore_for_ranking(preacts[l]) for l in layers], dim=1)
    mask = tokentopk_mask(orig, float(k), norm)
    act = orig * mask.to(orig.dtype)
    out, off = {}, 0
    for l in layers:
        f = preacts[l].shape[1]
        out[l] = act[:, off:off + f]
        off += f
    return out


# ---------------------------------------------------------------------------
# decoder  (reference clt/models/decoder.py:176-340, parallel.py:335-383)
# ---------------------------------------------------------------------------

def _affine_on_nonzero(a: torch.Tensor, offset: Optional[torch.Tensor],
                       scale: Optional[torch.Tensor]) -> torch.Tensor:
    """decoder.py:228-245 / 268-285: (a + offset[f]) * scale[f] on the non-zero
    entries only, offset first, each step rounded in the tensor dtype."""
    if offset is None and scale is None:
        return a
    nz = a != 0
    if not bool(nz.any()):
        return a
    a = a.clone()
    rows, cols = nz.nonzero(as_tuple=True)
    if offset is not None:
        a[rows, cols] += offset[cols]
    if scale is not None:
        a[rows, cols] *= scale[cols]
    return a


def decode(acts: Dict[int, torch.Tensor], layer_idx: int, *, tying: str,
           weights: Dict[str, torch.Tensor], biases: Dict[str, torch.Tensor],
           d_model: int, num_features: int, dtype: torch.dtype,
           feature_offset: Optional[List[torch.Tensor]] = None,
           feature_scale: Optional[List[torch.Tensor]] = None,
           skip_weights: Optional[Dict[str, torch.Tensor]] = None,
           source_inputs: Optional[Dict[int, torch.Tensor]] = None) -> torch.Tensor:
    """Decoder.decode (decoder.py:176-340).

    ``weights`` / ``biases`` are keyed like the reference's module names:
    "s->t" for untied decoders, "i" for tied ones; each weight is stored
    [d_model, F] (parallel.py:66-70).  The cross-source sum runs in ``dtype``
    exactly as the reference does (decoder.py:206, 316); the bias is added
    once per decoder call (parallel.py:380-381).
    """
    keys = sorted(acts.keys())
    if not keys:
        return torch.zeros((0, d_model), dtype=dtype)
    batch = 0
    for kk in keys:
        if acts[kk].numel() > 0:
            batch = acts[kk].shape[0]
            break
    rec = torch.zeros((batch, d_model), dtype=dtype)

    def usable(s):
        if s not in acts:
            return None
        a = acts[s].to(dtype)
        if a.numel() == 0 or a.shape[-1] != num_features:
            return None
        return a

    if tying == "per_target":
        summed = torch.zeros((batch, num_features), dtype=dtype)
        for s in range(layer_idx + 1):
            a = usable(s)
            if a is None:
                continue
            off = feature_offset[layer_idx] if feature_offset is not None else None
            sc = feature_scale[layer_idx] if feature_scale is not None else None
            summed += _affine_on_nonzero(a, off, sc)
        rec = F.linear(summed, weights[str(layer_idx)]) + biases[str(layer_idx)]
    else:
        for s in range(layer_idx + 1):
            a = usable(s)
            if a is None:
                continue
            if tying == "per_source":
                off = feature_offset[layer_idx] if feature_offset is not None else None
                sc = feature_scale[layer_idx] if feature_scale is not None else None
                a = _affine_on_nonzero(a, off, sc)
                name = str(s)
            else:
                name = f"{s}->{layer_idx}"
            dec = F.linear(a, weights[name]) + biases[name]
            if (tying == "none" and skip_weights is not None and source_inputs is not None
                    and s in source_inputs and f"{s}->{layer_idx}" in skip_weights):
                src = source_inputs[s].to(dtype)
                src2 = src.reshape(-1, src.shape[-1])
                dec = dec + src2 @ skip_weights[f"{s}->{layer_idx}"].T
            rec = rec + dec
    if tying in ("per_source", "per_target"):
        if (skip_weights is not None and source_inputs is not None
                and layer_idx in source_inputs):
            src = source_inputs[layer_idx].to(dtype)
            src2 = src.reshape(-1, src.shape[-1])
            rec = rec + src2 @ skip_weights[str(layer_idx)].T
    return rec


def decoder_norms(weights: Dict[str, torch.Tensor], num_layers: int,
                  num_features: int, tying: str, dtype: torch.dtype) -> torch.Tensor:
    """Decoder.get_decoder_norms at world_size 1 (decoder.py:374-485):
    norms[s, f] = sqrt(sum over the decoders source s feeds of ||W[:, f]||^2),
    squared norms accumulated in fp32, result cast to the model dtype."""
    out = torch.zeros(num_layers, num_features, dtype=dtype)
    for s in range(num_layers):
        acc = torch.zeros(num_features, dtype=torch.float32)
        if tying == "per_source":
            names = [str(s)]
        elif tying == "per_target":
            names = [str(t) for t in range(s, num_layers)]
        else:
            names = [f"{s}->{t}" for t in range(s, num_layers)]
        for n in names:
            acc += torch.norm(weights[n], dim=0).pow(2).to(torch.float32)
        out[s] = torch.sqrt(acc).to(dtype)
    return out


# ---------------------------------------------------------------------------
# whole forward  (reference clt/models/clt.py:186-277)
# ---------------------------------------------------------------------------

def feature_activations(inputs: Dict[int, torch.Tensor], *, enc_w: List[torch.Tensor],
                        enc_b: List[torch.Tensor], activation_fn: str, dtype: torch.dtype,
                        num_layers: int, k: Optional[float] = None,
                        topk_mode: str = "global",
                        log_threshold: Optional[torch.Tensor] = None,
                        timed_baseline: bool = False) -> Dict[int, torch.Tensor]:
    """get_feature_activations (clt.py:220-277).

    ``topk_mode="per_layer"`` follows the registry's per-layer functions
    (clt/activations/registry.py:43-98): the mask is computed per layer on the
    raw pre-activation.  (In the reference snapshot that mode is routed to
    ``encode`` and ends in the zero fallback, clt.py:227-234 and 135-149; the
    per-layer selection itself is what the registry defines.)
    """
    xs = {l: inputs[l].to(dtype) for l in inputs}
    pre = {l: encoder_preactivations(xs[l], enc_w[l], enc_b[l]) for l in sorted(xs)}
    if activation_fn == "batchtopk":
        if topk_mode == "per_layer":
            return {l: batchtopk_forward(pre[l], float(int(k)), pre[l], timed_baseline) for l in pre}
        return global_batchtopk(pre, num_layers, int(k), timed_baseline)
    if activation_fn == "topk":
        if topk_mode == "per_layer":
            return {l: tokentopk_forward(pre[l], float(k), pre[l]) for l in pre}
        return global_tokentopk(pre, num_layers, float(k))
    if activation_fn == "jumprelu":
        return {l: jumprelu_forward(pre[l], theta_from_log(log_threshold[l], dtype)) for l in pre}
    if activation_fn == "relu":
        return {l: F.relu(pre[l]) for l in pre}
    raise ValueError(activation_fn)


def forward(inputs: Dict[int, torch.Tensor], *, enc_w, enc_b, dec_w, dec_b,
            activation_fn: str, dtype: torch.dtype, num_layers: int, d_model: int,
            num_features: int, tying: str = "none", k: Optional[float] = None,
            topk_mode: str = "global", log_threshold=None, feature_offset=None,
            feature_scale=None, skip_weights=None, timed_baseline: bool = False
            ) -> Tuple[Dict[int, torch.Tensor], Dict[int, torch.Tensor]]:
    """CrossLayerTranscoder.forward (clt.py:186-218); returns (reconstructions,
    activations)."""
    acts = feature_activations(inputs, enc_w=enc_w, enc_b=enc_b, activation_fn=activation_fn,
                               dtype=dtype, num_layers=num_layers, k=k, topk_mode=topk_mode,
                               log_threshold=log_threshold, timed_baseline=timed_baseline)
    recs: Dict[int, torch.Tensor] = {}
    for t in range(num_layers):
        rel = {s: a for s, a in acts.items() if s <= t and a.numel() > 0}
        if t in inputs and rel:
            src = ({s: inputs[s] for s in range(t + 1) if s in inputs}
                   if skip_weights is not None else None)
            recs[t] = decode(rel, t, tying=tying, weights=dec_w, biases=dec_b, d_model=d_model,
                             num_features=num_features, dtype=dtype,
                             feature_offset=feature_offset, feature_scale=feature_scale,
                             skip_weights=skip_weights, source_inputs=src)
        elif t in inputs:
            x = inputs[t]
            b = x.shape[0] * x.shape[1] if x.dim() == 3 else x.shape[0]
            recs[t] = torch.zeros((b, d_model), dtype=dtype)
    return recs, acts


# ---------------------------------------------------------------------------
# post-hoc theta estimation and BatchTopK -> JumpReLU conversion
# ---------------------------------------------------------------------------

def theta_estimate_posthoc(batches: List[Dict[int, torch.Tensor]], *, activation_fn: str, k: float,
                           num_layers: int, num_features: int, dtype: torch.dtype):
    """ThetaManager.estimate_theta_posthoc up to the conversion (theta.py:175-416), for
    batches of pre-activation dicts in which every layer is present with the same token
    count.  Per batch: per-layer mean / unbiased std over the tokens and the z-score
    (theta.py:305-307), the averaged statistics (:314-318), the global BatchTopK / TokenTopK
    gate ranked on the z-score with the raw values kept (:350-391), and
    _update_min_selected_preactivations (:82-173): per feature the minimum of the z-scores where
    the gated activation is positive; where it is finite, sum += min and count += 1.
    Returns (sum, count, avg_means, avg_stds), all [L, F] in ``dtype``."""
    L, F_ = num_layers, num_features
    ssum = torch.zeros((L, F_), dtype=dtype)
    scnt = torch.zeros((L, F_), dtype=dtype)
    mus = torch.zeros((L, F_), dtype=dtype)
    sigmas = torch.zeros((L, F_), dtype=dtype)
    nb = torch.zeros(L, dtype=torch.long)
    for pre in batches:
        orig, norm = [], []
        for l in range(L):
            p = pre[l].to(dtype)
            mean = p.mean(dim=0, keepdim=True)
            std = p.std(dim=0, keepdim=True)
            orig.append(p)
            norm.append((p - mean) / (std + 1e-6))
            mus[l] += mean.squeeze(0)
            sigmas[l] += std.squeeze(0)
            nb[l] += 1
        gating = torch.cat(orig, dim=1)
        ranking = torch.cat(norm, dim=1)
        if activation_fn == "batchtopk":
            gated = batchtopk_forward(gating, float(int(k)), ranking)
        else:
            gated = tokentopk_forward(gating, float(k), ranking)
        for l in range(L):
            z = ranking[:, l * F_:(l + 1) * F_]
            active = gated[:, l * F_:(l + 1) * F_] > 0
            if active.any():
                per_feature_min = torch.where(active, z, torch.full_like(z, float("inf"))).amin(dim=0)
                valid = torch.isfinite(per_feature_min)
                ssum[l, valid] += per_feature_min[valid]
                scnt[l, valid] += 1
    active_batches = nb.unsqueeze(-1).clamp_min(1.0)
    mus /= active_batches
    sigmas /= active_batches
    return ssum, scnt, mus, sigmas


def theta_convert(ssum: torch.Tensor, scnt: torch.Tensor, mus: torch.Tensor, sigmas: torch.Tensor) -> torch.Tensor:
    """ThetaManager.convert_to_jumprelu_inplace at world_size 1 (theta.py:466-573): per layer the
    mean of the finite positive per-feature normalised thetas (fallback 1e-5), un-normalised
    with sigma.clamp_min(1e-6) and mu, clamped below at 1e-7; returns log(theta) [L, F]."""
    theta_raw = torch.zeros_like(ssum)
    for l in range(ssum.shape[0]):
        active = scnt[l] > 0
        per_feature = torch.full_like(ssum[l], float("inf"))
        if active.any():
            per_feature[active] = ssum[l][active] / scnt[l][active].clamp_min(1.0)
        pos = per_feature[torch.isfinite(per_feature) & (per_feature > 0)]
        scalar = pos.mean().item() if pos.numel() > 0 else 1e-5
        theta_raw[l] = scalar * sigmas[l].clamp_min(1e-6) + mus[l]
    theta_raw.clamp_min_(1e-7)
    return torch.log(theta_raw)


# ---------------------------------------------------------------------------
# MSE reconstruction loss and its gradients (torch autograd, as the reference trains)
# ---------------------------------------------------------------------------

def mse_loss_and_gradients(inputs: Dict[int, torch.Tensor], targets: Dict[int, torch.Tensor], *,
                           enc_w: List[torch.Tensor], enc_b: List[torch.Tensor],
                           dec_w: Dict[str, torch.Tensor], dec_b: Dict[str, torch.Tensor],
                           activation_fn: str, num_layers: int, k: Optional[float] = None,
                           theta: Optional[torch.Tensor] = None,
                           masks: Optional[Dict[int, torch.Tensor]] = None, tying: str = "none",
                           log_threshold: Optional[torch.Tensor] = None, bandwidth: float = 1.0,
                           model_dtype: torch.dtype = torch.float32,
                           normalization_method: str = "none", mean_tg: Optional[Dict[int, torch.Tensor]] = None,
                           std_tg: Optional[Dict[int, torch.Tensor]] = None,
                           skip_w: Optional[Dict[str, torch.Tensor]] = None,
                           feature_offset: Optional[List[torch.Tensor]] = None,
                           feature_scale: Optional[List[torch.Tensor]] = None):
    """loss = sum over layers of nn.MSELoss()(prediction', target') (losses.py:45-92; ' = the
    de-normalisation of losses.py:70-86: ``x * std + mean`` for "mean_std" with the target statistics,
    ``x / sqrt(d_model)`` for "sqrt_d_model") through the reference's forward (decoders untied, keys
    "s->t", or tied per source / per target, keys "i", decoder.py:176-340; skip connections
    ``skip_w`` with the same keys, decoder.py:297-338; the target's feature offset / scale on the
    non-zero activations of tied decoders, decoder.py:228-245, 268-285), and d loss / d parameter from
    torch autograd (trainer.py:751): F.linear backward for encoder and decoders, the straight-through
    gate of BatchTopK (activations.py:66-96: grad * mask) or the pass-through part of JumpReLU's backward
    (activations.py:183-220: grad * 1[x >= theta]).  Per-layer selection, fp32.
    ``masks`` (bool [T, F] per layer) replaces the gate computed here, for comparisons in which
    the other side selected on differently rounded pre-activations.
    With ``log_threshold`` ([L, F], the parameter itself) the JumpReLU runs through
    ``JumpReLUFunction`` with threshold = exp(log_threshold) cast to ``model_dtype`` and back
    (theta.py:70-79, bandwidth 1.0 at theta.py:41) and the result holds the gradient of
    "theta_manager.log_threshold" as well.
    Returns (loss, {state-dict key: gradient})."""
    L = num_layers
    params: Dict[str, torch.Tensor] = {}

    def param(name, t):
        params[name] = t.detach().float().clone().requires_grad_(True)
        return params[name]

    if log_threshold is not None:
        param("theta_manager.log_threshold", log_threshold)
    for l in range(L):
        param(f"encoder_module.encoders.{l}.weight", enc_w[l])
        param(f"encoder_module.encoders.{l}.bias_param", enc_b[l])
    for name in dec_w:
        param(f"decoder_module.decoders.{name}.weight", dec_w[name])
        param(f"decoder_module.decoders.{name}.bias_param", dec_b[name])
    for name, w in (skip_w or {}).items():
        param(f"decoder_module.skip_weights.{name}", w)
    for i, v in enumerate(feature_offset or []):
        param(f"decoder_module.feature_offset.{i}", v)
    for i, v in enumerate(feature_scale or []):
        param(f"decoder_module.feature_scale.{i}", v)
    acts = {}
    for l in range(L):
        pre = F.linear(inputs[l].float(), params[f"encoder_module.encoders.{l}.weight"],
                       params[f"encoder_module.encoders.{l}.bias_param"])
        if log_threshold is not None and activation_fn == "jumprelu":
            thr = torch.exp(params["theta_manager.log_threshold"][l]).to(model_dtype).float()
            acts[l] = JumpReLUFunction.apply(pre, thr, bandwidth)
            continue
        if masks is not None:
            mask = masks[l]
        elif activation_fn == "batchtopk":
            mask = batchtopk_mask(pre.detach(), int(k), pre.detach())
        elif activation_fn == "jumprelu":
            mask = pre.detach() >= theta[l].float()
        elif activation_fn == "relu":
            mask = pre.detach() > 0
        else:
            raise ValueError(activation_fn)
        acts[l] = pre * mask.to(pre.dtype)

    def affine(a, t):
        # the target's offset and scale act on the selected (non-zero) entries only (decoder.py:228-245)
        if feature_offset is None and feature_scale is None:
            return a
        nz = (a.detach() != 0).to(a.dtype)
        if feature_offset is not None:
            a = a + params[f"decoder_module.feature_offset.{t}"] * nz
        if feature_scale is not None:
            a = a * (params[f"decoder_module.feature_scale.{t}"] * nz + (1 - nz))
        return a

    loss = torch.zeros((), dtype=torch.float32)
    for t in range(L):
        rec = torch.zeros_like(targets[t], dtype=torch.float32)
        if tying == "per_target":      # one decoder per target over the summed activations, bias once
            summed = sum(affine(acts[s_], t) for s_ in range(t + 1))
            rec = F.linear(summed, params[f"decoder_module.decoders.{t}.weight"],
                           params[f"decoder_module.decoders.{t}.bias_param"])
        else:
            for s_ in range(t + 1):
                key = f"{s_}->{t}" if tying == "none" else str(s_)
                a = affine(acts[s_], t) if tying == "per_source" else acts[s_]
                rec = rec + F.linear(a, params[f"decoder_module.decoders.{key}.weight"],
                                     params[f"decoder_module.decoders.{key}.bias_param"])
                if skip_w is not None and tying == "none":
                    rec = rec + inputs[s_].float() @ params[f"decoder_module.skip_weights.{key}"].T
        if skip_w is not None and tying != "none":
            rec = rec + inputs[t].float() @ params[f"decoder_module.skip_weights.{t}"].T
        tgt = targets[t].float()
        if normalization_method == "mean_std" and mean_tg is not None and std_tg is not None and t in mean_tg and t in std_tg:
            rec = rec * std_tg[t].float() + mean_tg[t].float()
            tgt = tgt * std_tg[t].float() + mean_tg[t].float()
        elif normalization_method == "sqrt_d_model":
            rec = rec / (rec.shape[-1] ** 0.5)
            tgt = tgt / (tgt.shape[-1] ** 0.5)
        loss = loss + F.mse_loss(rec, tgt)
    loss.backward()
    return loss.detach(), {name: p.grad for name, p in params.items()}


# ---------------------------------------------------------------------------
# evaluation reductions
# ---------------------------------------------------------------------------

def sparsity_metrics(acts: Dict[int, torch.Tensor], num_features: int, num_layers: int) -> Dict[str, object]:
    """L0 per layer and its aggregates (reference clt/training/evaluator.py:194-244)."""
    if not acts or not any(v.numel() > 0 for v in acts.values()):
        return {"sparsity/total_l0": 0.0, "sparsity/avg_l0": 0.0, "sparsity/sparsity_fraction": 1.0,
                "layerwise/l0": {f"layer_{i}": 0.0 for i in range(num_layers)}}
    per_layer, total, valid = {}, 0.0, 0
    for l, a in acts.items():
        if a.numel() == 0 or a.shape[0] == 0:
            per_layer[f"layer_{l}"] = 0.0
            continue
        v = (a != 0).float().sum(dim=-1).mean().item()
        per_layer[f"layer_{l}"] = v
        total += v
        valid += 1
    avg = total / valid if valid > 0 else 0.0
    frac = 1.0 - (avg / num_features) if num_features > 0 else 1.0
    return {"sparsity/total_l0": total, "sparsity/avg_l0": avg, "sparsity/sparsity_fraction": max(0.0, min(1.0, frac)),
            "layerwise/l0": per_layer}


def feature_density_metrics(acts: Dict[int, torch.Tensor]) -> Dict[str, object]:
    """log10 firing density and the activation-count heuristic per feature
    (reference clt/training/evaluator.py:350-405, _log_density :71-74)."""
    if not acts or not any(v.numel() > 0 for v in acts.values()):
        return {"layerwise/log_feature_density": {}, "layerwise/consistent_activation_heuristic": {}}
    dens, heur = {}, {}
    for l, a in acts.items():
        if a.numel() == 0 or a.shape[0] == 0:
            continue
        fired = (a > 1e-6).float()
        dens[f"layer_{l}"] = torch.log10(fired.mean(dim=0) + 1e-10).tolist()
        heur[f"layer_{l}"] = (fired.sum(dim=0) / (fired.any(dim=0).float() + 1e-9)).tolist()
    return {"layerwise/log_feature_density": dens, "layerwise/consistent_activation_heuristic": heur}


def dead_feature_update(passes_since_fired: torch.Tensor, acts: Dict[int, torch.Tensor]) -> torch.Tensor:
    """New value of the per-feature counters after one batch (reference clt/training/trainer.py:693-712)."""
    n = passes_since_fired.clone()
    for l, a in acts.items():
        if l < n.shape[0] and a.numel() > 0:
            fired = (a > 1e-6).any(dim=0)
            if fired.shape[0] == n.shape[1]:
                n[l] += 1
                n[l][fired] = 0
    return n


def reconstruction_metrics(targets: Dict[int, torch.Tensor], recs: Dict[int, torch.Tensor], *, method: str = "none",
                           mean_tg: Optional[Dict[int, torch.Tensor]] = None,
                           std_tg: Optional[Dict[int, torch.Tensor]] = None,
                           d_model: Optional[int] = None) -> Dict[str, object]:
    """Explained variance and normalised MSE (reference clt/training/evaluator.py:246-345)."""
    mean_tg, std_tg = mean_tg or {}, std_tg or {}
    tot_ev, tot_nmse, n = 0.0, 0.0, 0
    lw_nmse, lw_ev = {}, {}
    for l, tgt in targets.items():
        if l not in recs:
            continue
        rec = recs[l]
        if method == "mean_std" and l in mean_tg and l in std_tg:
            mean, std = mean_tg[l].to(rec.dtype), std_tg[l].to(rec.dtype)
            tgt, rec = tgt * std + mean, rec * std + mean
        elif method == "sqrt_d_model" and d_model is not None:
            tgt, rec = tgt / (d_model ** 0.5), rec / (d_model ** 0.5)
        tf = tgt.reshape(-1, tgt.shape[-1]).float()
        rf = rec.reshape(-1, rec.shape[-1]).float()
        if tf.shape != rf.shape or tf.numel() == 0:
            continue
        mse = F.mse_loss(rf, tf, reduction="mean").item()
        tvar = torch.var(tf, dim=0, unbiased=False).mean().item()
        evar = torch.var(tf - rf, dim=0, unbiased=False).mean().item()
        ev = (1.0 - evar / tvar) if tvar > 1e-9 else (1.0 if evar < 1e-9 else 0.0)
        nmse = (mse / tvar) if tvar > 1e-9 else (0.0 if mse < 1e-9 else float("inf"))
        tot_ev += ev
        tot_nmse += nmse
        lw_nmse[f"layer_{l}"] = nmse
        lw_ev[f"layer_{l}"] = ev
        n += 1
    avg_ev = tot_ev / n if n > 0 else 0.0
    return {"reconstruction/explained_variance": max(0.0, min(1.0, avg_ev)),
            "reconstruction/normalized_mean_reconstruction_error": tot_nmse / n if n > 0 else 0.0,
            "layerwise/normalized_mse": lw_nmse, "layerwise/explained_variance": lw_ev}


# ---------------------------------------------------------------------------
# activation-store batch assembly
# ---------------------------------------------------------------------------

def store_parse_batch(idxs: np.ndarray, fetch_slice, *, num_layers: int, d_model: int, dtype: torch.dtype,
                      method: str = "none", mean_in=None, std_in=None, mean_tg=None, std_tg=None):
    """Inputs and targets of one batch from (chunk, row) indices (reference
    clt/training/data/manifest_activation_store.py:776-958, without the retry loop).
    ``fetch_slice(chunk_id, sorted_rows)`` returns Layer0_Inputs | Layer0_Targets | Layer1_Inputs | ...
    for the sorted rows; ``mean_*`` / ``std_*`` map layer -> fp32 [1, d] (std already + 1e-6)."""
    mean_in, std_in, mean_tg, std_tg = mean_in or {}, std_in or {}, mean_tg or {}, std_tg or {}
    itemsize = torch.finfo(dtype).bits // 8
    bytes_per_row = d_model * itemsize
    unique_chunks, inverse = np.unique(idxs[:, 0], return_inverse=True)
    rows_by_chunk = {int(c): idxs[inverse == i, 1] for i, c in enumerate(unique_chunks)}
    ins: Dict[int, List[torch.Tensor]] = {l: [] for l in range(num_layers)}
    tgs: Dict[int, List[torch.Tensor]] = {l: [] for l in range(num_layers)}
    for chunk_id, rows in rows_by_chunk.items():
        sorted_rows = np.sort(rows)
        raw = fetch_slice(chunk_id, sorted_rows)
        assert len(raw) == len(sorted_rows) * bytes_per_row * 2 * num_layers
        n = len(rows)
        per_tensor = n * bytes_per_row
        reorder = torch.as_tensor(np.searchsorted(sorted_rows, rows), dtype=torch.long)
        for l in range(num_layers):
            a = l * 2 * per_tensor
            inp = torch.frombuffer(bytearray(raw[a:a + per_tensor]), dtype=dtype).reshape(n, d_model)
            tgt = torch.frombuffer(bytearray(raw[a + per_tensor:a + 2 * per_tensor]), dtype=dtype).reshape(n, d_model)
            ins[l].append(inp[reorder])
            tgs[l].append(tgt[reorder])
    inputs = {l: torch.cat(v) for l, v in ins.items()}
    targets = {l: torch.cat(v) for l, v in tgs.items()}
    if method in ("mean_std", "sqrt_d_model"):
        for l in range(num_layers):
            x, t = inputs[l].float(), targets[l].float()
            if method == "mean_std":
                if l in mean_in and l in std_in:
                    x = (x - mean_in[l]) / std_in[l]
                if l in mean_tg and l in std_tg:
                    t = (t - mean_tg[l]) / std_tg[l]
            else:
                x, t = x * math.sqrt(d_model), t * math.sqrt(d_model)
            inputs[l], targets[l] = x.to(dtype), t.to(dtype)
    return inputs, targets


# ---------------------------------------------------------------------------
# float64 references used to pin the torch restatements above
# ---------------------------------------------------------------------------

def affine_f64(x: np.ndarray, w: np.ndarray, b: Optional[np.ndarray]) -> np.ndarray:
    """x . w^T + b in float64 (w is [out, in])."""
    y = x.astype(np.float64) @ w.astype(np.float64).T
    if b is not None:
        y = y + b.astype(np.float64)
    return y


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    """||a - b|| / ||b|| in float64 (0 when both are all-zero)."""
    a64 = a.detach().to(torch.float64).cpu()
    b64 = b.detach().to(torch.float64).cpu()
    den = float(torch.linalg.vector_norm(b64))
    num = float(torch.linalg.vector_norm(a64 - b64))
    if den == 0.0:
        return 0.0 if num == 0.0 else float("inf")
    return num / den
