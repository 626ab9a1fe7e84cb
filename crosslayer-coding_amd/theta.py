"""JumpReLU threshold holder.

Keeps the reference's parameter (``theta_manager.log_threshold`` [L, F], initialised to
log(jumprelu_threshold), clt/models/theta.py:50-61) and its ``jumprelu(x, layer)`` call
(theta.py:70-79): theta = exp(log_threshold[layer]) rounded to the model dtype, then
``x >= theta`` keeps x.

Post-hoc theta estimation (theta.py:175-430) runs, per batch, the global top-k selection on
the device (column statistics, selection ranked on the z-score, per-feature minimum of the
selected z-scores: three kernel groups, nothing dense besides the pre-activations the caller's
encoder produced) and keeps the reference's running buffers; the BatchTopK->JumpReLU
conversion (theta.py:432-636) is a one-off computation on [L, F] tensors.
"""

from __future__ import annotations

import logging
from typing import Callable, Dict, List, Optional, Tuple, cast

import torch
import torch.nn as nn

from . import engine
from .activations import JumpReLU, resolve_token_k
from .parallel import mark_replicated, require_single_rank

logger = logging.getLogger(__name__)


class ThetaManager(nn.Module):
    log_threshold: Optional[nn.Parameter]

    def __init__(self, config, process_group, device: torch.device, dtype: torch.dtype):
        super().__init__()
        require_single_rank(process_group)
        self.config = config
        self.process_group = process_group
        self.device = device
        self.dtype = dtype
        self.bandwidth = 1.0
        self.world_size, self.rank = 1, 0
        if config.activation_fn == "jumprelu":
            if config.jumprelu_threshold == 0:
                logger.warning(
                    f"Rank {self.rank}: jumprelu_threshold is 0, expecting to load log_threshold from checkpoint.")
            log_t = torch.log(torch.tensor(config.jumprelu_threshold, device=device, dtype=dtype))
            init = torch.ones(config.num_layers, config.num_features, device=device, dtype=dtype) * log_t
            self.log_threshold = nn.Parameter(init)
            mark_replicated(self.log_threshold)
        else:
            self.log_threshold = None
        for name in ("_sum_min_selected_preact", "_count_min_selected_preact", "_avg_layer_means",
                     "_avg_layer_stds", "_processed_batches_for_stats"):
            self.register_buffer(name, None, persistent=False)

    def thresholds(self, dtype: torch.dtype) -> torch.Tensor:
        """exp(log_threshold) for all layers, rounded to ``dtype``: [L, F], contiguous."""
        assert self.log_threshold is not None
        th = torch.exp(self.log_threshold.detach())
        return th.to(dtype).contiguous()

    def jumprelu(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor:
        if self.log_threshold is None:
            logger.error(f"Rank {self.rank}: log_threshold not initialized for JumpReLU. Returning input.")
            return x.to(device=self.device, dtype=self.dtype)
        if layer_idx >= self.log_threshold.shape[0]:
            logger.error(f"Rank {self.rank}: Invalid layer_idx {layer_idx} for log_threshold. Returning input.")
            return x.to(device=self.device, dtype=self.dtype)
        theta = torch.exp(self.log_threshold[layer_idx])
        theta = theta.to(device=self.device, dtype=self.dtype)
        return cast(torch.Tensor, JumpReLU.apply(x, theta, self.bandwidth))

    # ---- post-hoc estimation ----------------------------------------------------------------
    def _reset_estimation_buffers(self) -> None:
        L, F = self.config.num_layers, self.config.num_features
        for name in ("_sum_min_selected_preact", "_count_min_selected_preact", "_avg_layer_means", "_avg_layer_stds"):
            buf = getattr(self, name, None)
            if buf is None:
                setattr(self, name, torch.zeros((L, F), dtype=self.dtype, device=self.device))
            else:
                buf.data.zero_()
        if getattr(self, "_processed_batches_for_stats", None) is None:
            self._processed_batches_for_stats = torch.zeros(L, dtype=torch.long, device=self.device)
        else:
            self._processed_batches_for_stats.data.zero_()

    def _batch_slab(self, pre: Dict[int, torch.Tensor]) -> Optional[Tuple[torch.Tensor, List[int]]]:
        """[L, T, F] pre-activations of one batch with the reference's zero filling (theta.py:268-331):
        absent layers, empty tensors and tensors with another token count count as zeros and do not
        enter the averaged statistics.  Returns (slab, layers that do enter them)."""
        L, F = self.config.num_layers, self.config.num_features
        first = next((p for p in pre.values() if p.numel() > 0), None)
        if first is None:
            return None
        T = first.shape[0]
        good = [l for l in range(L) if l in pre and pre[l].numel() > 0 and pre[l].shape[0] == T and pre[l].shape[1] == F]
        for l in range(L):
            if l in pre and pre[l].numel() > 0 and pre[l].shape[0] != T:
                logger.warning(f"Rank {self.rank} Layer {l}: Mismatched token dim (expected {T}, got {pre[l].shape[0]}). Using zeros.")
        if len(good) == L:
            from .encoder import _as_slab
            return _as_slab([pre[l].to(device=self.device, dtype=self.dtype) for l in range(L)]), good
        slab = torch.zeros((L, T, F), dtype=self.dtype, device=self.device)
        for l in good:
            slab[l] = pre[l]
        return slab, good

    @torch.no_grad()
    def estimate_theta_posthoc(
        self,
        encode_all_layers_fn: Callable[[Dict[int, torch.Tensor]], Tuple[Dict[int, torch.Tensor], list]],
        data_iter,
        num_batches: Optional[int] = None,
        default_theta_value: float = 1e6,
    ) -> torch.Tensor:
        """Estimate theta post-hoc using a specified number of batches (theta.py:175-430)."""
        logger.info(f"Rank {self.rank}: Starting post-hoc theta estimation on device {self.device}.")
        self._reset_estimation_buffers()
        cfg = self.config
        ws = engine.Workspace(self.device)
        processed = 0
        for inputs_batch, _ in data_iter:
            if num_batches is not None and processed >= num_batches:
                break
            inputs = {k: v.to(device=self.device, dtype=self.dtype) for k, v in inputs_batch.items()}
            pre_dict, _ = encode_all_layers_fn(inputs)
            if not pre_dict:
                logger.warning(f"Rank {self.rank}: No preactivations. Skipping batch {processed + 1}.")
                processed += 1
                continue
            got = self._batch_slab(pre_dict)
            if got is None:
                logger.warning(f"Rank {self.rank}: All preactivations empty. Skipping batch {processed + 1}.")
                processed += 1
                continue
            slab, good = got
            L, T, F = slab.shape
            mean, std, denom = engine.colstats_full(slab)
            # averaged normalisation statistics, accumulated in the model dtype (theta.py:314-318)
            sel = slice(None) if len(good) == L else torch.tensor(good, device=self.device)
            self._avg_layer_means.data[sel] += mean[sel].to(self.dtype)
            self._avg_layer_stds.data[sel] += std[sel].to(self.dtype)
            self._processed_batches_for_stats.data[sel] += 1
            if len(good) < L:   # zero-filled layers rank on zeros: mean 0, denominator std 1 + 1e-6 (theta.py:281-282)
                bad = [l for l in range(L) if l not in good]
                mean[bad] = 0.0
                denom[bad] = (torch.ones((), dtype=self.dtype, device=self.device) + 1e-6).float()
            if cfg.activation_fn == "batchtopk":
                k = int(cfg.batchtopk_k) if cfg.batchtopk_k is not None else L * F
                surv = engine.batchtopk_select(slab, k, True, ws, stats=(mean, denom))
            elif cfg.activation_fn == "topk":
                if getattr(cfg, "topk_k", None) is None:
                    logger.error(f"Rank {self.rank}: 'topk_k' not found in config for 'topk' activation during theta "
                                 "estimation. Defaulting to all features for this batch.")
                    kk = L * F
                else:
                    kk = resolve_token_k(float(cfg.topk_k), L * F)
                surv = engine.tokentopk_select(slab, kk, True, ws, stats=(mean, denom))
            else:
                logger.error(f"Rank {self.rank}: Unsupported activation_fn '{cfg.activation_fn}' for theta estimation. "
                             "Cannot determine gating mechanism. Using zeros for activated_concatenated_posthoc.")
                surv = None
            if surv is not None:
                engine.selected_min_accumulate(surv, mean, denom, self._sum_min_selected_preact,
                                               self._count_min_selected_preact, ws)
            processed += 1
        logger.info(f"Rank {self.rank}: Processed {processed} batches for theta estimation and stats accumulation.")
        active = self._processed_batches_for_stats.data.unsqueeze(-1).clamp_min(1.0)
        self._avg_layer_means.data /= active
        self._avg_layer_stds.data /= active
        self.convert_to_jumprelu_inplace(default_theta_value=default_theta_value)
        logger.info(f"Rank {self.rank}: Post-hoc theta estimation and conversion to JumpReLU complete.")
        if self.log_threshold is not None:
            return torch.exp(self.log_threshold.data)
        return torch.empty(0, device=self.device, dtype=self.dtype)

    @torch.no_grad()
    def convert_to_jumprelu_inplace(self, default_theta_value: float = 1e6) -> None:
        """BatchTopK / TokenTopK -> JumpReLU from the estimated statistics (theta.py:432-636): per layer,
        the mean of the positive per-feature normalised thetas is un-normalised with the averaged
        per-feature mean and std."""
        cfg = self.config
        if cfg.activation_fn not in ["batchtopk", "topk"]:
            logger.warning(f"Rank {self.rank}: Model original activation_fn was {cfg.activation_fn}, not batchtopk or topk. "
                           "Skipping conversion to JumpReLU based on learned thetas.")
            if cfg.activation_fn == "relu":
                logger.error(f"Rank {self.rank}: Model is ReLU, cannot convert to JumpReLU via learned thetas.")
            return
        for name in ("_sum_min_selected_preact", "_count_min_selected_preact", "_avg_layer_means", "_avg_layer_stds"):
            if getattr(self, name, None) is None:
                raise RuntimeError(
                    f"Rank {self.rank}: Required buffer {name} for JumpReLU conversion not found or not populated. "
                    "Run estimate_theta_posthoc() with appropriate settings before converting.")
        theta_sum, theta_cnt = self._sum_min_selected_preact.clone(), self._count_min_selected_preact.clone()
        mus, sigmas = self._avg_layer_means.clone(), self._avg_layer_stds.clone()
        theta_raw = torch.zeros_like(theta_sum)
        fallback_norm_theta = 1e-5
        for l in range(cfg.num_layers):
            active = theta_cnt[l] > 0
            per_feature = torch.full_like(theta_sum[l], float("inf"))
            if active.any():
                per_feature[active] = theta_sum[l][active] / theta_cnt[l][active].clamp_min(1.0)
            pos = per_feature[torch.isfinite(per_feature) & (per_feature > 0)]
            if pos.numel() > 0:
                scalar = pos.mean().item()
                logger.info(f"Rank {self.rank} Layer {l}: Derived normalized theta (scalar, mean of positive active "
                            f"features) = {scalar:.4e}")
            else:
                scalar = fallback_norm_theta
                logger.warning(f"Rank {self.rank} Layer {l}: No positive, finite per-feature normalized thetas. "
                               f"Using fallback normalized theta = {scalar:.4e}")
            theta_raw[l] = scalar * sigmas[l].clamp_min(1e-6) + mus[l]
        min_final = 1e-7
        clamped = int((theta_raw < min_final).sum().item())
        if clamped > 0:
            logger.warning(f"Rank {self.rank}: Clamping {clamped} final raw theta values below {min_final} to {min_final} "
                           "before taking log.")
            theta_raw.clamp_min_(min_final)
        log_theta = torch.log(theta_raw)
        original = cfg.activation_fn
        cfg.activation_fn = "jumprelu"
        cfg.jumprelu_threshold = 0.0
        if original == "batchtopk":
            cfg.batchtopk_k = None
            cfg.batchtopk_straight_through = False
        elif original == "topk":
            for attr in ("topk_k", "topk_straight_through"):
                if hasattr(cfg, attr):
                    try:
                        delattr(cfg, attr)
                    except AttributeError:
                        setattr(cfg, attr, None)
        if self.log_threshold is None or not isinstance(self.log_threshold, nn.Parameter):
            self.log_threshold = nn.Parameter(log_theta.to(device=self.device, dtype=self.dtype))
        else:
            self.log_threshold.data = log_theta.to(device=self.log_threshold.device, dtype=self.log_threshold.dtype)
        mark_replicated(self.log_threshold)
        logger.info(f"Rank {self.rank}: Model converted to JumpReLU. activation_fn='{cfg.activation_fn}'.")
