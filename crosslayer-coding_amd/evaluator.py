"""Evaluation metrics with the reference evaluator's interface and keys
(clt/training/evaluator.py:28-345), computed from the survivor list.

The reference runs the model twice (``model(inputs)`` and ``get_feature_activations``) and scans
dense ``[T, F]`` tensors per layer; here one forward yields reconstructions and the survivor
list, `clt_survivor_metrics` turns the list into per-layer non-zero counts and per-feature firing
counts, and `clt_reconstruction_stats` reduces targets and reconstructions per layer.  The small
``[L]`` / ``[L, F]`` results are finished with the reference's own formulas.
"""

from __future__ import annotations

import logging
import time
from typing import Any, Dict, List, Optional, Tuple

import numpy as np
import torch

from . import _native as nat
from . import engine
from .engine import SurvivorList

logger = logging.getLogger(__name__)

FIRED_EPS = 1e-6  # evaluator.py:379, trainer.py:704


class DeadFeatureTracker:
    """Per-feature count of batches since the feature last fired, and the mask derived from it
    (Trainer.n_forward_passes_since_fired / dead_neurons_mask, clt/training/trainer.py:342-347,
    441-454, 693-712)."""

    def __init__(self, num_layers: int, num_features: int, dead_feature_window: int, device: torch.device):
        self.dead_feature_window = dead_feature_window
        self.n_forward_passes_since_fired = torch.zeros((num_layers, num_features), dtype=torch.long, device=device)

    def update(self, survivors: SurvivorList, fired: Optional[torch.Tensor] = None) -> None:
        """One batch: counters of the features that fired (value > 1e-6 on any token) go to zero, all
        others go up by one.  ``fired`` may carry the counts of `engine.survivor_metrics` if the caller
        has them already."""
        n = self.n_forward_passes_since_fired
        if survivors.L != n.shape[0] or survivors.F != n.shape[1]:
            logger.warning(f"Shape mismatch for dead neuron update. Survivors: ({survivors.L}, {survivors.F}), "
                           f"Counter: {tuple(n.shape)}. Skipping dead neuron update.")
            return
        if fired is None:
            _, fired = engine.survivor_metrics(survivors.trimmed(), FIRED_EPS)
        engine.dead_feature_update(fired, n)

    @property
    def dead_neurons_mask(self) -> torch.Tensor:
        return (self.n_forward_passes_since_fired > self.dead_feature_window).detach()


class CLTEvaluator:
    """Same constructor, methods and metric keys as the reference's CLTEvaluator (evaluator.py:28-68)."""

    def __init__(self, model, device: torch.device, start_time: Optional[float] = None,
                 mean_tg: Optional[Dict[int, torch.Tensor]] = None, std_tg: Optional[Dict[int, torch.Tensor]] = None,
                 normalization_method: str = "none", d_model: Optional[int] = None):
        self.model = model
        self.device = device
        self.start_time = start_time or time.time()
        self.mean_tg = mean_tg or {}
        self.std_tg = std_tg or {}
        valid = ["none", "mean_std", "sqrt_d_model"]
        if normalization_method not in valid:
            raise ValueError(f"Invalid normalization_method: {normalization_method}. Must be one of {valid}")
        self.normalization_method = normalization_method
        self.d_model = d_model
        self.metrics_history: List[Dict[str, Any]] = []

    # ---- small helpers with the reference's names (evaluator.py:70-97) ----
    @staticmethod
    def _log_density(density: torch.Tensor, eps: float = 1e-10) -> torch.Tensor:
        return torch.log10(density + eps)

    @staticmethod
    def _calculate_aggregate_metric(per_layer_data: Dict[str, List[float]]) -> Optional[float]:
        values: List[float] = []
        for key in per_layer_data:
            values.extend(per_layer_data[key])
        return float(np.mean(values)) if values else None

    @staticmethod
    def _calculate_aggregate_histogram_data(per_layer_data: Dict[str, List[float]]) -> List[float]:
        values: List[float] = []
        for key in per_layer_data:
            values.extend(per_layer_data[key])
        return values

    # ---- from dense activations to the survivor list ----
    def _as_survivors(self, activations) -> Optional[Tuple[List[int], SurvivorList]]:
        """A survivor list plus the layers it covers.  Accepts the list itself (all layers) or the
        reference's ``{layer: dense [T, F]}``, which is compacted on the device."""
        if isinstance(activations, SurvivorList):
            return list(range(activations.L)), activations.trimmed()   # raises for a batch without a valid list
        layers = sorted(l for l, a in activations.items() if a.numel() > 0 and a.shape[0] > 0)
        if not layers:
            return None
        dense = torch.stack([activations[l] for l in layers]).contiguous()
        nat.require_device(dense, "CLTEvaluator")
        return layers, engine.threshold_select(dense, None, nat.PRED_NONZERO)

    def _counts(self, activations, present: Optional[List[int]] = None):
        """(layers, tokens, entries != 0 per layer, firing tokens per (layer, feature)).  ``present``: the
        layers the batch really held, when ``activations`` is a survivor list over all num_layers with
        empty rows for the others: the reference's metrics run over the layers get_feature_activations
        returned (evaluator.py:194-244, 350-405), so the absent ones must not enter the averages."""
        got = self._as_survivors(activations)
        if got is None:
            return None
        layers, surv = got
        nonzero, fired = engine.survivor_metrics(surv, FIRED_EPS)
        if present is not None and list(present) != layers:
            idx = torch.tensor([layers.index(l) for l in present], device=nonzero.device)
            layers, nonzero, fired = list(present), nonzero[idx], fired[idx]
        return layers, surv.T, nonzero, fired

    # ---- metrics (evaluator.py:194-244) ----
    def _compute_sparsity(self, activations, counts=None) -> Dict[str, Any]:
        cfg = self.model.config
        counts = counts if counts is not None else (self._counts(activations) if _has_data(activations) else None)
        if counts is None:
            logger.warning("Warning: Received empty activations for sparsity computation. Returning zeros.")
            return {"sparsity/total_l0": 0.0, "sparsity/avg_l0": 0.0, "sparsity/sparsity_fraction": 1.0,
                    "layerwise/l0": {f"layer_{i}": 0.0 for i in range(cfg.num_layers)}}
        layers, T, nonzero, _ = counts
        # mean over tokens of the per-token count, in fp32 as the reference computes it
        l0 = (nonzero.to(torch.float32) / T).tolist()
        per_layer = {f"layer_{l}": l0[i] for i, l in enumerate(layers)}
        if not isinstance(activations, SurvivorList):
            for l, a in activations.items():
                per_layer.setdefault(f"layer_{l}", 0.0)
        total = float(sum(l0))
        avg = total / len(layers) if layers else 0.0
        F = cfg.num_features
        frac = 1.0 - (avg / F) if F > 0 else 1.0
        return {"sparsity/total_l0": total, "sparsity/avg_l0": avg,
                "sparsity/sparsity_fraction": max(0.0, min(1.0, frac)), "layerwise/l0": per_layer}

    # ---- evaluator.py:350-405 ----
    def _compute_feature_density(self, activations, counts=None) -> Dict[str, Any]:
        counts = counts if counts is not None else (self._counts(activations) if _has_data(activations) else None)
        if counts is None:
            return {"layerwise/log_feature_density": {}, "layerwise/consistent_activation_heuristic": {}}
        layers, T, _, fired = counts
        tokens_active = fired.to(torch.float32)                       # act_bool.sum(dim=0)
        log_density = self._log_density(tokens_active / T).tolist()   # act_bool.mean(dim=0)
        heuristic = (tokens_active / ((fired > 0).float() + 1e-9)).tolist()
        return {"layerwise/log_feature_density": {f"layer_{l}": log_density[i] for i, l in enumerate(layers)},
                "layerwise/consistent_activation_heuristic": {f"layer_{l}": heuristic[i] for i, l in enumerate(layers)}}

    # ---- evaluator.py:246-345 ----
    def _compute_reconstruction_metrics(self, targets: Dict[int, torch.Tensor],
                                        reconstructions: Dict[int, torch.Tensor]) -> Dict[str, Any]:
        layers = [l for l, t in targets.items() if l in reconstructions
                  and t.numel() > 0 and t.reshape(-1, t.shape[-1]).shape == reconstructions[l].reshape(
                      -1, reconstructions[l].shape[-1]).shape]
        layerwise_nmse: Dict[str, float] = {}
        layerwise_ev: Dict[str, float] = {}
        total_ev = total_nmse = 0.0
        if layers:
            rec = torch.stack([reconstructions[l].reshape(-1, reconstructions[l].shape[-1]) for l in layers]).contiguous()
            tgt = torch.stack([targets[l].reshape(-1, targets[l].shape[-1]).to(rec.dtype) for l in layers]).contiguous()
            d = rec.shape[-1]
            mode, mean, std, scale = "none", None, None, 1.0
            if self.normalization_method == "mean_std" and any(l in self.mean_tg and l in self.std_tg for l in layers):
                # layers without statistics keep their values: x * 1 + 0 is exact in every dtype
                mode = "mean_std"
                mean = torch.zeros((len(layers), d), dtype=rec.dtype, device=rec.device)
                std = torch.ones((len(layers), d), dtype=rec.dtype, device=rec.device)
                for i, l in enumerate(layers):
                    if l in self.mean_tg and l in self.std_tg:
                        mean[i] = self.mean_tg[l].to(rec.device, rec.dtype).reshape(-1)
                        std[i] = self.std_tg[l].to(rec.device, rec.dtype).reshape(-1)
            elif self.normalization_method == "sqrt_d_model" and self.d_model is not None:
                mode, scale = "sqrt_d_model", self.d_model ** 0.5
            stats = engine.reconstruction_stats(rec, tgt, mode, mean, std, scale).tolist()
            for i, l in enumerate(layers):
                mse, tvar, evar = stats[i]
                ev = (1.0 - evar / tvar) if tvar > 1e-9 else (1.0 if evar < 1e-9 else 0.0)
                nmse = (mse / tvar) if tvar > 1e-9 else (0.0 if mse < 1e-9 else float("inf"))
                total_ev += ev
                total_nmse += nmse
                layerwise_nmse[f"layer_{l}"] = nmse
                layerwise_ev[f"layer_{l}"] = ev
        n = len(layers)
        avg_ev = total_ev / n if n > 0 else 0.0
        return {"reconstruction/explained_variance": max(0.0, min(1.0, avg_ev)),
                "reconstruction/normalized_mean_reconstruction_error": total_nmse / n if n > 0 else 0.0,
                "layerwise/normalized_mse": layerwise_nmse, "layerwise/explained_variance": layerwise_ev}

    # ---- evaluator.py:407-441 ----
    def _compute_dead_neuron_metrics(self, dead_neuron_mask: Optional[torch.Tensor]) -> Dict[str, Any]:
        out: Dict[str, Any] = {"layerwise/dead_features": {}}
        if dead_neuron_mask is not None:
            dead_neuron_mask = dead_neuron_mask.to(self.device)
            expected = (self.model.config.num_layers, self.model.config.num_features)
            if tuple(dead_neuron_mask.shape) == expected:
                per_layer = dead_neuron_mask.sum(dim=1).tolist()
                out["layerwise/dead_features"] = {f"layer_{i}": per_layer[i] for i in range(expected[0])}
            else:
                logger.warning(f"Warning: Received dead_neuron_mask with unexpected shape {dead_neuron_mask.shape}. "
                               f"Expected {expected}. Skipping dead neuron eval metrics.")
        return out

    # ---- evaluator.py:99-192 ----
    @torch.no_grad()
    def compute_metrics(self, inputs: Dict[int, torch.Tensor], targets: Dict[int, torch.Tensor],
                        dead_neuron_mask: Optional[torch.Tensor] = None) -> Dict[str, Any]:
        inputs = {k: v.to(self.device) for k, v in inputs.items()}
        targets = {k: v.to(self.device) for k, v in targets.items()}
        res = self.model.forward_with_survivors(inputs)
        if res is not None:
            reconstructions, activations = res
        else:
            reconstructions = self.model(inputs)
            activations = self.model.get_feature_activations(inputs)
        present = sorted(inputs) if res is not None else None
        counts = self._counts(activations, present) if _has_data(activations) else None
        sparsity = self._compute_sparsity(activations, counts)
        reconstruction = self._compute_reconstruction_metrics(targets, reconstructions)
        density = self._compute_feature_density(activations, counts)
        dead = self._compute_dead_neuron_metrics(dead_neuron_mask)

        log_density = density.get("layerwise/log_feature_density", {})
        heuristic = density.get("layerwise/consistent_activation_heuristic", {})
        density_mean = self._calculate_aggregate_metric(log_density)
        heuristic_mean = self._calculate_aggregate_metric(heuristic)
        density_hist = self._calculate_aggregate_histogram_data(log_density)
        heuristic_hist = self._calculate_aggregate_histogram_data(heuristic)
        if density_mean is not None:
            sparsity["sparsity/feature_density_mean"] = density_mean
        if heuristic_mean is not None:
            sparsity["sparsity/consistent_activation_heuristic_mean"] = heuristic_mean
        if density_hist:
            sparsity["sparsity/log_feature_density_agg_hist"] = density_hist
        if heuristic_hist:
            sparsity["sparsity/consistent_activation_heuristic_agg_hist"] = heuristic_hist
        dead["dead_features/total_eval"] = sum(dead.get("layerwise/dead_features", {}).values())
        return {**reconstruction, **sparsity, **density, **dead}


def _has_data(activations) -> bool:
    if isinstance(activations, SurvivorList):
        return activations.T > 0 and activations.L > 0
    return bool(activations) and any(v.numel() > 0 for v in activations.values())
