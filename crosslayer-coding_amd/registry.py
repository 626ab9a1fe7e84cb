"""Activation registry: name -> fn(model, preact, layer_idx).

The reference's plugin table (clt/activations/registry.py:13-108) with the same four
built-in entries; the per-layer BatchTopK / TopK entries are the ones the per_layer
top-k mode resolves to (registry.py:43-98).
"""

from __future__ import annotations

import logging
from typing import Callable, Dict, cast

import torch

logger = logging.getLogger(__name__)

ActivationCallable = Callable[[object, torch.Tensor, int], torch.Tensor]
ACTIVATION_REGISTRY: Dict[str, ActivationCallable] = {}


def register_activation_fn(name: str) -> Callable[[ActivationCallable], ActivationCallable]:
    def decorator(fn: ActivationCallable) -> ActivationCallable:
        if name in ACTIVATION_REGISTRY:
            logger.warning(f"Activation function '{name}' is already registered. Overwriting.")
        ACTIVATION_REGISTRY[name] = fn
        return fn

    return decorator


def get_activation_fn(name: str) -> ActivationCallable:
    fn = ACTIVATION_REGISTRY.get(name)
    if fn is None:
        raise ValueError(
            f"Activation function '{name}' not found in registry. Available: {list(ACTIVATION_REGISTRY.keys())}")
    return fn


@register_activation_fn("relu")
def relu_activation(model, preact: torch.Tensor, layer_idx: int) -> torch.Tensor:
    from . import _native as nat
    from . import engine

    nat.require_device(preact, "relu")
    p2 = preact.detach().reshape(1, -1, preact.shape[-1]).contiguous()
    surv = engine.threshold_select(p2, None, nat.PRED_GT_ZERO)
    return engine.densify(surv)[0].view(preact.shape)


@register_activation_fn("jumprelu")
def jumprelu_activation(model, preact: torch.Tensor, layer_idx: int) -> torch.Tensor:
    return model.jumprelu(preact, layer_idx)


@register_activation_fn("batchtopk")
def batchtopk_per_layer_activation(model, preact: torch.Tensor, layer_idx: int) -> torch.Tensor:
    from .activations import BatchTopK

    logger.warning(
        f"Rank {model.rank}: 'encode' called for BatchTopK on layer {layer_idx}. "
        f"This applies TopK per-layer, not globally. Use 'get_feature_activations' for global BatchTopK.")
    if model.config.batchtopk_k is not None:
        k = int(model.config.batchtopk_k)
    else:
        k = preact.size(1)
        logger.warning(
            f"Rank {model.rank}: batchtopk_k not set in config for per-layer BatchTopK on layer {layer_idx}. "
            f"Defaulting to k={k} (all features for this layer).")
    return cast(torch.Tensor, BatchTopK.apply(preact, float(k), model.config.batchtopk_straight_through, preact))


@register_activation_fn("topk")
def topk_per_layer_activation(model, preact: torch.Tensor, layer_idx: int) -> torch.Tensor:
    from .activations import TokenTopK

    logger.warning(
        f"Rank {model.rank}: 'encode' called for TopK (TokenTopK) on layer {layer_idx}. "
        f"This applies TopK per-layer, not globally. Use 'get_feature_activations' for global TopK.")
    if getattr(model.config, "topk_k", None) is not None:
        k = float(model.config.topk_k)
    else:
        k = float(preact.size(1))
        logger.warning(
            f"Rank {model.rank}: topk_k not set in config for per-layer TopK on layer {layer_idx}. "
            f"Defaulting to k={k} (all features for this layer).")
    ste = getattr(model.config, "topk_straight_through", True)
    return cast(torch.Tensor, TokenTopK.apply(preact, k, ste, preact))
