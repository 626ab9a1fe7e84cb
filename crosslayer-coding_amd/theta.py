"""JumpReLU threshold holder.

Keeps the reference's parameter (``theta_manager.log_threshold`` [L, F], initialised to
log(jumprelu_threshold), clt/models/theta.py:50-61) and its ``jumprelu(x, layer)`` call
(theta.py:70-79): theta = exp(log_threshold[layer]) rounded to the model dtype, then
``x >= theta`` keeps x.  Post-hoc theta estimation and BatchTopK->JumpReLU conversion
(theta.py:82-636) are training-side tools and are not part of this build.
"""

from __future__ import annotations

import logging
from typing import Optional, cast

import torch
import torch.nn as nn

from .activations import JumpReLU
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
        return torch.exp(self.log_threshold.detach()).to(dtype).contiguous()

    def jumprelu(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor:
        if self.log_threshold is None:
            logger.error(f"Rank {self.rank}: log_threshold not initialized for JumpReLU. Returning input.")
            return x.to(device=self.device, dtype=self.dtype)
        if layer_idx >= self.log_threshold.shape[0]:
            logger.error(f"Rank {self.rank}: Invalid layer_idx {layer_idx} for log_threshold. Returning input.")
            return x.to(device=self.device, dtype=self.dtype)
        theta = torch.exp(self.log_threshold[layer_idx]).to(device=self.device, dtype=self.dtype)
        return cast(torch.Tensor, JumpReLU.apply(x, theta, self.bandwidth))

    def estimate_theta_posthoc(self, *args, **kwargs):
        raise NotImplementedError("post-hoc theta estimation is a training-side tool outside this build")

    def convert_to_jumprelu_inplace(self, *args, **kwargs):
        raise NotImplementedError("BatchTopK->JumpReLU conversion is a training-side tool outside this build")
