"""Abstract transcoder contract and the single-file save/load of the reference
(clt/models/base.py:13-101)."""

from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import asdict, is_dataclass
from typing import Dict, Optional

import torch
import torch.nn as nn

from .config import CLTConfig


class BaseTranscoder(nn.Module, ABC):
    config: CLTConfig

    def __init__(self, config: CLTConfig):
        super().__init__()
        self.config = config

    @abstractmethod
    def encode(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor: ...

    @abstractmethod
    def decode(self, a: Dict[int, torch.Tensor], layer_idx: int) -> torch.Tensor: ...

    @abstractmethod
    def forward(self, inputs: Dict[int, torch.Tensor]) -> Dict[int, torch.Tensor]: ...

    def save(self, path: str) -> None:
        """{"config": dict, "state_dict": ...} in one torch file (base.py:65-79)."""
        cfg = asdict(self.config) if is_dataclass(self.config) else dict(self.config.__dict__)
        torch.save({"config": cfg, "state_dict": self.state_dict()}, path)

    @classmethod
    def load(cls, path: str, device: Optional[torch.device] = None):
        ckpt = torch.load(path, map_location=device, weights_only=True)
        model = cls(CLTConfig(**ckpt["config"]), None, device)
        model.load_state_dict(ckpt["state_dict"])
        return model
