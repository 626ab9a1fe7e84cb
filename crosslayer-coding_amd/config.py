"""Model configuration accepted by the MI355X CrossLayerTranscoder.

Field names, defaults, validation and the JSON round trip follow the reference's
``CLTConfig`` (clt/config/clt_config.py:10-124) so that a ``cfg.json`` written by the
reference's trainer loads unchanged.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, fields
from typing import Optional

_ACTIVATIONS = ("jumprelu", "relu", "batchtopk", "topk")
_NORMALIZATIONS = ("none", "mean_std", "sqrt_d_model")
_TYINGS = ("none", "per_source", "per_target")
# normalization_method spellings of older checkpoints (clt_config.py:99-106)
_LEGACY_NORMALIZATION = {
    "auto": "mean_std",
    "estimated_mean_std": "mean_std",
    "auto_sqrt_d_model": "sqrt_d_model",
    "estimated_mean_std_sqrt_d_model": "sqrt_d_model",
}


@dataclass
class CLTConfig:
    num_features: int
    num_layers: int
    d_model: int
    model_name: Optional[str] = None
    normalization_method: str = "none"
    activation_fn: str = "jumprelu"
    jumprelu_threshold: float = 0.03
    batchtopk_k: Optional[int] = None
    batchtopk_straight_through: bool = True
    topk_k: Optional[float] = None
    topk_straight_through: bool = True
    topk_mode: str = "global"
    clt_dtype: Optional[str] = None
    expected_input_dtype: Optional[str] = None
    mlp_input_template: Optional[str] = None
    mlp_output_template: Optional[str] = None
    tl_input_template: Optional[str] = None
    tl_output_template: Optional[str] = None
    decoder_tying: str = "none"
    enable_feature_offset: bool = False
    enable_feature_scale: bool = False
    skip_connection: bool = False

    def __post_init__(self):
        assert self.num_features > 0, "Number of features must be positive"
        assert self.num_layers > 0, "Number of layers must be positive"
        assert self.d_model > 0, "Model dimension must be positive"
        assert self.normalization_method in _NORMALIZATIONS, (
            f"Invalid normalization_method: {self.normalization_method}. Must be one of {list(_NORMALIZATIONS)}")
        assert self.activation_fn in _ACTIVATIONS, (
            f"Invalid activation_fn: {self.activation_fn}. Must be one of {list(_ACTIVATIONS)}")
        if self.activation_fn == "batchtopk":
            if self.batchtopk_k is None:
                raise ValueError("batchtopk_k must be specified for BatchTopK.")
            if self.batchtopk_k <= 0:
                raise ValueError("batchtopk_k must be positive.")
        if self.activation_fn == "topk":
            if self.topk_k is None:
                raise ValueError("topk_k must be specified for TopK activation function.")
            if self.topk_k <= 0:
                raise ValueError("topk_k must be positive if specified.")
        assert self.decoder_tying in _TYINGS, (
            f"Invalid decoder_tying: {self.decoder_tying}. Must be one of {list(_TYINGS)}")

    @classmethod
    def from_json(cls, json_path: str) -> "CLTConfig":
        with open(json_path, "r") as fh:
            raw = json.load(fh)
        raw.setdefault("decoder_tying", "none")
        raw.setdefault("enable_feature_offset", False)
        raw.setdefault("enable_feature_scale", False)
        if raw.get("normalization_method") in _LEGACY_NORMALIZATION:
            raw["normalization_method"] = _LEGACY_NORMALIZATION[raw["normalization_method"]]
        if raw.pop("sqrt_d_model_normalize", False):
            raw["normalization_method"] = "sqrt_d_model"
        return cls(**raw)

    def to_json(self, json_path: str) -> None:
        with open(json_path, "w") as fh:
            json.dump({f.name: getattr(self, f.name) for f in fields(self)}, fh, indent=4)
