"""Synthetic CLT workloads: weights and inputs of the benchmark configurations.

Weights   W_enc[l] ~ U(+-1/sqrt(d_model))  [F, d_model]
          W_dec    ~ U(+-1/sqrt(F))         stored [d_model, F] (checkpoint layout)
          biases 0; drawn in fp32, then cast to the model dtype.
Inputs    x[l] = N(0,1)[T, d_model] * scale[l][d_model], scale ~ LogNormal(0, 0.5),
          4 fixed outlier dimensions (the same for every layer) multiplied by 20, then
          standardised with ONE mean and std per layer taken over the whole [T, d_model]
          block (a per-dimension standardisation would undo the scales and the outliers).
JumpReLU  theta ~ LogNormal(-1, 0.5); the encoder bias is set per feature to
          theta - mean - 2.512 * std of the bias-free pre-activation over the batch, so that
          about 0.6 % of the features fire per token.
Seeds     1000 + index of the workload for weights, +50 for inputs, +70 for thresholds.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .config import CLTConfig


@dataclass(frozen=True)
class Workload:
    name: str
    index: int
    num_layers: int
    d_model: int
    num_features: int
    tokens: int
    dtype: str
    activation_fn: str = "batchtopk"
    k: Optional[int] = 200
    topk_mode: str = "per_layer"
    decoder_tying: str = "none"

    def config(self) -> CLTConfig:
        return CLTConfig(
            num_features=self.num_features, num_layers=self.num_layers, d_model=self.d_model,
            activation_fn=self.activation_fn, batchtopk_k=self.k if self.activation_fn == "batchtopk" else None,
            topk_k=float(self.k) if self.activation_fn == "topk" else None, topk_mode=self.topk_mode,
            clt_dtype=self.dtype, decoder_tying=self.decoder_tying, jumprelu_threshold=0.03)

    def scaled(self, name: str, **kw) -> "Workload":
        base = dict(self.__dict__)
        base.update(kw)
        base["name"] = name
        return Workload(**base)


WORKLOADS: Dict[str, Workload] = {
    # small GPT-2-shaped, fp32 (the case a CPU also runs)
    "c0": Workload("c0", 0, 12, 768, 6144, 1024, "float32"),
    # GPT-2-small x32, bf16: the headline
    "c1": Workload("c1", 1, 12, 768, 24576, 4096, "bfloat16"),
    # Pythia-410m-shaped JumpReLU
    "c2": Workload("c2", 2, 24, 1024, 32768, 4096, "bfloat16", activation_fn="jumprelu", k=None),
    # Pythia-1B-shaped, one decoder per target
    "c3": Workload("c3", 3, 16, 2048, 16384, 8192, "bfloat16", decoder_tying="per_target"),
}


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def decoder_names(wl: Workload):
    L = wl.num_layers
    if wl.decoder_tying == "none":
        return [f"{s}->{t}" for s in range(L) for t in range(s, L)]
    return [str(i) for i in range(L)]


def make_inputs(wl: Workload, device="cpu", seed: Optional[int] = None) -> torch.Tensor:
    """Input slab [L, T, d_model] in the workload dtype."""
    device = torch.device(device)
    dtype = getattr(torch, wl.dtype)
    gw = _gen(device, 1000 + wl.index if seed is None else seed)
    gi = _gen(device, 1050 + wl.index if seed is None else seed + 50)
    L, T, d = wl.num_layers, wl.tokens, wl.d_model
    outliers = torch.randperm(d, generator=gw, device=device)[:4]
    out = torch.empty(L, T, d, dtype=dtype, device=device)
    for l in range(L):
        scale = torch.exp(0.5 * torch.randn(d, generator=gi, device=device))
        x = torch.randn(T, d, generator=gi, device=device) * scale
        x[:, outliers] *= 20.0
        x = (x - x.mean()) / x.std()
        out[l] = x.to(dtype)
    return out


def make_targets(wl: Workload, device="cpu", seed: Optional[int] = None) -> torch.Tensor:
    """Reconstruction targets [L, T, d_model] of the training-step workload: N(0, 1) per coordinate
    times a per-dimension scale ~ LogNormal(0, 0.5), standardised per layer."""
    device = torch.device(device)
    dtype = getattr(torch, wl.dtype)
    g = _gen(device, 1090 + wl.index if seed is None else seed + 90)
    L, T, d = wl.num_layers, wl.tokens, wl.d_model
    out = torch.empty(L, T, d, dtype=dtype, device=device)
    for l in range(L):
        y = torch.randn(T, d, generator=g, device=device) * torch.exp(0.5 * torch.randn(d, generator=g, device=device))
        out[l] = ((y - y.mean()) / y.std()).to(dtype)
    return out


def make_state_dict(wl: Workload, device="cpu", seed: Optional[int] = None,
                    inputs: Optional[torch.Tensor] = None) -> Dict[str, torch.Tensor]:
    """Checkpoint-layout parameters (the keys ``CrossLayerTranscoder.state_dict()`` has)."""
    device = torch.device(device)
    dtype = getattr(torch, wl.dtype)
    g = _gen(device, 1001 + wl.index if seed is None else seed + 1)
    L, d, F = wl.num_layers, wl.d_model, wl.num_features
    sd: Dict[str, torch.Tensor] = {}
    be, bd = 1.0 / math.sqrt(d), 1.0 / math.sqrt(F)
    for l in range(L):
        w = (torch.rand(F, d, generator=g, device=device) * 2 - 1) * be
        sd[f"encoder_module.encoders.{l}.weight"] = w.to(dtype)
        sd[f"encoder_module.encoders.{l}.bias_param"] = torch.zeros(F, dtype=dtype, device=device)
    for name in decoder_names(wl):
        w = (torch.rand(d, F, generator=g, device=device) * 2 - 1) * bd
        sd[f"decoder_module.decoders.{name}.weight"] = w.to(dtype)
        sd[f"decoder_module.decoders.{name}.bias_param"] = torch.zeros(d, dtype=dtype, device=device)
    if wl.activation_fn == "jumprelu":
        gt = _gen(device, 1070 + wl.index if seed is None else seed + 70)
        theta = torch.exp(-1.0 + 0.5 * torch.randn(L, F, generator=gt, device=device))
        sd["theta_manager.log_threshold"] = torch.log(theta).to(dtype)
        if inputs is not None:
            # calibrate the encoder bias on the given batch; 2.512 = z-score of the 99.4 % quantile
            theta_used = torch.exp(sd["theta_manager.log_threshold"].float())
            for l in range(L):
                pre0 = inputs[l].float() @ sd[f"encoder_module.encoders.{l}.weight"].float().T
                b = theta_used[l] - pre0.mean(dim=0) - 2.512 * pre0.std(dim=0)
                sd[f"encoder_module.encoders.{l}.bias_param"] = b.to(dtype)
    return sd


def build_model(wl: Workload, device, seed: Optional[int] = None
                ) -> Tuple["torch.nn.Module", Dict[int, torch.Tensor], torch.Tensor]:
    """(model on ``device`` with the synthetic weights, inputs dict of slab views, slab)."""
    from .clt import CrossLayerTranscoder

    device = torch.device(device)
    x = make_inputs(wl, device, seed)
    model = CrossLayerTranscoder(wl.config(), None, device)
    sd = make_state_dict(wl, device, seed, inputs=x)
    model.load_state_dict(sd)
    del sd
    return model, {l: x[l] for l in range(wl.num_layers)}, x
