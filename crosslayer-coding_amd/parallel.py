"""Parameter holders with the reference's names and shapes, at world_size 1.

The reference shards these layers over a process group (clt/models/parallel.py); this
build runs one GPU, so a layer is just its full ``weight`` / ``bias_param`` pair:

    ColumnParallelLinear  weight [out, in], bias_param [out]   init U(+-1/sqrt(out))
    RowParallelLinear     weight [out, in], bias_param [out]   init U(+-1/sqrt(L*d_model))

(shapes clt/models/parallel.py:53-75, init :82-93).  ``forward`` of either layer runs
the HIP kernels, so code that calls ``model.encoder_module.encoders[l](x)`` or
``model.decoder_module.decoders[key](a)`` directly keeps working.
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn

from . import _native as nat
from . import engine


def mark_replicated(param: nn.Parameter) -> None:
    """Tag a parameter as replicated across tensor-parallel ranks (models/__init__.py:4-11)."""
    param.__dict__["_is_replicated"] = True


def is_replicated(param: nn.Parameter) -> bool:
    return getattr(param, "_is_replicated", False)


def _world_size(process_group) -> int:
    if process_group is None:
        return 1
    import torch.distributed as dist

    if not (dist.is_available() and dist.is_initialized()):
        return 1
    return dist.get_world_size(process_group)


def require_single_rank(process_group) -> None:
    if _world_size(process_group) != 1:
        raise NotImplementedError(
            "this build implements the CLT forward path on one GPU (world_size 1); "
            "feature sharding over a process group is not part of it")


class _Linear(nn.Module):
    bias_param: Optional[nn.Parameter]

    def __init__(self, in_features: int, out_features: int, bias: bool, process_group, bound: float,
                 device=None, dtype=None, weight_storage: Optional[torch.Tensor] = None,
                 bias_storage: Optional[torch.Tensor] = None):
        super().__init__()
        require_single_rank(process_group)
        self.process_group = process_group
        self.world_size, self.rank = 1, 0
        self.bias = bias
        self.full_in_features = self.local_in_features = in_features
        self.full_out_features = self.local_out_features = out_features
        self.dtype = dtype if dtype is not None else torch.float32
        w = weight_storage if weight_storage is not None else torch.empty(
            out_features, in_features, device=device, dtype=self.dtype)
        assert w.shape == (out_features, in_features)
        self.weight = nn.Parameter(w)
        with torch.no_grad():
            self.weight.uniform_(-bound, bound)
        if bias:
            b = bias_storage if bias_storage is not None else torch.empty(
                out_features, device=device, dtype=self.dtype)
            self.bias_param = nn.Parameter(b)
            with torch.no_grad():
                self.bias_param.zero_()
        else:
            self.bias_param = None


class ColumnParallelLinear(_Linear):
    """Encoder layer: y = x @ weight.T + bias_param (parallel.py:282-294)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, process_group=None,
                 device=None, dtype=None, weight_storage=None, bias_storage=None, **_unused):
        super().__init__(in_features, out_features, bias, process_group, 1.0 / math.sqrt(out_features),
                         device, dtype, weight_storage, bias_storage)

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        nat.require_device(input_, "ColumnParallelLinear")
        lead = input_.shape[:-1]
        x = input_.detach().to(self.weight.dtype).reshape(1, -1, self.full_in_features).contiguous()
        b = self.bias_param.detach().unsqueeze(0) if self.bias_param is not None else None
        y = engine.encode(x, self.weight.detach().unsqueeze(0), b)
        return y[0].view(*lead, self.full_out_features)


class RowParallelLinear(_Linear):
    """Decoder layer: y = a @ weight.T + bias_param with weight [d_model, F]
    (parallel.py:335-383).  ``a`` is compacted to its non-zeros and decoded sparsely."""

    def __init__(self, in_features: int, out_features: int, *, bias: bool = True, process_group=None,
                 d_model_for_init: int, num_layers_for_init: int, device=None, dtype=None, **_unused):
        if d_model_for_init is None or num_layers_for_init is None:
            raise ValueError("d_model_for_init and num_layers_for_init must be provided for RowParallelLinear init")
        super().__init__(in_features, out_features, bias, process_group,
                         1.0 / math.sqrt(num_layers_for_init * d_model_for_init), device, dtype)
        if self.bias_param is not None:
            mark_replicated(self.bias_param)
        self._packed: Optional[torch.Tensor] = None
        self._packed_key = None

    def packed_weight(self) -> torch.Tensor:
        """Feature-major [F, d] copy of ``weight``, made anew on every call: a layer used on its own is not a
        hot path, and a write through ``weight.data`` leaves no trace a cache could be keyed on."""
        w = self.weight
        if self._packed is None or self._packed.device != w.device or self._packed.dtype != w.dtype:
            self._packed = torch.empty(self.full_in_features, engine.decoder_pitch(self.full_out_features, w.dtype),
                                       device=w.device, dtype=w.dtype)
        engine.pack_decoder(w.detach().contiguous(), self._packed)
        return self._packed

    def forward(self, input_: torch.Tensor) -> torch.Tensor:
        nat.require_device(input_, "RowParallelLinear")
        if input_.size(-1) > self.full_in_features:
            raise ValueError(
                f"RowParallelLinear (rank {self.rank}): Input slice size ({input_.size(-1)}) "
                f"unexpectedly greater than expected padded size ({self.full_in_features}).")
        lead = input_.shape[:-1]
        a = input_.detach().to(self.weight.dtype).reshape(1, -1, input_.size(-1))
        if a.size(-1) < self.full_in_features:
            a = torch.nn.functional.pad(a, (0, self.full_in_features - a.size(-1)))
        surv = engine.threshold_select(a.contiguous(), None, nat.PRED_NONZERO)
        bias = self.bias_param.detach().float().unsqueeze(0).contiguous() if self.bias_param is not None else None
        out = engine.decode_sparse(surv, self.packed_weight().unsqueeze(0), "per_source", self.full_out_features,
                                   bias_sum=bias)
        return out[0].view(*lead, self.full_out_features)
