"""Encoder stack: L independent projections x[l] -> x[l] @ W[l].T + b[l].

Interface of the reference's ``Encoder`` (clt/models/encoder.py:14-164): the same
``encoders`` ModuleList (state-dict keys ``encoders.{l}.weight`` / ``.bias_param``),
``get_preactivations`` with its log-and-return-zeros behaviour for bad inputs, and
``encode_all_layers``.  The L weight matrices live in one [L, F, d] slab (each
parameter is a view of it) so that all layers are projected by a single MFMA launch.
"""

from __future__ import annotations

import logging
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from . import engine
from .parallel import ColumnParallelLinear, require_single_rank

logger = logging.getLogger(__name__)


class Encoder(nn.Module):
    def __init__(self, config, process_group, device: torch.device, dtype: torch.dtype):
        super().__init__()
        require_single_rank(process_group)
        self.config = config
        self.process_group = process_group
        self.device = device
        self.dtype = dtype
        self.world_size, self.rank = 1, 0
        L, F, d = config.num_layers, config.num_features, config.d_model
        self._w_slab = torch.empty(L, F, d, device=device, dtype=dtype)
        self._b_slab = torch.empty(L, F, device=device, dtype=dtype)
        self.encoders = nn.ModuleList(
            ColumnParallelLinear(d, F, bias=True, process_group=process_group, device=device, dtype=dtype,
                                 weight_storage=self._w_slab[l], bias_storage=self._b_slab[l])
            for l in range(L))

    # ---- slab bookkeeping -------------------------------------------------------
    def stacked(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """([L, F, d] weights, [L, F] biases) that alias the per-layer parameters.

        ``module.to(...)`` and similar replace a parameter's storage; when any layer no
        longer aliases the slab, the slab is rebuilt from the parameters and they are
        pointed back at it.
        """
        w0 = self.encoders[0].weight
        ok = (self._w_slab.device == w0.device and self._w_slab.dtype == w0.dtype)
        if ok:
            for l, enc in enumerate(self.encoders):
                if (enc.weight.data_ptr() != self._w_slab[l].data_ptr()
                        or enc.bias_param.data_ptr() != self._b_slab[l].data_ptr()):
                    ok = False
                    break
        if not ok:
            with torch.no_grad():
                w = torch.stack([e.weight.detach() for e in self.encoders]).contiguous()
                b = torch.stack([e.bias_param.detach() for e in self.encoders]).contiguous()
                for l, enc in enumerate(self.encoders):
                    enc.weight.data = w[l]
                    enc.bias_param.data = b[l]
            self._w_slab, self._b_slab = w, b
            self.device, self.dtype = w.device, w.dtype
        return self._w_slab, self._b_slab

    # ---- reference interface ------------------------------------------------------
    def _zeros(self, rows: int) -> torch.Tensor:
        return torch.zeros((rows, self.config.num_features), device=self.device, dtype=self.dtype)

    def check_input(self, x: torch.Tensor, layer_idx: int) -> Tuple[Optional[torch.Tensor], int]:
        """Validate one layer's input the way get_preactivations does (encoder.py:63-121).

        Returns (x as [tokens, d_model] or None when the fallback applies, fallback rows).
        """
        d = self.config.d_model
        if x.dim() == 2:
            flat, rows = x, x.shape[0]
        elif x.dim() == 3:
            rows = x.shape[0] * x.shape[1]
            if x.shape[2] != d:
                logger.warning(f"Rank {self.rank}: Input d_model {x.shape[2]} != config {d} layer {layer_idx}")
                return None, rows
            flat = x.reshape(-1, d)
        else:
            logger.warning(f"Rank {self.rank}: Cannot handle input shape {x.shape} for preactivations layer {layer_idx}")
            return None, (x.shape[0] if x.dim() > 0 else 0)
        if flat.shape[1] != d:
            logger.warning(f"Rank {self.rank}: Input d_model {flat.shape[1]} != config {d} layer {layer_idx}")
            return None, rows
        if not (0 <= layer_idx < len(self.encoders)) and not (-len(self.encoders) <= layer_idx < 0):
            logger.error(
                f"Rank {self.rank}: Invalid layer index {layer_idx} requested for encoder. "
                f"Max index is {len(self.encoders) - 1}.")
            return None, rows
        return flat, rows

    def get_preactivations(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor:
        """Pre-activations [tokens, F] of one layer; zeros of the expected shape (plus a log
        line) for an input the layer cannot take."""
        x = x.to(device=self.device, dtype=self.dtype)
        flat, rows = self.check_input(x, layer_idx)
        if flat is None:
            return self._zeros(rows)
        w, b = self.stacked()
        l = layer_idx % len(self.encoders)
        return engine.encode(flat.detach().contiguous().unsqueeze(0), w[l:l + 1], b[l:l + 1])[0]

    def encode_all_layers(self, inputs: Dict[int, torch.Tensor]
                          ) -> Tuple[Dict[int, torch.Tensor], List[Tuple[int, int, int]]]:
        """Pre-activations of every given layer, in sorted layer order, plus
        (layer, batch, seq_len) of each input (encoder.py:133-164)."""
        shapes: List[Tuple[int, int, int]] = []
        for l in sorted(inputs.keys()):
            x = inputs[l]
            if x.dim() == 3:
                shapes.append((l, x.shape[0], x.shape[1]))
            elif x.dim() == 2:
                shapes.append((l, x.shape[0], 1))
        slab = self.encode_slab(inputs)
        if slab is not None:
            layers, pre = slab
            return {l: pre[i] for i, l in enumerate(layers)}, shapes
        return {l: self.get_preactivations(inputs[l], l) for l in sorted(inputs.keys())}, shapes

    # ---- fused path ---------------------------------------------------------------
    def encode_slab(self, inputs: Dict[int, torch.Tensor], out: Optional[torch.Tensor] = None):
        """All given layers in one launch.  Returns (sorted layers, pre [n, T, F]) or None when
        some input needs the per-layer fallbacks (bad shape, unequal token counts, bad index)."""
        prep = self.prepare_slab(inputs)
        if prep is None:
            return None
        layers, x_slab, ws, bs = prep
        return layers, engine.encode(x_slab, ws, bs, out=out)

    def prepare_slab(self, inputs: Dict[int, torch.Tensor]):
        """(sorted layers, x [n, T, d], weights [n, F, d], biases [n, F]) of the given layers, or
        None when some input needs the per-layer fallbacks."""
        layers = sorted(inputs.keys())
        if not layers:
            return None
        L, d = self.config.num_layers, self.config.d_model
        flats = []
        T = None
        for l in layers:
            x = inputs[l]
            if not (0 <= l < L) or x.dim() not in (2, 3) or x.shape[-1] != d:
                return None
            f = x.to(device=self.device, dtype=self.dtype).reshape(-1, d)
            if T is None:
                T = f.shape[0]
            if f.shape[0] != T or T == 0:
                return None
            flats.append(f)
        w, b = self.stacked()
        x_slab = _as_slab(flats)
        if layers == list(range(L)):
            ws, bs = w, b
        else:
            idx = torch.tensor(layers, device=w.device)
            ws, bs = w.index_select(0, idx), b.index_select(0, idx)
        return layers, x_slab, ws, bs


def _as_slab(flats: List[torch.Tensor]) -> torch.Tensor:
    """[n, T, d] view when the per-layer inputs already sit back to back in memory, else a copy."""
    first = flats[0]
    T, d = first.shape
    step = T * d * first.element_size()
    base = first.data_ptr()
    contiguous = all(f.is_contiguous() and f.data_ptr() == base + i * step for i, f in enumerate(flats))
    if contiguous and len(flats) > 1:
        try:
            return first.detach().as_strided((len(flats), T, d), (T * d, d, 1))
        except RuntimeError:
            pass
    return torch.stack([f.detach() for f in flats]).contiguous()
