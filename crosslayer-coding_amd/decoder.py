"""Decoder stack: rec[t] = sum over sources s <= t of a[s] . W_dec + bias.

Interface and parameter layout of the reference's ``Decoder``
(clt/models/decoder.py:14-485): ``decoders`` is a ModuleDict keyed "s->t" (untied) or
a ModuleList (per_source / per_target tying) of layers whose ``weight`` is [d_model, F];
optional ``skip_weights``, ``feature_offset``, ``feature_scale``; ``decode`` and
``get_decoder_norms`` with the same arguments, log messages and zero fallbacks.

Internally every decoder matrix also exists as a feature-major [F, d_model] copy in one
slab, so that the contribution of an active feature is one contiguous read, and the
activations are handled as survivor lists (non-zeros only).
"""

from __future__ import annotations

import logging
import weakref
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn

from . import _native as nat
from . import engine
from .engine import SurvivorList
from .parallel import RowParallelLinear, require_single_rank

logger = logging.getLogger(__name__)


def merge_layer_lists(parts: List[Tuple[int, SurvivorList]], L: int, T: int, F: int,
                      dtype: torch.dtype, device: torch.device) -> SurvivorList:
    """One survivor list over L layers from single-layer lists given as (layer, list),
    layers ascending; layers that are not given get empty rows."""
    counts = torch.zeros(L * T, dtype=torch.int64, device=device)
    cols, vals = [], []
    for s, sl in parts:
        counts[s * T:(s + 1) * T] = (sl.row_ptr[1:] - sl.row_ptr[:-1]).to(torch.int64)
        cols.append(sl.col)
        vals.append(sl.val)
    row_ptr = torch.zeros(L * T + 1, dtype=torch.int32, device=device)
    row_ptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
    col = torch.cat(cols) if cols else torch.empty(0, dtype=torch.int32, device=device)
    val = torch.cat(vals) if vals else torch.empty(0, dtype=dtype, device=device)
    return SurvivorList(row_ptr, col, val, T, F, L, dtype)


class _SyncedModuleDict(nn.ModuleDict):
    """The decoders by key.  Reading an entry first brings the checkpoint-layout parameters up to date when an
    optimiser step has left them behind the feature-major working copy (``Decoder.sync_parameters``)."""

    def _sync(self):
        owner = self.__dict__.get("_owner")
        if owner is not None and owner() is not None:
            owner().sync_parameters()

    def __getitem__(self, key):
        self._sync()
        return super().__getitem__(key)

    def __iter__(self):
        self._sync()
        return super().__iter__()

    def values(self):
        self._sync()
        return super().values()

    def items(self):
        self._sync()
        return super().items()


class _SyncedModuleList(nn.ModuleList):
    """Same for tied decoders (a list)."""

    def _sync(self):
        owner = self.__dict__.get("_owner")
        if owner is not None and owner() is not None:
            owner().sync_parameters()

    def __getitem__(self, idx):
        self._sync()
        return super().__getitem__(idx)

    def __iter__(self):
        self._sync()
        return super().__iter__()


class Decoder(nn.Module):
    def __init__(self, config, process_group, device: torch.device, dtype: torch.dtype):
        super().__init__()
        require_single_rank(process_group)
        self.config = config
        self.process_group = process_group
        self.device = device
        self.dtype = dtype
        self.world_size, self.rank = 1, 0
        L, F, d = config.num_layers, config.num_features, config.d_model
        tied = config.decoder_tying in ("per_source", "per_target")

        def make():
            return RowParallelLinear(F, d, bias=True, process_group=process_group, d_model_for_init=d,
                                     num_layers_for_init=L, device=device, dtype=dtype)

        # the optimiser's in-kernel decoder step updates the feature-major working copy only and leaves the
        # checkpoint-layout parameters behind until something reads them (sync_parameters)
        self._params_behind = False
        self._sync_table = None
        if tied:
            self.decoders = _SyncedModuleList(make() for _ in range(L))
            for dec in self.decoders:  # tied decoders start at zero (decoder.py:80-86)
                nn.init.zeros_(dec.weight)
                nn.init.zeros_(dec.bias_param)
        else:
            self.decoders = _SyncedModuleDict({f"{s}->{t}": make() for s in range(L) for t in range(s, L)})
        self.decoders.__dict__["_owner"] = weakref.ref(self)
        self.register_state_dict_pre_hook(lambda module, prefix, keep_vars: module.sync_parameters())

        def square():
            return nn.Parameter(torch.zeros(d, d, device=device, dtype=dtype))

        if config.skip_connection:
            if tied:
                self.skip_weights = nn.ParameterList(square() for _ in range(L))
            else:
                self.skip_weights = nn.ParameterDict({f"{s}->{t}": square() for s in range(L) for t in range(s, L)})
        else:
            self.skip_weights = None

        # per-target affine on the selected features, tied decoders only (decoder.py:141-172)
        self.feature_offset = None
        self.feature_scale = None
        if tied and config.enable_feature_offset:
            self.feature_offset = nn.ParameterList(
                nn.Parameter(torch.zeros(F, device=device, dtype=dtype)) for _ in range(L))
        if tied and config.enable_feature_scale:
            self.feature_scale = nn.ParameterList(
                nn.Parameter(torch.ones(F, device=device, dtype=dtype) if i == 0
                             else torch.full((F,), 0.1, device=device, dtype=dtype)) for i in range(L))

        self.register_buffer("_cached_decoder_norms", None, persistent=False)
        self._slab: Optional[torch.Tensor] = None
        self._slab_keys: List[Optional[tuple]] = []
        self._norm_key = None
        self._bias_cache: Dict[int, Tuple[tuple, torch.Tensor]] = {}     # kept for callers that clear it; unused
        # writes to the parameters that no version counter shows (``weight.data.copy_(...)``): every use of the
        # packed copy checks a sampled fingerprint of the parameters on the device and repacks there what changed
        self.watch_parameter_data = True
        self._fp_state: Optional[torch.Tensor] = None
        self._fp_changed: Optional[torch.Tensor] = None
        self._fp_fresh = False
        self._tables: Dict[str, tuple] = {}
        self._compact_cache: Dict[int, tuple] = {}
        # decoders tied per target: targets whose summed activations are dense enough go through the
        # matrix cores (see dense_split); False keeps every target on the row gather
        self.dense_route = True
        self.last_route: Dict[str, Tuple[int, int]] = {}

    # ---- decoder bookkeeping -------------------------------------------------------
    def _ordered(self) -> List[RowParallelLinear]:
        """Decoder layers in slot order (untied: "0->0", "0->1", ..., as created)."""
        mods = self.decoders._modules      # straight to the registry: no parameter sync for internal walks
        cached = self.__dict__.get("_ordered_cache")
        if cached is not None and cached[0] is mods and cached[1] == len(mods) and all(
                a is b for a, b in zip(cached[3], mods.values())):
            return cached[2]
        if isinstance(self.decoders, nn.ModuleDict):
            L = self.config.num_layers
            out = [mods[f"{s}->{t}"] for s in range(L) for t in range(s, L)]
        else:
            out = list(mods.values())
        self.__dict__["_ordered_cache"] = (mods, len(mods), out, list(mods.values()))
        return out

    # ---- parameters behind the working copy -------------------------------------------
    def mark_parameters_behind(self) -> None:
        """The feature-major slab now holds newer decoder weights than the checkpoint-layout parameters."""
        self._params_behind = True

    def sync_parameters(self) -> None:
        """Rewrite the checkpoint-layout decoder weights [d, F] from the feature-major slab when a step has left
        them behind.  Runs by itself before anything hands the parameters out: ``state_dict``,
        ``parameters`` / ``named_parameters``, ``decoders[key]``, ``.to(...)``."""
        if not self._params_behind:
            return
        self._params_behind = False
        import ctypes
        ws = [lin.weight.data for lin in self._ordered()]
        ptrs = tuple(w.data_ptr() for w in ws)
        if self._sync_table is None or self._sync_table[0] != ptrs:
            self._sync_table = (ptrs, torch.tensor(ptrs, dtype=torch.int64, device=ws[0].device),
                                (ctypes.c_void_p * len(ptrs))(*ptrs))
        d, F = ws[0].shape
        engine.unpack_decoders(self._slab, self._sync_table[1], self._sync_table[2], d, F)
        self.note_parameters_written()     # the parameters hold new values: record them before a caller writes more

    def named_parameters(self, *args, **kwargs):
        self.sync_parameters()
        return super().named_parameters(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self.sync_parameters()
        return super()._apply(fn, *args, **kwargs)

    def _slots(self) -> List[Tuple[int, int]]:
        """(source, target) fed by each slot; tied decoders report (i, i)."""
        L = self.config.num_layers
        if self.config.decoder_tying == "none":
            return [(s, t) for s in range(L) for t in range(s, L)]
        return [(i, i) for i in range(L)]

    def _pointer_table(self, name: str, tensors) -> torch.Tensor:
        """Device int64 tensor with the addresses of ``tensors``, rebuilt only when one has moved."""
        ptrs = tuple(t.data_ptr() for t in tensors)
        ent = self._tables.get(name)
        if ent is None or ent[0] != ptrs or ent[1].device != tensors[0].device:
            # through pinned memory and an asynchronous copy: building the table must not synchronise a forward
            host = torch.tensor(ptrs, dtype=torch.int64).pin_memory()
            ent = (ptrs, host.to(tensors[0].device, non_blocking=True), host)
            self._tables[name] = ent
        return ent[1]

    def note_parameters_written(self) -> None:
        """A kernel of this library has just written the decoder parameters and the packed copy alike: the stored
        fingerprints are of the old values.  They are taken again right here, behind that kernel on the stream, so
        that a write the caller makes afterwards through ``.data`` still differs from what is stored."""
        self._fp_fresh = False
        decs = self._ordered()
        if (self.watch_parameter_data and self._fp_state is not None and self._slab is not None
                and self._fp_state.device == decs[0].weight.device and all(dec.weight.is_contiguous() for dec in decs)):
            engine.decoder_fingerprint(self._pointer_table("w", [dec.weight for dec in decs]), self.config.d_model,
                                       self.config.num_features, decs[0].weight.dtype, self._fp_state, self._fp_changed, True)
            self._fp_fresh = True

    def packed(self) -> torch.Tensor:
        """[n_dec, F, pitch] feature-major slab (``engine.decoder_pitch``), true to the parameters: matrices
        whose parameter changed are repacked - by the host where the parameter's version counter shows it, by the
        device itself where only the data does (``weight.data.fill_(...)``; ``watch_parameter_data``)."""
        decs = self._ordered()
        w0 = decs[0].weight
        F, d = self.config.num_features, self.config.d_model
        if (self._slab is None or self._slab.device != w0.device or self._slab.dtype != w0.dtype
                or self._slab.shape[0] != len(decs)):
            self._slab = engine.alloc_packed(len(decs), F, d, w0.dtype, w0.device)
            self._slab_keys = [None] * len(decs)
            self.device, self.dtype = w0.device, w0.dtype
            self._fp_state = None
        for i, dec in enumerate(decs):
            w = dec.weight
            key = (w.data_ptr(), w._version)
            if self._slab_keys[i] != key:
                engine.pack_decoder(w.detach().contiguous(), self._slab[i])
                self._slab_keys[i] = key
                self._repacks = getattr(self, "_repacks", 0) + 1
        if self.watch_parameter_data and not getattr(self, "_params_behind", False) \
                and all(dec.weight.is_contiguous() for dec in decs):
            if self._fp_state is None or self._fp_state.device != w0.device:
                self._fp_state = torch.zeros(16 * len(decs), dtype=torch.int64, device=w0.device)
                self._fp_changed = torch.zeros(len(decs), dtype=torch.int32, device=w0.device)
                self._fp_fresh = False
            table = self._pointer_table("w", [dec.weight for dec in decs])
            if not self._fp_fresh:
                # first use (or after invalidate_packed): the slab has just been made from these values: record them
                engine.decoder_fingerprint(table, d, F, w0.dtype, self._fp_state, self._fp_changed, True)
                self._fp_fresh = True
            else:
                engine.decoder_fingerprint(table, d, F, w0.dtype, self._fp_state, self._fp_changed, False)
                engine.pack_decoders_if(table, self._slab, d, F, self._fp_changed)
                # copies derived from the slab (the optimiser's tiles) cannot know whether the device repacked
                if getattr(self, "_derived_copies", False):
                    self._repacks = getattr(self, "_repacks", 0) + 1
        return self._slab

    def packed_generation(self):
        """Changes whenever ``packed()`` has rebuilt any matrix from its parameter: other copies derived from the
        slab (the optimiser's tiled weights) are stale then."""
        return (None if self._slab is None else self._slab.data_ptr(), getattr(self, "_repacks", 0))

    def invalidate_packed(self) -> None:
        """Force a repack on next use (needed only after writes that bypass autograd
        version counting, e.g. through ``.data``)."""
        self._params_behind = False        # the parameters are what counts from here on
        self._slab_keys = [None] * len(self._slab_keys)
        self._bias_cache.clear()
        self._cached_decoder_norms = None
        self._fp_fresh = False

    def bias_sum(self, src_mask: int) -> torch.Tensor:
        """[L, d] fp32: for every target the sum of the biases of the decoders that run for
        it - one per contributing source (decoder.py:294-295 / parallel.py:380-381), or the
        target's own decoder for per_target tying (decoder.py:250-251)."""
        decs = self._ordered()
        bs = [dec.bias_param for dec in decs]
        if all(b is not None and b.is_contiguous() and b.is_cuda for b in bs):
            # computed anew on every call (one small launch): a write to a bias shows whichever way it was made
            return engine.bias_sum(self._pointer_table("b", bs), self.config.d_model, self.config.num_layers,
                                   self.config.decoder_tying, src_mask, bs[0].dtype)
        L, d = self.config.num_layers, self.config.d_model
        B = torch.stack([dec.bias_param.detach() for dec in decs]).float()
        tying = self.config.decoder_tying
        if tying == "per_target":
            return B.contiguous()
        out = torch.zeros(L, d, dtype=torch.float32, device=B.device)
        if tying == "none":
            first = 0
            for s in range(L):
                if (src_mask >> s) & 1:
                    out[s:] += B[first:first + L - s]
                first += L - s
        else:
            run = torch.zeros(d, dtype=torch.float32, device=B.device)
            for t in range(L):
                if (src_mask >> t) & 1:
                    run = run + B[t]
                out[t] = run
        return out

    def _affine(self):
        L = self.config.num_layers
        off = torch.stack([p.detach() for p in self.feature_offset]).contiguous() if self.feature_offset is not None else None
        sc = torch.stack([p.detach() for p in self.feature_scale]).contiguous() if self.feature_scale is not None else None
        assert off is None or off.shape[0] == L
        return off, sc

    def _skip_term(self, x2d: torch.Tensor, w_skip: torch.Tensor) -> torch.Tensor:
        """x @ w_skip.T in fp32 (decoder.py:310, 332) through the encoder's MFMA kernel."""
        x = x2d.detach().to(device=self.device, dtype=self.dtype).reshape(1, -1, self.config.d_model).contiguous()
        return engine.encode(x, w_skip.detach().unsqueeze(0).contiguous(), None)[0].float()

    # ---- fused path ------------------------------------------------------------------
    # Rates behind the choice between the two decode routes.  Both are measured on the GPU at hand, once per
    # process and shape (``route_rates``): the matrix-core kernel on the very product the dense route would
    # run, and a bare gather of decoder rows from a table the size of one L2 (clt_probe_gather), of which the
    # sparse decode - survivor lists, partial rows and arithmetic around the same loads - delivers a fraction.
    GATHER_EFFICIENCY = 0.62          # sparse decode / bare gather, see bench.py's roofline.frac (0.60 - 0.67)
    _rate_cache: Dict[tuple, Tuple[float, float]] = {}
    rate_override: Optional[Tuple[float, float]] = None     # (gather bytes / s, MFMA flop / s): tests and experiments

    def route_rates(self, T: int, F: int, d: int, dtype: torch.dtype, batch: int = 1) -> Tuple[float, float]:
        """(bytes / s of decoder rows the row gather delivers, flop / s of the dense product [T, F] x [F, d]);
        ``batch``: that many products with one left operand in one launch, as the dense route of untied decoders
        runs them (a single product of few tiles leaves most compute units idle)."""
        if self.rate_override is not None:
            return self.rate_override
        dev = self._ordered()[0].weight.device
        key = (dev.index, T, F, d, dtype, batch)
        hit = Decoder._rate_cache.get(key)
        if hit is not None:
            return hit

        def best_of(fn, reps=3):
            fn()
            best = float("inf")
            for _ in range(reps):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                fn()
                b.record()
                b.synchronize()
                best = min(best, a.elapsed_time(b) * 1e-3)
            return best

        esize = torch.finfo(dtype).bits // 8
        # the dense product itself, on scratch operands of the real shape
        x = torch.zeros((1, T, F), dtype=dtype, device=dev).expand(batch, T, F)
        w = torch.zeros((batch, d, F), dtype=dtype, device=dev)
        out = torch.empty((batch, T, d), dtype=dtype, device=dev)
        mfma = 2.0 * T * F * d * batch / best_of(lambda: engine.encode(x, w, None, out=out))
        del x, w, out
        # a bare gather of rows of this width from 4 MB (what an XCD's L2 holds of a decoder matrix)
        row_bytes = max(16, min(d * esize, 2048) // 16 * 16)
        n_rows = max(1, (4 << 20) // row_bytes)
        n_idx = max(1, (1 << 30) // row_bytes)
        g = torch.Generator(device=dev).manual_seed(0)
        table = torch.randint(0, 1 << 30, (n_rows * row_bytes // 4,), dtype=torch.int32, device=dev, generator=g)
        idx = torch.randint(0, n_rows, (n_idx,), dtype=torch.int32, device=dev, generator=g)
        sink = torch.empty(256 * 8 * 256, dtype=torch.float32, device=dev)
        lib, stream = nat.load(), nat.current_stream(dev)

        def probe():
            nat.check(lib.clt_probe_gather(table.data_ptr(), n_rows, row_bytes, idx.data_ptr(), n_idx, 256 * 8, 0,
                                           sink.data_ptr(), stream), "clt_probe_gather")

        gather = self.GATHER_EFFICIENCY * n_idx * row_bytes / best_of(probe)
        Decoder._rate_cache[key] = (gather, mfma)
        return gather, mfma

    def dense_split(self, surv: SurvivorList, src_mask: int, t_begin: int, t_end: int,
                    skip_add: Optional[torch.Tensor]) -> int:
        """First target of [t_begin, t_end) that is decoded as a dense product (``t_end``: none is).

        Decoders tied per target multiply the SUM of the activations of all sources <= t
        (decoder.py:208-251), so target t gathers (t + 1) k T decoder rows of d elements from one matrix:
        with every further source the gather grows and the dense product ``summed [T, F] @ W[t].T`` does
        not.  The dense route is taken from the first target on for which
        ``2 T F d / MFMA rate < rows gathered x d x element size / gather rate`` (``route_rates``).  Untied and per-source
        decoders have no such sum - each (source, target) pair has its own operand or its own matrix - and go dense
        only at high densities (``dense_pairs_wanted``)."""
        cfg = self.config
        if cfg.decoder_tying == "per_target" and self._beyond_gather_layers(skip_add, affine_ok=True):
            return t_begin
        if cfg.decoder_tying != "per_target" or not self.dense_route:
            return t_end
        T, F, d = surv.T, surv.F, cfg.d_model
        esize = torch.finfo(surv.dtype).bits // 8
        # shapes the MFMA kernel of clt_encode takes (K = F in whole 128-byte stages, 256 x 256 tiles)
        if surv.dtype not in (torch.bfloat16, torch.float16, torch.float32) or T < 256 or d < 256 or d % 4 or F % (128 // esize):
            return t_end
        if engine.decode_route(T, d, F, cfg.num_layers, cfg.decoder_tying, surv.dtype) == nat.ROUTE_GENERIC:
            # rows wider than the gather kernels of this tying hold (d_model beyond 2560 in 16-bit elements): the
            # generic kernel that would serve them is two orders of magnitude slower than the product
            return t_begin
        gather_rate, mfma_rate = self.route_rates(T, F, d, surv.dtype)
        dense_s = 2.0 * T * F * d / mfma_rate
        per_layer = self._survivors_per_layer(surv)
        n_src = 0
        for t in range(t_end):
            n_src += (src_mask >> t) & 1
            if t >= t_begin and n_src * per_layer * d * esize / gather_rate > dense_s:
                return t
        return t_end

    @staticmethod
    def _survivors_per_layer(surv: SurvivorList) -> float:
        """Survivors of one source layer, from a host-side figure: the exact total where the list was sized from
        it, else the last total seen for the shape; a threshold list whose total is not known yet is priced at
        2 % density (its arrays are sized for the largest list, which says nothing about the batch)."""
        total = surv.nnz_hint
        if total is None:
            total = surv.col.numel() if surv.status is None else min(surv.col.numel(), surv.L * surv.T * surv.F // 50)
        return total / max(1, surv.L)

    # a (source, target) pair goes to the dense product when its gather is priced this many times dearer
    DENSE_PAIR_MARGIN = 1.25
    # layers the gather and survivor-list kernels take (the set of source layers a batch has inputs for travels
    # through them as one 64-bit word); deeper models run on the dense formulations only
    MAX_GATHER_LAYERS = 64

    def _beyond_gather_layers(self, skip_add: Optional[torch.Tensor], affine_ok: bool) -> bool:
        """True for a model of more layers than the gather kernels take: its decode and gradients are the dense
        products whatever the density (what the reference runs).  Raises for what those do not cover."""
        if self.config.num_layers <= self.MAX_GATHER_LAYERS:
            return False
        affine = self.feature_offset is not None or self.feature_scale is not None
        if affine and not affine_ok:
            raise NotImplementedError(
                f"num_layers = {self.config.num_layers} > {self.MAX_GATHER_LAYERS}: such models run on the dense products, "
                "which cover the per-target feature offset / scale only in the forward of decoders tied per target")
        return True

    def dense_pairs_wanted(self, surv: SurvivorList, skip_add: Optional[torch.Tensor], any_tying: bool = False) -> bool:
        """Untied and per-source decoders at densities the survivor gather was not made for (a ReLU model, JumpReLU
        thresholds at the start of a training run, a very large k): every active (token, feature) of a source
        fetches a decoder row per target, k T rows of d elements, while the reference's dense product
        ``a[s] @ W[s->t].T`` (decoder.py:253-316) costs 2 T F d whatever the density.  With the measured rates of
        ``route_rates`` the product wins above roughly 1.5 - 2 % of the features active per token."""
        if self.config.num_layers > self.MAX_GATHER_LAYERS:
            return self.dense_pairs_wanted_for(0.0, surv.T, surv.dtype, skip_add, any_tying)
        if surv.nnz_hint is None and surv.status is not None:
            return False                # a threshold list of unknown size (first forward of a shape): the gather
        return self.dense_pairs_wanted_for(self._survivors_per_layer(surv), surv.T, surv.dtype, skip_add, any_tying)

    def dense_pairs_wanted_for(self, per_layer: float, T: int, dtype: torch.dtype, skip_add: Optional[torch.Tensor],
                               any_tying: bool = False) -> bool:
        """``dense_pairs_wanted`` for ``per_layer`` survivors per source layer in a batch of ``T`` tokens.
        ``any_tying``: decoders tied per target included (their forward has its own rule, ``dense_split``; the
        gradients ask here)."""
        cfg = self.config
        if cfg.decoder_tying == "per_target" and not any_tying:
            return False
        if self._beyond_gather_layers(skip_add, affine_ok=False):
            return True
        if not self.dense_route:
            return False
        if self.feature_offset is not None or self.feature_scale is not None:
            return False
        F, d = cfg.num_features, cfg.d_model
        esize = torch.finfo(dtype).bits // 8
        if dtype not in (torch.bfloat16, torch.float16, torch.float32) or T < 256 or d < 256 or d % 4 or F % (128 // esize):
            return False
        if engine.decode_route(T, d, F, cfg.num_layers, cfg.decoder_tying, dtype) == nat.ROUTE_GENERIC:
            return True                 # rows no gather kernel holds (wide and not whole cache lines): the product
        if per_layer < 0.004 * T * F:
            return False                # no plausible pair of rates sends so sparse a batch to the product
        if self.rate_override is None and torch.cuda.is_current_stream_capturing():
            return False                # (the rates are measured with events on first use: not under a capture)
        # a launch of the dense route multiplies a source with all its targets, (L + 1) / 2 of them on average
        batch = max(1, (cfg.num_layers + 1) // 2) if cfg.decoder_tying == "none" else 1
        gather_rate, mfma_rate = self.route_rates(T, F, d, dtype, batch)
        gather_s = per_layer * d * esize / gather_rate
        return gather_s > self.DENSE_PAIR_MARGIN * 2.0 * T * F * d / mfma_rate

    @staticmethod
    def _add_skip(out: torch.Tensor, skip_add: Optional[torch.Tensor], t_begin: int, t_end: int) -> None:
        """out[t] += the skip-connection terms (fp32 [L, T, d], ``skip_all_targets``) of the targets [t_begin, t_end)."""
        if skip_add is not None and t_end > t_begin:
            out[t_begin:t_end] = (out[t_begin:t_end].float() + skip_add[t_begin:t_end]).to(out.dtype)

    def _decode_dense_pairs(self, surv: Optional[SurvivorList], src_mask: int, t_begin: int, t_end: int, ws,
                            dense: Optional[Dict[int, torch.Tensor]] = None,
                            skip_add: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Targets [t_begin, t_end) of untied or per-source decoders as the reference's dense products: per source
        layer the survivors are scattered into a dense [T, F] operand, one launch of the matrix-core kernel
        multiplies it with the decoders of all its targets (checkpoint layout [d, F], bias included, one rounding
        per product as ``F.linear`` has), and the products are added per target in source order in the model dtype
        (decoder.py:283-316: ``reconstruction += decoded``).  ``dense`` {source layer: [T, F] activations}: operands
        that are dense already (``clt_threshold_dense``) instead of a survivor list."""
        cfg = self.config
        L, F, d = cfg.num_layers, cfg.num_features, cfg.d_model
        if dense is not None:
            some = next(iter(dense.values()))
            T, dtype, dev = some.shape[0], some.dtype, some.device
            acc = None
        else:
            T, dtype, dev = surv.T, surv.dtype, surv.row_ptr.device
            acc = (ws.typed("dense_sum", (T, F), dtype) if ws is not None
                   else torch.empty((T, F), dtype=dtype, device=dev))
        out = torch.zeros((L, T, d), dtype=dtype, device=dev)
        decs = self._ordered()
        first = 0                       # slot of (s, s) in the untied order (s, t) = (0, 0), (0, 1), ..
        for s in range(min(t_end, L)):
            row0 = first
            first += L - s
            if not (src_mask >> s) & 1:
                continue
            lo = max(s, t_begin)
            if lo >= t_end:
                continue
            if dense is not None:
                acc = dense[s]
            else:
                engine.accumulate_dense(surv, s, acc, True)
            if cfg.decoder_tying == "none":
                lins = [decs[row0 + (t - s)] for t in range(lo, t_end)]
            else:                       # one decoder per source: the same product goes to every target >= s
                lins = [decs[s]]
            w = torch.stack([lin.weight.detach() for lin in lins])
            b = torch.stack([lin.bias_param.detach() for lin in lins])
            prod = engine.encode(acc.unsqueeze(0).expand(len(lins), T, F), w, b)
            if cfg.decoder_tying == "none":
                out[lo:t_end] += prod
            else:
                out[lo:t_end] += prod[0]
        self._add_skip(out, skip_add, t_begin, t_end)
        return out

    def _decode_dense(self, surv: SurvivorList, src_mask: int, t_first: int, t_end: int, out: torch.Tensor, ws) -> None:

        """Targets [t_first, t_end) of decoders tied per target as dense products: the reference's own
        formulation (decoder.py:208-251) - activations summed over the sources in the model dtype, one
        ``F.linear`` with the target's decoder in its checkpoint layout - with the sum built by scattering
        the survivor lists and the product on the MFMA kernel."""
        T, F = surv.T, surv.F
        acc = (ws.typed("dense_sum", (T, F), surv.dtype) if ws is not None
               else torch.empty((T, F), dtype=surv.dtype, device=out.device))
        off, sc = self._affine()
        affine = off is not None or sc is not None
        started = False
        for t in range(t_end):
            if affine:
                # the affine terms are the TARGET's: the sum is rebuilt for every target
                if t < t_first:
                    continue
                engine.accumulate_dense(surv, -1, acc, True)
                for s in range(t + 1):
                    if (src_mask >> s) & 1:
                        engine.accumulate_dense(surv, s, acc, False, off[t] if off is not None else None,
                                                sc[t] if sc is not None else None)
            else:
                if (src_mask >> t) & 1:
                    engine.accumulate_dense(surv, t, acc, not started)
                    started = True
                if t < t_first:
                    continue
                if not started:
                    engine.accumulate_dense(surv, -1, acc, True)
                    started = True
            lin = self.decoders[t]          # (brings the parameters up to date if a step left them behind)
            engine.encode(acc.unsqueeze(0), lin.weight.detach().unsqueeze(0), lin.bias_param.detach().unsqueeze(0),
                          out=out[t].unsqueeze(0))

    def decode_survivors(self, surv: SurvivorList, src_mask: int, t_begin: int = 0, t_end: Optional[int] = None,
                         skip_add: Optional[torch.Tensor] = None, ws=None) -> torch.Tensor:
        """Reconstructions [L, T, d] (rows outside [t_begin, t_end) are not written)."""
        cfg = self.config
        t_end = cfg.num_layers if t_end is None else t_end
        if self.dense_pairs_wanted(surv, skip_add):
            self.last_route = {"sparse_targets": (t_begin, t_begin), "dense_targets": (t_begin, t_end)}
            return self._decode_dense_pairs(surv, src_mask, t_begin, t_end, ws, skip_add=skip_add)
        split = self.dense_split(surv, src_mask, t_begin, t_end, skip_add)
        self.last_route = {"sparse_targets": (t_begin, split), "dense_targets": (split, t_end)}
        out = None
        if split < t_end:
            out = torch.empty((surv.L, surv.T, cfg.d_model), dtype=surv.dtype, device=surv.row_ptr.device)
            self._decode_dense(surv, src_mask, split, t_end, out, ws)
            self._add_skip(out, skip_add, split, t_end)
            if split == t_begin:
                return out
        off, sc = self._affine()
        return engine.decode_sparse(surv, self.packed(), cfg.decoder_tying, cfg.d_model,
                                    bias_sum=self.bias_sum(src_mask), feat_offset=off, feat_scale=sc,
                                    skip_add=skip_add, t_begin=t_begin, t_end=split, src_mask=src_mask, out=out, ws=ws)

    def skip_all_targets(self, inputs: Dict[int, torch.Tensor], src_mask: int, T: int) -> Optional[torch.Tensor]:
        """[L, T, d] fp32 skip-connection terms for every target present in ``inputs``."""
        if self.skip_weights is None:
            return None
        L, d = self.config.num_layers, self.config.d_model
        out = torch.zeros(L, T, d, dtype=torch.float32, device=self.device)
        for t in range(L):
            if t not in inputs:
                continue
            if self.config.decoder_tying == "none":
                for s in range(t + 1):
                    if (src_mask >> s) & 1 and s in inputs and f"{s}->{t}" in self.skip_weights:
                        out[t] += self._skip_term(inputs[s], self.skip_weights[f"{s}->{t}"])
            else:
                out[t] += self._skip_term(inputs[t], self.skip_weights[t])
        return out

    # ---- reference interface -----------------------------------------------------------
    def _compact(self, a2d: torch.Tensor, orig: torch.Tensor) -> SurvivorList:
        ent = self._compact_cache.get(id(orig))
        if ent is not None and ent[0]() is orig and ent[1] == orig._version:
            return ent[2]
        sl = engine.threshold_select(a2d.detach().contiguous().unsqueeze(0), None, nat.PRED_NONZERO)
        if len(self._compact_cache) > 4 * self.config.num_layers + 8:
            self._compact_cache.clear()
        try:
            self._compact_cache[id(orig)] = (weakref.ref(orig), orig._version, sl)
        except TypeError:
            pass
        return sl

    def decode(self, a: Dict[int, torch.Tensor], layer_idx: int,
               source_inputs: Optional[Dict[int, torch.Tensor]] = None) -> torch.Tensor:
        """Reconstruction [tokens, d_model] of ``layer_idx`` from dense activations ``a``."""
        cfg = self.config
        d, F = cfg.d_model, cfg.num_features
        keys = sorted(a.keys())
        if not keys:
            logger.warning(f"Rank {self.rank}: No activation keys available in decode method for layer {layer_idx}")
            return torch.zeros((0, d), device=self.device, dtype=self.dtype)
        batch = 0
        for k in keys:
            if a[k].numel() > 0:
                batch = a[k].shape[0] if a[k].dim() <= 2 else a[k].numel() // a[k].shape[-1]
                break
        if batch == 0:
            return torch.zeros((0, d), device=self.device, dtype=self.dtype)
        parts: List[Tuple[int, SurvivorList]] = []
        src_mask = 0
        for s in range(layer_idx + 1):
            if s not in a:
                continue
            act = a[s]
            if act.numel() == 0:
                continue
            if act.shape[-1] != F:
                logger.warning(
                    f"Rank {self.rank}: Activation tensor for layer {s} has incorrect feature dimension "
                    f"{act.shape[-1]}, expected {F}. Skipping decode contribution.")
                continue
            a2 = act.to(device=self.device, dtype=self.dtype).reshape(-1, F)
            if a2.shape[0] != batch:
                raise ValueError(f"activation rows {a2.shape[0]} of layer {s} do not match batch {batch}")
            nat.require_device(a2, "decode")
            parts.append((s, self._compact(a2, act)))
            src_mask |= 1 << s
        L = cfg.num_layers
        surv = merge_layer_lists(parts, L, batch, F, self.dtype, self.device)
        skip = None
        if self.skip_weights is not None and source_inputs is not None:
            acc = torch.zeros(batch, d, dtype=torch.float32, device=self.device)
            if cfg.decoder_tying == "none":
                for s, _ in parts:
                    if s in source_inputs and f"{s}->{layer_idx}" in self.skip_weights:
                        acc += self._skip_term(source_inputs[s], self.skip_weights[f"{s}->{layer_idx}"])
            elif layer_idx in source_inputs:
                acc += self._skip_term(source_inputs[layer_idx], self.skip_weights[layer_idx])
            skip = torch.zeros(L, batch, d, dtype=torch.float32, device=self.device)
            skip[layer_idx] = acc
        out = self.decode_survivors(surv, src_mask, layer_idx, layer_idx + 1, skip_add=skip)
        return out[layer_idx]

    def get_decoder_norms(self) -> torch.Tensor:
        """[L, F] L2 norm of each feature's decoder vectors over the decoders its source
        feeds (decoder.py:374-485); cached until ``_cached_decoder_norms`` is cleared or a
        decoder weight changes."""
        decs = self._ordered()
        key = tuple((dec.weight.data_ptr(), dec.weight._version) for dec in decs)
        if self._cached_decoder_norms is not None and self._norm_key == key:
            return self._cached_decoder_norms
        norms = engine.decoder_norms(self.packed(), self.config.num_layers, self.config.decoder_tying,
                                     self.config.d_model)
        self._cached_decoder_norms = norms
        self._norm_key = key
        return norms
