"""CrossLayerTranscoder for one MI355X.

Drop-in for the forward path of the reference class (clt/models/clt.py:22-425): same
constructor, ``encode`` / ``decode`` / ``forward`` / ``get_feature_activations`` /
``get_preactivations`` / ``_encode_all_layers`` / ``get_decoder_norms`` / ``jumprelu``,
same sub-module and parameter names (so ``state_dict()`` and safetensors checkpoints are
interchangeable), same log-and-return-zeros handling of bad inputs.

``forward`` never materialises dense activations: one MFMA launch projects all layers,
the selection kernels turn the pre-activations into survivor lists, and the sparse
decoder writes every target layer.  ``get_feature_activations`` densifies those lists
because its callers index [tokens, features] tensors.

The kernels implement inference: results carry no autograd graph.
"""

from __future__ import annotations

import logging
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from . import _native as nat
from . import engine
from .activations import resolve_token_k
from .base import BaseTranscoder
from .config import CLTConfig
from .decoder import Decoder
from .encoder import Encoder
from .engine import SurvivorList, Workspace
from .parallel import require_single_rank
from .registry import get_activation_fn
from .theta import ThetaManager

logger = logging.getLogger(__name__)


class _NullTimer:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


class _ReconstructionsWithGraph(torch.autograd.Function):
    """``forward`` as one node of an autograd graph: the reconstructions of all layers as functions of every
    parameter.  The forward is the fused HIP path; the backward hands d loss / d reconstruction to the same
    kernels ``loss_and_gradients`` uses (activations.py:66-96, 183-220 for the gates; the products are the
    reference's linear layers, parallel.py:282-294, 335-383).  The inputs get no gradient."""

    @staticmethod
    def forward(ctx, model, inputs, names, *params):
        with torch.no_grad():
            recs, surv = model.forward_with_survivors(inputs)
            surv = surv.trimmed()
            # the list lives in the model's workspace, which the next forward overwrites: keep a copy
            ctx.surv = SurvivorList(surv.row_ptr.clone(), surv.col.clone(), surv.val.clone(), surv.T, surv.F, surv.L,
                                    surv.dtype, None, surv.nnz_hint)
        ctx.model, ctx.inputs, ctx.names = model, inputs, names
        ctx.versions = [p._version for p in params]
        ctx.params = params
        L = model.config.num_layers
        return tuple(recs[l] for l in range(L))

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, *grad_outs):
        model = ctx.model
        if any(p._version != v for p, v in zip(ctx.params, ctx.versions)):
            raise RuntimeError("a parameter of the CrossLayerTranscoder was modified in place between forward and "
                               "backward: the gradient would be taken at other weights than the output was")
        surv = ctx.surv
        L, T, d = surv.L, surv.T, model.config.d_model
        g = torch.zeros((L, T, d), dtype=torch.float32, device=surv.row_ptr.device)
        for l, go in enumerate(grad_outs):
            if go is not None:
                g[l] = go.reshape(T, d)
        g_model = g.to(model.dtype)
        raw = model._raw_gradients_from(ctx.inputs, surv, g, g_model, g.sum(dim=1))
        named = model._named_gradients(raw)
        grads = []
        for name, p in zip(ctx.names, ctx.params):
            gp = named.get(name)
            grads.append(None if gp is None or not p.requires_grad else gp.to(p.dtype).reshape(p.shape))
        return (None, None, None, *grads)


MAX_LAYERS = Decoder.MAX_GATHER_LAYERS     # beyond: dense formulations only


class CrossLayerTranscoder(BaseTranscoder):
    device: torch.device
    dtype: torch.dtype

    def __init__(self, config: CLTConfig, process_group=None, device: Optional[torch.device] = None,
                 profiler: Optional[Any] = None):
        super().__init__(config)
        require_single_rank(process_group)
        if config.num_layers > MAX_LAYERS:
            # said here, not by the first forward: the gather and survivor-list kernels keep the set of layers a batch
            # has inputs for in one 64-bit word; a deeper model decodes and trains through the dense products
            # (TokenTopK's selection keeps per-layer counters for up to 1024 layers)
            if config.activation_fn == "topk" and config.num_layers > 1024:
                raise NotImplementedError(f"num_layers = {config.num_layers} > 1024 together with TokenTopK: not built")
        self.process_group = process_group
        self.world_size, self.rank = 1, 0
        self.profiler = profiler
        # per-layer BatchTopK: let the encoder epilogue collect the candidates (same result, one
        # dense write and one dense read less); False forces the separate encode + select kernels
        self.fuse_encode_select = True
        self._density_ppm = 20000   # JumpReLU survivor density the candidate pool is sized for
        self.dtype = self._resolve_dtype(config.clt_dtype)
        if device is not None:
            self.device = torch.device(device)
        else:
            self.device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
        logger.info(f"CLT TP model initialized on rank {self.rank} with device {self.device} and dtype {self.dtype}")
        self.encoder_module = Encoder(config, process_group, self.device, self.dtype)
        self.decoder_module = Decoder(config, process_group, self.device, self.dtype)
        self.theta_manager = ThetaManager(config, process_group, self.device, self.dtype)
        self._ws: Optional[Workspace] = None
        # threshold activations (JumpReLU, ReLU): a forward reads nothing back when survivor arrays that hold ANY
        # batch of the shape fit this many bytes (None: an eighth of the device memory); beyond that it reads
        # the survivor total back once per forward and sizes the arrays exactly
        self.threshold_list_budget_bytes: Optional[int] = None
        # survivor totals on their way back to the host (they tune the candidate pool, nothing depends on them)
        self._thr_key, self._thr_elems, self._thr_last_total = None, 0, None
        self._thr_pending: List[tuple] = []

    # ---- small helpers ---------------------------------------------------------------
    def _resolve_dtype(self, dtype_input: Optional[Union[str, torch.dtype]]) -> torch.dtype:
        if isinstance(dtype_input, torch.dtype):
            return dtype_input
        if isinstance(dtype_input, str):
            cand = getattr(torch, dtype_input, None)
            if isinstance(cand, torch.dtype):
                return cand
            logger.warning(f"Unsupported CLT dtype string: '{dtype_input}'. Defaulting to float32.")
        return torch.float32

    def _workspace(self) -> Workspace:
        dev = self.encoder_module.encoders[0].weight.device
        if self._ws is None or self._ws.device != dev:
            self._ws = Workspace(dev)
        return self._ws

    def _timed(self, name: str):
        return self.profiler.timer(name) if self.profiler else _NullTimer()

    def _record(self, name: str, timer) -> None:
        if self.profiler and hasattr(timer, "elapsed"):
            self.profiler.record(name, timer.elapsed)

    def _sync_device(self) -> None:
        """Follow the parameters after ``module.to(...)``."""
        w = self.encoder_module.encoders[0].weight
        if w.device != self.device or w.dtype != self.dtype:
            self.device, self.dtype = w.device, w.dtype
            for m in (self.encoder_module, self.decoder_module, self.theta_manager):
                m.device, m.dtype = w.device, w.dtype

    # ---- float16 models ----------------------------------------------------------------------------------
    # The forward path (encoder, selection, decode, evaluator reductions) and theta estimation have float16
    # kernels of their own; the backward and the optimiser step are built for float32 and bfloat16 only.
    def _is_half(self) -> bool:
        self._sync_device()
        return self.dtype == torch.float16

    def _no_half(self, what: str) -> None:
        if self._is_half():
            raise NotImplementedError(f"{what} is not built for float16 models (float32 and bfloat16 only)")

    def release_workspace(self) -> None:
        """Free the cached scratch buffers (pre-activations, selection workspace)."""
        if self._ws is not None:
            self._ws.release()

    # ---- reference API: thin delegations ------------------------------------------------
    def jumprelu(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor:
        self._sync_device()
        return self.theta_manager.jumprelu(x, layer_idx)

    def get_preactivations(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor:
        self._sync_device()
        self._note_no_graph("get_preactivations")
        return self.encoder_module.get_preactivations(x, layer_idx)

    def _encode_all_layers(self, inputs: Dict[int, torch.Tensor]
                           ) -> Tuple[Dict[int, torch.Tensor], List[Tuple[int, int, int]]]:
        self._sync_device()
        return self.encoder_module.encode_all_layers(inputs)

    def decode(self, a: Dict[int, torch.Tensor], layer_idx: int,
               source_inputs: Optional[Dict[int, torch.Tensor]] = None) -> torch.Tensor:
        self._sync_device()
        return self.decoder_module.decode(a, layer_idx, source_inputs)

    def get_decoder_norms(self) -> torch.Tensor:
        self._sync_device()
        return self.decoder_module.get_decoder_norms()

    @property
    def log_threshold(self) -> Optional[torch.nn.Parameter]:
        tm = getattr(self, "theta_manager", None)
        return tm.log_threshold if tm is not None else None

    @log_threshold.setter
    def log_threshold(self, new_param: Optional[torch.nn.Parameter]) -> None:
        if getattr(self, "theta_manager", None) is None:
            raise AttributeError("ThetaManager is not initialised; cannot set log_threshold.")
        self.theta_manager.log_threshold = new_param

    @torch.no_grad()
    def estimate_theta_posthoc(self, data_iter, num_batches: Optional[int] = None, default_theta_value: float = 1e6,
                               device: Optional[torch.device] = None) -> torch.Tensor:
        """Estimate theta post-hoc using a specified number of batches (clt.py:282-307).  The
        estimation runs where the model lives; ``device`` is accepted for signature parity."""
        if device is not None and torch.device(device) != self.theta_manager.device:
            logger.info(f"Rank {self.rank}: theta estimation stays on {self.theta_manager.device} (asked for {device}).")
        return self.theta_manager.estimate_theta_posthoc(
            encode_all_layers_fn=self.encoder_module.encode_all_layers, data_iter=data_iter, num_batches=num_batches,
            default_theta_value=default_theta_value)

    @torch.no_grad()
    def convert_to_jumprelu_inplace(self, default_theta_value: float = 1e6) -> None:
        """BatchTopK / TokenTopK -> JumpReLU from the estimated statistics (clt.py:309-318); the
        ThetaManager updates the config object it shares with the model."""
        self.theta_manager.convert_to_jumprelu_inplace(default_theta_value=default_theta_value)
        logger.info(f"Rank {self.rank}: CLT model config updated by ThetaManager. New activation_fn='{self.config.activation_fn}'.")

    # ---- loss and gradients --------------------------------------------------------------------
    def _denorm_args(self, normalization_method, mean_tg, std_tg):
        """(mode, mean [L, d], std [L, d], scale) of the de-normalisation the reference's LossManager applies
        before the loss (losses.py:70-86): "mean_std" uses the target statistics of the layers that have them
        and leaves the others alone, as the reference does.  The method defaults to CLTConfig.normalization_method;
        the reference's LossManager reads TrainingConfig.normalization_method, which its trainer sets to the same
        value - pass ``normalization_method`` when the two differ."""
        cfg = self.config
        method = cfg.normalization_method if normalization_method is None else normalization_method
        L, d = cfg.num_layers, cfg.d_model
        if method == "mean_std":
            have = [l for l in range(L) if mean_tg and std_tg and l in mean_tg and l in std_tg]
            if not have:
                return "none", None, None, 1.0          # no statistics given: the reference leaves the tensors alone
            # a layer without statistics is left alone by the reference: mean 0 and std 1 do exactly that
            # (x * 1 + 0 is x in any dtype, and the gradient's factor is 1)
            mean = torch.zeros((L, d), device=self.device, dtype=self.dtype)
            std = torch.ones((L, d), device=self.device, dtype=self.dtype)
            for l in have:
                mean[l] = mean_tg[l].to(device=self.device, dtype=self.dtype).reshape(-1)[-d:]
                std[l] = std_tg[l].to(device=self.device, dtype=self.dtype).reshape(-1)[-d:]
            return "mean_std", mean, std, 1.0
        if method == "sqrt_d_model":
            return "sqrt_d_model", None, None, float(d) ** 0.5
        return "none", None, None, 1.0

    def _loss_and_raw_gradients(self, inputs: Dict[int, torch.Tensor], targets: Dict[int, torch.Tensor],
                                normalization_method: Optional[str] = None, mean_tg=None, std_tg=None,
                                decoder_step=None):
        """(per-layer losses [L] fp32, raw gradients): ``enc_w`` [L, F, d], ``enc_b`` [L, F],
        ``dec_w`` [n_dec, F, d] (feature-major, decoders in slot order: "s->t" pairs, or one per source /
        per target for tied decoders), ``dec_b`` [n_dec, d] (bias gradient of each decoder); all fp32."""
        cfg = self.config
        L, d, F = cfg.num_layers, cfg.d_model, cfg.num_features
        if sorted(inputs) != list(range(L)) or sorted(targets) != list(range(L)):
            raise ValueError("loss_and_gradients needs inputs and targets for every layer")
        dense = self._dense_threshold_activations(inputs, "dense_acts")
        if dense is not None:
            # a threshold model in the dense regime: no survivor list, forward and gradients on dense operands
            acts = dense[1]
            ws = self._workspace()
            dec = self.decoder_module
            skip = dec.skip_all_targets(inputs, (1 << L) - 1, acts.shape[1]) if cfg.skip_connection else None
            rec = dec._decode_dense_pairs(None, (1 << L) - 1, 0, L, ws, dense={l: acts[l] for l in range(L)}, skip_add=skip)
            dec.last_route = {"sparse_targets": (0, 0), "dense_targets": (0, L), "survivor_list": False}
            tgt = torch.stack([targets[l].to(device=self.device, dtype=self.dtype).reshape(-1, d) for l in range(L)])
            mode, mean, std, scale = self._denorm_args(normalization_method, mean_tg, std_tg)
            loss_l, g, g_model, bias_grad = engine.mse_loss_grad(rec, tgt.contiguous(), ws, mode, mean, std, scale)
            return loss_l, self._raw_gradients_dense(inputs, None, g, g_model, bias_grad, acts=acts)
        res = self._survivors(inputs)
        if res is None:
            raise ValueError("inputs do not form one [layers, tokens, d_model] batch")
        _, T, surv = res
        surv = surv.trimmed()      # buffers indexed by survivor are sized from the list: exact arrays (one read-back)
        ws = self._workspace()
        mask = (1 << L) - 1
        dec = self.decoder_module
        skip = dec.skip_all_targets(inputs, mask, T) if cfg.skip_connection else None
        rec = dec.decode_survivors(surv, mask, skip_add=skip, ws=ws)
        tgt = torch.stack([targets[l].to(device=self.device, dtype=self.dtype).reshape(-1, d) for l in range(L)])
        mode, mean, std, scale = self._denorm_args(normalization_method, mean_tg, std_tg)
        loss_l, g, g_model, bias_grad = engine.mse_loss_grad(rec, tgt.contiguous(), ws, mode, mean, std, scale)
        return loss_l, self._raw_gradients_from(inputs, surv, g, g_model, bias_grad, decoder_step)

    def _raw_gradients_from(self, inputs: Dict[int, torch.Tensor], surv, g: torch.Tensor, g_model: torch.Tensor,
                            bias_grad: torch.Tensor, decoder_step=None):
        """The raw parameter gradients (see ``_loss_and_raw_gradients``) of any loss, given d loss / d reconstruction:
        ``g`` fp32 [L, T, d], ``g_model`` the same in the model dtype, ``bias_grad`` [L, d] its sums over tokens.
        ``surv`` is the (trimmed) survivor list of the forward on ``inputs``."""
        cfg = self.config
        L, d, F = cfg.num_layers, cfg.d_model, cfg.num_features
        ws = self._workspace()
        mask = (1 << L) - 1
        dec = self.decoder_module
        affine = dec.feature_offset is not None or dec.feature_scale is not None
        too_wide = d > engine.BACKWARD_MAX_D_MODEL and not affine      # rows beyond what the list kernels hold per lane
        if L > MAX_LAYERS and affine:
            raise NotImplementedError(f"num_layers = {L} > {MAX_LAYERS} with a feature offset / scale: the gradients of "
                                      "such models come from the dense formulation, which does not cover them")
        if too_wide or dec.dense_pairs_wanted(surv, None, any_tying=True):
            # so many survivors that the reference's dense products are the cheaper formulation, or a d_model the
            # survivor-list kernels do not take (the decoder step is then not fused: ``dec_w`` is returned and the
            # optimiser applies it)
            return self._raw_gradients_dense(inputs, surv, g, g_model, bias_grad)
        off, sc = dec._affine()                     # per-target feature offset / scale of tied decoders, or None
        dval = engine.decode_backward_values(surv, dec.packed(), g, cfg.decoder_tying, mask, ws, feat_scale=sc)
        lists = engine.feature_lists(surv, ws)
        d_off, d_sc = (engine.feature_affine_grad(lists, surv, ws, off, sc, mask) if (off is not None or sc is not None)
                       else (None, None))
        # ``decoder_step`` (an optimiser whose ``fuses_decoder_step()`` holds): the decoder weights take their
        # step inside the weight-gradient kernel, after everything that reads the old decoders (below)
        dw_dec = None if decoder_step is not None else engine.decoder_weight_grad(lists, surv, g_model, cfg.decoder_tying, off, sc)
        _, x_slab, _, _ = self.encoder_module.prepare_slab(inputs)
        x_slab = x_slab.contiguous()
        dw_enc, db_enc = engine.encoder_weight_grad(lists, dval, x_slab, F)
        d_skip = None
        if dec.skip_weights is not None:
            # rec[t] += x[s] @ W_skip[s->t].T (untied, every pair) or x[t] @ W_skip[t].T (tied): dW = g[t].T @ x
            pairs = [(s_, t) for s_ in range(L) for t in range(s_, L)] if cfg.decoder_tying == "none" else [(t, t) for t in range(L)]
            d_skip = torch.empty((len(pairs), d, d), dtype=torch.float32, device=g.device)
            for i, (s_, t) in enumerate(pairs):
                engine.skip_weight_grad(g[t], x_slab[s_], d_skip[i])
        theta_grad = None
        if cfg.activation_fn == "jumprelu" and self.theta_manager.log_threshold is not None:
            theta_grad = self._log_threshold_gradient(x_slab, g_model, ws, surv, dval if sc is not None else None)
        if decoder_step is not None:
            decoder_step.decoder_weight_step(lists, surv, g_model)
        # bias_grad[t] = column sums of d loss / d rec[t]; a decoder's bias takes the rows of the targets
        # it is added to: its own pair's target, all targets >= its source, or its target (once)
        if cfg.decoder_tying == "none":
            dec_b = bias_grad[torch.tensor([t for s_ in range(L) for t in range(s_, L)], device=bias_grad.device)]
        elif cfg.decoder_tying == "per_source":
            dec_b = torch.flip(torch.cumsum(torch.flip(bias_grad, dims=[0]), dim=0), dims=[0])
        else:
            dec_b = bias_grad
        return {"enc_w": dw_enc, "enc_b": db_enc, "dec_w": dw_dec, "dec_b": dec_b.contiguous(), "theta": theta_grad,
                "skip": d_skip, "feat_offset": d_off, "feat_scale": d_sc}

    def _log_threshold_gradient(self, x_slab: torch.Tensor, g_model: torch.Tensor, ws, surv=None, dval=None) -> torch.Tensor:
        """fp32 [L, F] gradient of ``log_threshold`` (JumpReLU.backward, activations.py:196-199, through
        theta = exp(log_threshold), theta.py:70-79).  The band |x - theta| <= bandwidth / 2 holds elements
        on both sides of the threshold, so this part is dense: per source layer, d loss / d activation
        is one product of the stacked loss gradients [T, (L-s) d] with the stacked decoders [F, (L-s) d]
        on the MFMA kernel, reduced over tokens together with the dense pre-activations.  Behind a per-target
        feature scale (decoder.py:228-285: applied to the non-zero activations only) the kept elements of the
        band carry every target's scale: their entries of the product are replaced by ``dval``, the scaled
        value gradients of the survivor list; the elements below the threshold keep the plain product."""
        cfg = self.config
        L, F = cfg.num_layers, cfg.num_features
        tying = cfg.decoder_tying
        w, b = self.encoder_module.stacked()
        pre = engine.encode(x_slab.contiguous(), w, b, out=ws.typed("pre", tuple(x_slab.shape[:2]) + (F,), self.dtype))
        theta = self.theta_manager.thresholds(self.dtype)
        packed = self.decoder_module.packed()
        out = torch.empty((L, F), dtype=torch.float32, device=pre.device)
        T = g_model.shape[1]
        g_model = g_model.contiguous()
        dact_buf = ws.typed("theta_dact", (T, F), self.dtype)
        for s_ in range(L):
            dact = self._dense_activation_gradient(s_, g_model, packed, dact_buf)
            if dval is not None:
                engine.scatter_survivor_values(surv, dval, s_, dact)
            engine.jumprelu_theta_grad(pre[s_], dact, theta[s_].contiguous(), self.theta_manager.bandwidth, out[s_], ws)
        # theta = exp(log_threshold): the reference casts theta to the model dtype for the forward
        return out * torch.exp(self.theta_manager.log_threshold.detach().float())

    def _dense_activation_gradient(self, s_: int, g_model: torch.Tensor, packed: torch.Tensor,
                                   out: torch.Tensor) -> torch.Tensor:
        """d loss / d activation of source layer ``s_`` for every element, [T, F] in the model dtype: the product of
        the stacked loss gradients [T, (L-s) d] with the stacked decoders [F, (L-s) d] on the MFMA kernel (what
        autograd forms behind the reference's dense decode, decoder.py:253-338)."""
        cfg = self.config
        L, F, d, tying = cfg.num_layers, cfg.num_features, cfg.d_model, cfg.decoder_tying
        T, pitch = g_model.shape[1], packed.shape[2]
        piece = 64 if self.dtype == torch.bfloat16 else 32      # elements of K the matrix-core kernel takes at a time
        targets = list(range(s_, L))
        n = len(targets)
        if tying == "none":
            slots = [s_ * L - (s_ * (s_ - 1)) // 2 + (t - s_) for t in targets]
        elif tying == "per_source":
            slots = [s_] * n
        else:
            slots = targets
        if T >= 256 and F >= 256 and F % 4 == 0 and d % piece == 0 and (n * d // piece) % 2 == 0:
            # both operands where they lie: segment q = target s + q, in the gradient slab [L, T, d] and
            # in the packed decoders [n_dec, F, pitch] (one matrix for all targets when tied per source)
            return engine.encode_segmented(g_model[s_:], packed[slots[0]:], n, d, T * d, d,
                                           0 if tying == "per_source" else F * pitch, pitch, T, F, out=out)
        stacked_w = torch.cat([packed[i][:, :d] for i in slots], dim=1).unsqueeze(0)   # [1, F, n d]
        stacked_g = torch.cat([g_model[t] for t in targets], dim=1).unsqueeze(0)       # [1, T, n d]
        return engine.encode(stacked_g.contiguous(), stacked_w.contiguous(), None)[0]  # [T, F]

    def _raw_gradients_dense(self, inputs: Dict[int, torch.Tensor], surv, g: torch.Tensor, g_model: torch.Tensor,
                             bias_grad: torch.Tensor, acts: Optional[torch.Tensor] = None):
        """The raw gradients of ``_raw_gradients_from`` at densities the survivor-list kernels were not made for
        (``Decoder.dense_pairs_wanted``, any tying; no skip, no feature affine): autograd's own
        dense formulation behind the reference's dense forward, every product on the MFMA kernel -
        d loss / d activation per source (``_dense_activation_gradient``), gated by list membership (the
        straight-through rule of BatchTopK / TokenTopK, ``input >= threshold`` of JumpReLU, activations.py:68-96,
        192-194), ``dW_enc = dpre.T @ x``, ``dW_dec[s->t] = a[s].T @ g[t]``.  Products are rounded to the model
        dtype like the reference's autograd results, then kept in fp32.  ``acts`` [L, T, F]: dense activations of a
        threshold model in place of a survivor list (every kept element is non-zero there - it passed a positive
        threshold - so membership is ``acts != 0``)."""
        cfg = self.config
        L, d, F, tying = cfg.num_layers, cfg.d_model, cfg.num_features, cfg.decoder_tying
        T = surv.T if acts is None else acts.shape[1]
        ws = self._workspace()
        dec = self.decoder_module
        packed = dec.packed()
        dev = g.device
        _, x_slab, _, _ = self.encoder_module.prepare_slab(inputs)
        x_slab = x_slab.contiguous()
        g_model = g_model.contiguous()
        n_dec = len(dec._ordered())
        dw_dec = torch.empty((n_dec, F, d), dtype=torch.float32, device=dev)
        dw_enc = torch.empty((L, F, d), dtype=torch.float32, device=dev)
        db_enc = torch.empty((L, F), dtype=torch.float32, device=dev)
        if tying == "per_source":
            # one decoder per source serves every target >= s: its gradient takes the sum of their loss gradients
            g_t = torch.flip(torch.cumsum(torch.flip(g, dims=[0]), dim=0), dims=[0]).to(self.dtype)
        else:
            g_t = g_model
        summed = None       # per-target tying: the running sum of the sources' activations that target s multiplies
        g_t = g_t.transpose(1, 2).contiguous()                                 # [L, d, T]: K = tokens
        member = None
        if acts is None:
            member = SurvivorList(surv.row_ptr, surv.col, torch.ones_like(surv.val), surv.T, surv.F, surv.L, surv.dtype,
                                  surv.status, surv.nnz_hint)
        theta = pre = theta_out = None
        if cfg.activation_fn == "jumprelu" and self.theta_manager.log_threshold is not None:
            w, b = self.encoder_module.stacked()
            pre = engine.encode(x_slab, w, b, out=ws.typed("pre", (L, T, F), self.dtype))
            theta = self.theta_manager.thresholds(self.dtype)
            theta_out = torch.empty((L, F), dtype=torch.float32, device=dev)
        dact_buf = ws.typed("theta_dact", (T, F), self.dtype)
        a_buf = ws.typed("dense_sum", (T, F), self.dtype) if acts is None else None
        m_buf = ws.typed("dense_member", (T, F), self.dtype) if acts is None else None
        row0 = 0
        for s_ in range(L):
            dact = self._dense_activation_gradient(s_, g_model, packed, dact_buf)
            if theta_out is not None:
                engine.jumprelu_theta_grad(pre[s_], dact, theta[s_].contiguous(), self.theta_manager.bandwidth, theta_out[s_], ws)
            if acts is None:
                engine.accumulate_dense(member, s_, m_buf, True)
                dpre = dact * m_buf
            else:
                dpre = dact * (acts[s_] != 0)
            db_enc[s_] = dpre.sum(0, dtype=torch.float32)
            dw_enc[s_] = engine.encode(dpre.t().contiguous().unsqueeze(0), x_slab[s_].t().contiguous().unsqueeze(0), None)[0]
            del dpre
            if acts is None:
                engine.accumulate_dense(surv, s_, a_buf, True)
            a_s = a_buf if acts is None else acts[s_]
            if tying == "per_target":
                # decoder.py:208-246: ``summed_activation += activation_tensor`` in the model dtype, then one product
                summed = a_s.clone() if summed is None else summed.add_(a_s)
                a_s = summed
            a_t = a_s.t().contiguous()                                         # [F, T]
            if tying == "none":
                n = L - s_
                dw_dec[row0:row0 + n] = engine.encode(a_t.unsqueeze(0).expand(n, F, T), g_t[s_:], None)
                row0 += n
            else:
                dw_dec[s_] = engine.encode(a_t.unsqueeze(0), g_t[s_:s_ + 1], None)[0]
            del a_t
        theta_grad = None
        if theta_out is not None:
            theta_grad = theta_out * torch.exp(self.theta_manager.log_threshold.detach().float())
        if tying == "none":
            dec_b = bias_grad[torch.tensor([t for s_ in range(L) for t in range(s_, L)], device=bias_grad.device)]
        elif tying == "per_source":
            dec_b = torch.flip(torch.cumsum(torch.flip(bias_grad, dims=[0]), dim=0), dims=[0])
        else:
            dec_b = bias_grad
        d_skip = None
        if dec.skip_weights is not None:
            # rec[t] += x[s] @ W_skip[s->t].T (untied, every pair) or x[t] @ W_skip[t].T (tied): dW = g[t].T @ x
            pairs = [(s_, t) for s_ in range(L) for t in range(s_, L)] if tying == "none" else [(t, t) for t in range(L)]
            d_skip = torch.empty((len(pairs), d, d), dtype=torch.float32, device=dev)
            for i, (s_, t) in enumerate(pairs):
                engine.skip_weight_grad(g[t], x_slab[s_], d_skip[i])
        return {"enc_w": dw_enc, "enc_b": db_enc, "dec_w": dw_dec, "dec_b": dec_b.contiguous(), "theta": theta_grad,
                "skip": d_skip, "feat_offset": None, "feat_scale": None}

    @torch.no_grad()
    def loss_and_gradients(self, inputs: Dict[int, torch.Tensor], targets: Dict[int, torch.Tensor],
                           normalization_method: Optional[str] = None, mean_tg=None, std_tg=None):
        """MSE reconstruction loss (sum over layers of the per-layer mean, losses.py:45-92) and the
        gradients torch autograd gives the reference for it, computed from the survivor list:
        returns (loss [fp32 scalar tensor], {state-dict key: fp32 gradient in the parameter's shape}).
        Like the reference's LossManager, the loss is measured on de-normalised tensors:
        ``normalization_method`` (default: the config's) "mean_std" with the activation store's target
        statistics ``mean_tg`` / ``std_tg`` ({layer: tensor [d_model]}), "sqrt_d_model", or "none".
        Needs every layer present, equal token counts and a top-k or JumpReLU / ReLU activation; decoders
        untied or tied per source / per target, with or without skip connections and the per-target feature
        offset / scale (decoder.py:228-338)."""
        self._no_half("loss_and_gradients")
        L = self.config.num_layers
        loss_l, raw = self._loss_and_raw_gradients(inputs, targets, normalization_method, mean_tg, std_tg)
        return loss_l.sum(), self._named_gradients(raw)

    def _named_gradients(self, raw) -> Dict[str, Optional[torch.Tensor]]:
        """{state-dict key: fp32 gradient in the parameter's shape} from the raw gradient tensors."""
        L = self.config.num_layers
        grads: Dict[str, Optional[torch.Tensor]] = {}
        for l in range(L):
            grads[f"encoder_module.encoders.{l}.weight"] = raw["enc_w"][l]
            grads[f"encoder_module.encoders.{l}.bias_param"] = raw["enc_b"][l]
        if self.config.decoder_tying == "none":
            keys = [f"{s_}->{t}" for s_ in range(L) for t in range(s_, L)]
        else:
            keys = [str(i) for i in range(L)]
        for slot, key in enumerate(keys):
            grads[f"decoder_module.decoders.{key}.weight"] = raw["dec_w"][slot].t()   # [d, F] view
            grads[f"decoder_module.decoders.{key}.bias_param"] = raw["dec_b"][slot]
        if raw.get("theta") is not None:
            grads["theta_manager.log_threshold"] = raw["theta"]
        if raw.get("skip") is not None:
            for slot, key in enumerate(keys):
                grads[f"decoder_module.skip_weights.{key}"] = raw["skip"][slot]
        for name in ("feat_offset", "feat_scale"):
            if raw.get(name) is not None:
                for t in range(L):
                    grads[f"decoder_module.feature_{name[5:]}.{t}"] = raw[name][t]
        return grads

    @torch.no_grad()
    def training_step(self, inputs: Dict[int, torch.Tensor], targets: Dict[int, torch.Tensor], optimizer,
                      normalization_method: Optional[str] = None, mean_tg=None, std_tg=None) -> torch.Tensor:
        """One optimisation step on the MSE reconstruction loss (trainer.py:663-778 without the
        auxiliary losses): forward, gradients, ``optimizer.step``; returns the loss before the step.
        De-normalisation arguments as in ``loss_and_gradients``."""
        self._no_half("training_step")
        fuse = optimizer if getattr(optimizer, "fuses_decoder_step", lambda: False)() else None
        loss_l, raw = self._loss_and_raw_gradients(inputs, targets, normalization_method, mean_tg, std_tg, decoder_step=fuse)
        optimizer.step(raw)
        return loss_l.sum()

    # ---- encode (per-layer activations) ---------------------------------------------------
    def encode(self, x: torch.Tensor, layer_idx: int) -> torch.Tensor:
        """Activations [tokens, F] of one layer for relu / jumprelu; for the top-k family the
        reference logs an error and returns zeros here (clt.py:135-149), and so does this."""
        self._sync_device()
        x = x.to(device=self.device, dtype=self.dtype)
        preact = self.get_preactivations(x, layer_idx)
        F = self.config.num_features

        def zeros(rows: int) -> torch.Tensor:
            return torch.zeros((rows, F), device=self.device, dtype=self.dtype)

        if preact.numel() == 0:
            logger.warning(f"Rank {self.rank}: Received empty preactivations for encode layer {layer_idx}.")
            rows = x.shape[0] if x.dim() == 2 else x.shape[0] * x.shape[1] if x.dim() == 3 else 0
            return zeros(rows)
        if preact.shape[-1] != F:
            logger.warning(
                f"Rank {self.rank}: Received invalid preactivations shape {preact.shape} for encode layer {layer_idx}.")
            return zeros(preact.shape[0])
        fn = self.config.activation_fn
        try:
            if fn == "jumprelu":
                return self.theta_manager.jumprelu(preact, layer_idx)
            if fn == "relu":
                return get_activation_fn("relu")(self, preact, layer_idx)
            logger.error(
                f"Rank {self.rank}: Unsupported activation function '{fn}' encountered in encode method path. "
                f"Expected jumprelu or relu.")
        except ValueError as e:
            logger.error(f"Rank {self.rank}: Error getting activation function '{fn}' for layer {layer_idx}: {e}")
        return zeros(preact.shape[0])

    # ---- survivors: the fused encode + select ------------------------------------------------
    def _select(self, pre: torch.Tensor) -> SurvivorList:
        """Selection over a slab pre [n, T, F] of the layers present, per the config."""
        cfg = self.config
        ws = self._workspace()
        fn = cfg.activation_fn
        glob = cfg.topk_mode != "per_layer"
        if fn == "batchtopk":
            with self._timed("batchtopk_activation") as tm:
                # the reference times the mask computation inside its helper separately (activations.py:335-341)
                with self._timed("batchtopk_compute_mask") as tm_mask:
                    surv = engine.batchtopk_select(pre, int(cfg.batchtopk_k), glob, ws)
                self._record("batchtopk_compute_mask", tm_mask)
            self._record("batchtopk_activation", tm)
            return surv
        if fn == "topk":
            n, _, F = pre.shape
            kk = resolve_token_k(float(cfg.topk_k), n * F if glob else F)
            with self._timed("topk_activation") as tm:
                surv = engine.tokentopk_select(pre, kk, glob, ws)
            self._record("topk_activation", tm)
            return surv
        raise AssertionError(fn)

    def _survivors(self, inputs: Dict[int, torch.Tensor]):
        """(layers, T, survivor list over those layers) or None when the inputs need the
        reference's per-layer fallbacks."""
        self._sync_device()
        cfg = self.config
        layers = sorted(inputs.keys())
        if not layers:
            return None
        fn = cfg.activation_fn
        # pre-activation slab: reused scratch, it never leaves this function
        x0 = inputs[layers[0]]
        if x0.dim() not in (2, 3):
            return None
        T = x0.shape[0] if x0.dim() == 2 else x0.shape[0] * x0.shape[1]
        n = len(layers)
        ws = self._workspace()
        pre_buf = ws.typed("pre", (n, T, cfg.num_features), self.dtype) if T > 0 else None
        prep = self.encoder_module.prepare_slab(inputs)
        if prep is None:
            return None
        _, x_slab, w_slab, b_slab = prep
        if fn == "batchtopk" and cfg.topk_mode == "per_layer" and self.fuse_encode_select:
            # the encoder keeps only the candidates above a sampled cut; nothing dense is written
            k = int(cfg.batchtopk_k)
            if engine.encode_collect_supported(x_slab, w_slab, b_slab, k):
                with self._timed("batchtopk_activation") as tm:
                    surv = engine.collect_select(engine.encode_collect(x_slab, w_slab, b_slab, k, pre_buf, ws))
                self._record("batchtopk_activation", tm)
                return layers, T, surv
        if fn in ("jumprelu", "relu"):
            return layers, T, self._threshold_survivors(fn, layers, T, x_slab, w_slab, b_slab, pre_buf, ws)
        pre = engine.encode(x_slab, w_slab, b_slab, out=pre_buf)
        if fn in ("batchtopk", "topk"):
            surv = self._select(pre)
        else:
            return None
        return layers, T, surv

    # ---- threshold activations: exact survivor lists without a read-back ---------------------------------
    def _note_threshold_total(self, total: int, first: bool) -> None:
        """The candidate pool of the fused route follows the density seen: set from the first total of a
        shape, raised by a later one that comes close to it.  Only speed depends on it."""
        self._thr_last_total = total
        want = int(2e6 * total / max(1, self._thr_elems))
        if first:
            self._density_ppm = min(1000000, max(2000, want))
        elif want > self._density_ppm:
            self._density_ppm = min(1000000, want)

    def _poll_threshold_runs(self) -> None:
        """Look at the totals of earlier forwards whose copies have arrived (no waiting)."""
        keep = []
        for host, ev, key in self._thr_pending:
            if not ev.query():
                keep.append((host, ev, key))
                continue
            if key == self._thr_key and int(host[0]) >= 0:
                self._note_threshold_total(int(host[0]), self._thr_last_total is None)
        self._thr_pending = keep

    def _threshold_reads_back(self, n: int, T: int, F: int) -> bool:
        budget = self.threshold_list_budget_bytes
        if budget is None:
            budget = torch.cuda.get_device_properties(self.device).total_memory // 8
        item = torch.empty((), dtype=self.dtype).element_size()
        return engine.max_list_entries(n, T, F) * (4 + item) > budget

    def _threshold_survivors(self, fn: str, layers: List[int], T: int, x_slab, w_slab, b_slab, pre_buf, ws) -> SurvivorList:
        """JumpReLU / ReLU survivors (clt.py:271-277, theta.py:70-79).  The number of survivors depends on the
        data.  When arrays for the largest list the shape can produce are affordable, col / val get that size
        and the forward is a pure sequence of launches on the current stream: the fused route collects into a
        pool sized from the density seen so far, and a batch that outgrows the pool is redone by the device
        itself on the dense route (engine.encode_threshold), so the list is exact for any batch.  Otherwise
        the total is read back once per forward and the arrays are sized exactly."""
        cfg = self.config
        n, F = len(layers), cfg.num_features
        key = (fn, tuple(layers), T, self.dtype)
        if key != self._thr_key:
            self._thr_key, self._thr_pending, self._thr_last_total = key, [], None
        self._thr_elems = n * T * F
        # under stream capture (a HIP graph of the forward) nothing may be asked of events or copied for the host:
        # the pool keeps the size it has, which only speed depends on
        capturing = torch.cuda.is_current_stream_capturing()
        if not capturing:
            self._poll_threshold_runs()
        theta = None
        if fn == "jumprelu":
            theta = self.theta_manager.thresholds(self.dtype)
            if layers != list(range(cfg.num_layers)):
                theta = theta.index_select(0, torch.tensor(layers, device=theta.device)).contiguous()
        read_back = pre_buf is None or self._threshold_reads_back(n, T, F)
        surv = None
        if fn == "jumprelu" and self.fuse_encode_select:
            # thresholds applied in the encoder epilogue; the pool is sized from the density seen so far
            surv = engine.encode_threshold(x_slab, w_slab, b_slab, theta, ws, self._density_ppm,
                                           pre_scratch=None if read_back else pre_buf)
            if surv is None and read_back:
                self._density_ppm = min(1000000, 4 * self._density_ppm)
        if surv is None:
            pre = engine.encode(x_slab, w_slab, b_slab, out=pre_buf)
            surv = engine.threshold_select(pre, theta, nat.PRED_GE_THETA if fn == "jumprelu" else nat.PRED_GT_ZERO, ws,
                                           read_back=read_back)
        if surv.status is None:
            self._note_threshold_total(int(surv.nnz_hint), self._thr_last_total is None)
        elif capturing:
            surv.nnz_hint = self._thr_last_total
        else:
            # the total travels to pinned memory behind the kernels; a later forward looks at it
            surv.nnz_hint = self._thr_last_total
            host = torch.empty(1, dtype=torch.int32, pin_memory=True)
            host.copy_(surv.row_ptr[-1:], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            self._thr_pending.append((host, ev, key))
        return surv

    def _expand_layers(self, layers: List[int], surv: SurvivorList) -> SurvivorList:
        """Re-index a list over the present layers to all num_layers (absent layers: empty rows)."""
        L, T = self.config.num_layers, surv.T
        if layers == list(range(L)):
            return surv
        counts = torch.zeros(L * T, dtype=torch.int64, device=surv.row_ptr.device)
        per_row = (surv.row_ptr[1:] - surv.row_ptr[:-1]).to(torch.int64)
        for i, l in enumerate(layers):
            counts[l * T:(l + 1) * T] = per_row[i * T:(i + 1) * T]
        row_ptr = torch.zeros(L * T + 1, dtype=torch.int32, device=counts.device)
        row_ptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
        return SurvivorList(row_ptr, surv.col, surv.val, T, surv.F, L, surv.dtype, surv.status, surv.nnz_hint)

    # ---- get_feature_activations -------------------------------------------------------------
    def get_feature_activations(self, inputs: Dict[int, torch.Tensor]) -> Dict[int, torch.Tensor]:
        """Dense activations per layer (clt.py:220-277)."""
        self._sync_device()
        self._note_no_graph("get_feature_activations")
        cfg = self.config
        topk_family = cfg.activation_fn in ("batchtopk", "topk")
        got = self._dense_threshold_activations(inputs, "pre")
        if got is not None:
            # a threshold model in the dense regime: the gated pre-activations are the answer (fp32 for JumpReLU, as
            # the reference's ``(x >= theta).float() * x`` is)
            layers, acts = got
            dense = acts.float() if cfg.activation_fn == "jumprelu" else acts.clone()
            return {l: dense[i] for i, l in enumerate(layers)}
        res = self._survivors(inputs)
        if res is not None:
            layers, T, surv = res
            dense = engine.densify(surv, out_f32=(cfg.activation_fn == "jumprelu"))
            if surv.status is not None:
                engine.poison_if(dense, surv.status)      # a batch no list can hold: NaN, never zeros
            return {l: dense[i] for i, l in enumerate(layers)}
        # inputs that need the per-layer fallbacks
        proc = {l: x.to(device=self.device, dtype=self.dtype) for l, x in inputs.items()}
        if not topk_family:
            return {l: self.encode(proc[l], l) for l in sorted(proc.keys())}
        return self._topk_from_preacts(inputs, proc)

    def _topk_from_preacts(self, inputs, proc) -> Dict[int, torch.Tensor]:
        """Top-k family when some layer took a fallback: follows the helper's zero-filling of
        empty or mismatched layers (activations.py:250-297) on a stacked copy."""
        cfg = self.config
        F = cfg.num_features
        pre_dict, _ = self._encode_all_layers(proc)
        if not pre_dict:
            out = {}
            for l, x in inputs.items():
                rows = x.shape[0] * x.shape[1] if x.dim() == 3 else x.shape[0] if x.dim() == 2 else 0
                out[l] = torch.zeros((rows, F), device=self.device, dtype=self.dtype)
            return out
        first = next((p for p in pre_dict.values() if p.numel() > 0), None)
        if first is None:
            logger.warning(f"Rank {self.rank}: No valid preactivations found in dict for BatchTopK. Returning empty dict.")
            return {l: torch.empty((0, F), device=self.device, dtype=self.dtype) for l in pre_dict}
        T = first.shape[0]
        layers = [l for l in range(cfg.num_layers) if l in pre_dict]
        slabs = []
        for l in layers:
            p = pre_dict[l]
            if p.numel() == 0:
                p = torch.zeros((T, F), device=self.device, dtype=self.dtype)
            elif p.shape[0] != T:
                logger.warning(
                    f"Rank {self.rank} Layer {l}: Mismatched batch dim ({p.shape[0]} vs {T}). Using zeros.")
                p = torch.zeros((T, F), device=self.device, dtype=self.dtype)
            slabs.append(p)
        if not layers:
            return {l: torch.empty((T, F), device=self.device, dtype=self.dtype) for l in pre_dict}
        pre = torch.stack(slabs).contiguous()
        dense = engine.densify(self._select(pre))
        return {l: dense[i] for i, l in enumerate(layers)}

    # ---- forward ---------------------------------------------------------------------------
    def forward_with_survivors(self, inputs: Dict[int, torch.Tensor]):
        """(reconstructions, survivor list over all num_layers) from one pass, or None when the inputs
        need the per-layer fallbacks.  The list is what get_feature_activations would densify; the
        evaluator and the dead-feature counters read it directly."""
        cfg = self.config
        L = cfg.num_layers
        res = self._survivors(inputs)
        if res is None:
            return None
        layers, T, surv = res
        full = self._expand_layers(layers, surv)
        src_mask = 0
        for l in layers:
            src_mask |= 1 << l
        skip = (self.decoder_module.skip_all_targets(inputs, src_mask, T) if cfg.skip_connection else None)
        targets = [t for t in range(L) if t in inputs]
        out = self.decoder_module.decode_survivors(full, src_mask, min(targets), max(targets) + 1, skip_add=skip,
                                                   ws=self._workspace())
        if full.status is not None:
            # a threshold batch with more survivors than a list can hold has no reconstruction here: the
            # device overwrites the output with NaN rather than leave what an empty list decodes to
            engine.poison_if(out, full.status)
        return {t: out[t] for t in targets}, full

    def _dense_threshold_activations(self, inputs: Dict[int, torch.Tensor], buffer: str):
        """(layers, dense activations [n, T, F] in workspace buffer ``buffer``) of a JumpReLU / ReLU model when the
        survivor total last seen for this shape sends the decode to its dense products, else None."""
        cfg = self.config
        fn = cfg.activation_fn
        if fn not in ("jumprelu", "relu") or torch.cuda.is_current_stream_capturing():
            return None
        if self._thr_last_total is None or not inputs:
            return None
        # the cheap questions first: this is asked on every forward of a threshold model
        x0 = next(iter(inputs.values()))
        if not isinstance(x0, torch.Tensor) or x0.dim() not in (2, 3):
            return None
        n, T, F = len(inputs), x0.numel() // max(1, x0.shape[-1]), cfg.num_features
        key = (fn, tuple(sorted(inputs)), T, self.dtype)
        if key != self._thr_key:
            return None
        self._poll_threshold_runs()
        if self._thr_last_total is None:
            return None
        if not self.decoder_module.dense_pairs_wanted_for(self._thr_last_total / n, T, self.dtype, None):
            return None
        prep = self.encoder_module.prepare_slab(inputs)
        if prep is None:
            return None
        layers, x_slab, w_slab, b_slab = prep
        if x_slab.shape[1] != T:
            return None
        pre = engine.encode(x_slab, w_slab, b_slab, out=self._workspace().typed(buffer, (n, T, F), self.dtype))
        theta = None
        if fn == "jumprelu":
            theta = self.theta_manager.thresholds(self.dtype)
            if layers != list(range(cfg.num_layers)):
                theta = theta.index_select(0, torch.tensor(layers, device=theta.device)).contiguous()
        total = engine.threshold_dense(pre, theta, nat.PRED_GE_THETA if fn == "jumprelu" else nat.PRED_GT_ZERO)
        host = torch.empty(1, dtype=torch.int64, pin_memory=True)
        host.copy_(total, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._thr_pending.append((host, ev, key))
        return layers, pre

    def _forward_dense_thresholds(self, inputs: Dict[int, torch.Tensor]) -> Optional[Dict[int, torch.Tensor]]:
        """The forward of a JumpReLU / ReLU model whose recent batches were dense enough for the decode to run as
        dense products (``Decoder.dense_pairs_wanted_for`` on the survivor total last seen for this shape): no
        survivor list is made at all - the pre-activations are stored, gated in place (``clt_threshold_dense``) and
        multiplied as they are; the number kept travels to the host behind the kernels like the list totals do,
        so the route follows the density back down.  None: the list route is the one to take."""
        got = self._dense_threshold_activations(inputs, "pre")
        if got is None:
            return None
        layers, pre = got
        dec = self.decoder_module
        ws = self._workspace()
        src_mask = 0
        for l in layers:
            src_mask |= 1 << l
        skip = dec.skip_all_targets(inputs, src_mask, pre.shape[1]) if self.config.skip_connection else None
        out = dec._decode_dense_pairs(None, src_mask, min(layers), max(layers) + 1, ws,
                                      dense={l: pre[i] for i, l in enumerate(layers)}, skip_add=skip)
        dec.last_route = {"sparse_targets": (min(layers), min(layers)), "dense_targets": (min(layers), max(layers) + 1),
                          "survivor_list": False}
        return {t: out[t] for t in layers}

    def _note_no_graph(self, what: str) -> None:
        """Say once per model that ``what`` returns tensors outside the autograd graph although gradients are on:
        a loss term built on them (the reference's sparsity / pre-activation penalties, losses.py:94-328) would
        silently contribute nothing to ``param.grad``."""
        if torch.is_grad_enabled() and not self.__dict__.get("_told_no_graph", {}).get(what):
            if any(p.requires_grad for p in self.encoder_module.parameters()):
                self.__dict__.setdefault("_told_no_graph", {})[what] = True
                logger.warning(f"Rank {self.rank}: {what} returns tensors without an autograd graph; only forward() is "
                               f"differentiable here. Loss terms built on {what} add nothing to the gradients.")

    def _graph_route_ok(self, inputs: Dict[int, torch.Tensor]) -> bool:
        """Whether the gradient kernels take this batch: every layer present, one token count, right width."""
        cfg = self.config
        if sorted(inputs) != list(range(cfg.num_layers)):
            return False
        counts = set()
        for x in inputs.values():
            if not isinstance(x, torch.Tensor) or x.dim() not in (2, 3) or x.shape[-1] != cfg.d_model or x.numel() == 0:
                return False
            counts.add(x.numel() // cfg.d_model)
        return len(counts) == 1 and cfg.activation_fn in ("batchtopk", "topk", "jumprelu", "relu")

    def forward(self, inputs: Dict[int, torch.Tensor]) -> Dict[int, torch.Tensor]:
        """Reconstruction of every layer present in ``inputs`` (clt.py:186-218).  With gradients enabled and
        parameters that ask for them the result carries an autograd graph, as the reference's does: ``loss.backward()``
        on any function of the reconstructions fills ``param.grad`` (inputs of every layer with equal token counts;
        float32 / bfloat16)."""
        self._sync_device()
        cfg = self.config
        L, d = cfg.num_layers, cfg.d_model
        if torch.is_grad_enabled() and self.dtype != torch.float16:
            named = list(self.named_parameters())
            if any(p.requires_grad for _, p in named):
                if self._graph_route_ok(inputs):
                    outs = _ReconstructionsWithGraph.apply(self, inputs, [n for n, _ in named], *[p for _, p in named])
                    return {l: outs[l] for l in range(L)}
                if not getattr(self, "_warned_no_graph", False):
                    self._warned_no_graph = True
                    logger.warning(f"Rank {self.rank}: forward builds no autograd graph for these inputs (it needs one "
                                   f"2-D or 3-D tensor per layer with equal token counts); gradients will not flow.")
        dense = self._forward_dense_thresholds(inputs)
        if dense is not None:
            return dense
        res = self.forward_with_survivors(inputs)
        if res is not None:
            return res[0]
        # fallback wiring over dense activations
        acts = self.get_feature_activations(inputs)
        recs: Dict[int, torch.Tensor] = {}
        for t in range(L):
            rel = {s: v for s, v in acts.items() if s <= t and v.numel() > 0}
            if t in inputs and rel:
                src = {s: inputs[s] for s in range(t + 1) if s in inputs} if cfg.skip_connection else None
                recs[t] = self.decode(rel, t, src)
            elif t in inputs:
                x = inputs[t]
                rows = 0
                if x.dim() >= 1:
                    rows = x.shape[0] * x.shape[1] if x.dim() == 3 else x.shape[0]
                else:
                    logger.warning(
                        f"Rank {self.rank}: Could not determine batch size for fallback tensor in forward layer "
                        f"{t} from input shape {x.shape}. Using 0.")
                recs[t] = torch.zeros((rows, d), device=self.device, dtype=self.dtype)
        return recs

    # ---- parameters that an optimiser step may have left behind the kernels' working copy ------------------
    def named_parameters(self, *args, **kwargs):
        self.decoder_module.sync_parameters()
        return super().named_parameters(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self.decoder_module.sync_parameters()
        return super()._apply(fn, *args, **kwargs)

    # ---- checkpoints -----------------------------------------------------------------------
    def load_state_dict(self, state_dict: Dict[str, torch.Tensor], strict: bool = True):
        """nn.Module.load_state_dict plus the reference's migrations (clt.py:347-425): an untied
        checkpoint loaded into a per_source model keeps the diagonal "s->s" decoders, and
        feature_offset / feature_scale saved under encoder_module move to decoder_module."""
        sd = dict(state_dict)
        if self.config.decoder_tying == "per_source" and any("decoders." in k and "->" in k for k in sd):
            logger.warning(
                "Loading old untied decoder checkpoint into tied decoder model. "
                "This will use weights from the first target layer for each source layer.")
            new_sd = {}
            for k, v in sd.items():
                if "decoders." in k and "->" in k:
                    parts = k.split(".")
                    i = parts.index("decoders") + 1
                    s, t = (int(p) for p in parts[i].split("->"))
                    if s == t:
                        new_sd[".".join(parts[:i] + [str(s), parts[-1]])] = v
                else:
                    new_sd[k] = v
            sd = new_sd
        for i in range(self.config.num_layers):
            for name in ("feature_offset", "feature_scale"):
                old, new = f"encoder_module.{name}.{i}", f"decoder_module.{name}.{i}"
                if old in sd and new not in sd:
                    logger.info(f"Migrating {old} to {new}")
                    sd[new] = sd.pop(old)
        result = super().load_state_dict(sd, strict=strict)
        self.decoder_module.invalidate_packed()
        return result
