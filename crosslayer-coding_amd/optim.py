"""Adam for the transcoder's encoder / decoder parameters, driven by the sparse gradients of
``CrossLayerTranscoder.loss_and_gradients``.

The reference trains with ``torch.optim.Adam`` / ``AdamW`` over autograd gradients
(clt/training/trainer.py:290-312, 751-778).  Here the moments are fp32 whatever the parameter dtype,
the decoder moments live in the feature-major layout of the gradients, and one kernel per decoder
matrix updates the checkpoint-layout parameter and its feature-major working copy together, so no
repacking follows a step.  Semantics: torch.optim.Adam without weight decay or amsgrad.
"""

from __future__ import annotations

import ctypes
from typing import Dict, Tuple

import torch

from . import _native as nat


class CLTAdam:
    def __init__(self, model, lr: float = 1e-4, betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-8):
        self.model = model
        self.lr, self.betas, self.eps = float(lr), (float(betas[0]), float(betas[1])), float(eps)
        self.step_count = 0
        self.fuse_decoder_step = True    # untied decoders: Adam inside the weight-gradient kernel (training_step)
        self.tile_decoder_step = True    # ... over column tiles, when the shape allows (moments and a weight copy tiled)
        # the in-kernel decoder step rewrites the feature-major slab only; the checkpoint-layout parameters follow
        # when something reads them (Decoder.sync_parameters).  False: rewrite them in every step
        self.defer_parameter_sync = True
        self._dec_layout = "rows"        # layout of state["dec_w"]: "rows" [n_dec, F, d] or "tiles" [n_dec, d // CS, F, CS]
        self._w_tiles = None             # tiled copy of the decoder weights, valid while _w_tiles_gen matches the slab
        self._w_tiles_gen = None
        cfg = model.config
        L, F, d = cfg.num_layers, cfg.num_features, cfg.d_model
        dev = model.device
        n_dec = L * (L + 1) // 2 if cfg.decoder_tying == "none" else L
        z = lambda *shape: torch.zeros(shape, dtype=torch.float32, device=dev)   # noqa: E731
        self._tables: Dict[str, tuple] = {}
        self.state: Dict[str, Tuple[torch.Tensor, torch.Tensor]] = {
            "enc_w": (z(L, F, d), z(L, F, d)), "enc_b": (z(L, F), z(L, F)),
            "dec_w": (z(n_dec, F, d), z(n_dec, F, d)), "dec_b": (z(n_dec, d), z(n_dec, d)),
        }
        if cfg.activation_fn == "jumprelu" and model.theta_manager.log_threshold is not None:
            self.state["theta"] = (z(L, F), z(L, F))
        dec = model.decoder_module
        if dec.skip_weights is not None:
            self.state["skip"] = (z(len(dec.skip_weights), d, d), z(len(dec.skip_weights), d, d))
        if dec.feature_offset is not None:
            self.state["feat_offset"] = (z(L, F), z(L, F))
        if dec.feature_scale is not None:
            self.state["feat_scale"] = (z(L, F), z(L, F))

    def _adam(self, param: torch.Tensor, grad: torch.Tensor, m: torch.Tensor, v: torch.Tensor) -> None:
        assert param.is_contiguous() and grad.is_contiguous() and grad.dtype == torch.float32 and grad.numel() == param.numel()
        code = nat.load().clt_adam_step(nat.ptr(param), nat.ptr(grad), nat.ptr(m), nat.ptr(v), param.numel(), self.lr,
                                        self.betas[0], self.betas[1], self.eps, self.step_count,
                                        nat.dtype_code(param.dtype), nat.current_stream(param.device))
        nat.check(code, "clt_adam_step")

    def _pointer_table(self, key: str, tensors):
        """(device int64 tensor, host ctypes array) holding the data pointers of ``tensors``."""
        ptrs = tuple(t.data_ptr() for t in tensors)
        ent = self._tables.get(key)
        if ent is None or ent[0] != ptrs:
            host = (ctypes.c_void_p * len(ptrs))(*ptrs)
            dev = torch.tensor(ptrs, dtype=torch.int64, device=tensors[0].device)
            ent = (ptrs, dev, host)
            self._tables[key] = ent
        return ent[1], ent[2]

    def fuses_decoder_step(self) -> bool:
        """Whether the decoder weights can take their Adam step inside the weight-gradient kernel: untied
        decoders without the per-target feature offset / scale (``fuse_decoder_step = False`` switches it off)."""
        dec = self.model.decoder_module
        return (self.fuse_decoder_step and self.model.config.decoder_tying == "none"
                and dec.feature_offset is None and dec.feature_scale is None)

    def _decoder_moments_to(self, layout: str) -> None:
        """Regroup both decoder moments: "rows" [n_dec, F, d] <-> "tiles" [n_dec, d // CS, F, CS] (CS = 32 bytes of
        the model dtype).  Happens when the route of the decoder step changes, normally once."""
        if layout == self._dec_layout:
            return
        cfg = self.model.config
        F, d = cfg.num_features, cfg.d_model
        cs = 32 // self.model.decoder_module._ordered()[0].weight.element_size()
        out = []
        for t in self.state["dec_w"]:
            n_dec = t.shape[0]
            if layout == "tiles":
                out.append(t.view(n_dec, F, d // cs, cs).permute(0, 2, 1, 3).contiguous())
            else:
                out.append(t.permute(0, 2, 1, 3).contiguous().view(n_dec, F, d))
            del t
        self.state["dec_w"] = tuple(out)
        self._dec_layout = layout

    def decoder_moments(self):
        """(m, v) of the decoder weights as [n_dec, F, d] whatever layout the optimiser keeps them in."""
        m, v = self.state["dec_w"]
        if self._dec_layout == "rows":
            return m, v
        n_dec, ns, F, cs = m.shape
        return tuple(t.permute(0, 2, 1, 3).contiguous().view(n_dec, F, ns * cs) for t in (m, v))

    @torch.no_grad()
    def decoder_weight_step(self, lists, surv, g_model) -> None:
        """The decoder weights' part of the NEXT ``step`` (which must follow with ``raw["dec_w"] = None``), taken
        straight from the survivor lists: gradient rows go from registers into the update of the moments and
        of the working copy of the weights; the checkpoint-layout parameters are then rewritten from that copy.
        Two routes: over column tiles (tiled moments and a tiled weight copy, the gather of d loss /
        d reconstruction served from LDS) when ``engine.decoder_tile_width`` takes the shape, else row by row on
        the feature-major slab.  The row route is bit-identical to gradient-then-Adam; the tile route sums the
        lists it cuts between lanes in another fixed association (equal to fp32 rounding, repeatable)."""
        from . import engine
        dec = self.model.decoder_module
        packed = dec.packed()
        ws = [lin.weight.data for lin in dec._ordered()]
        assert all(w.is_contiguous() and w.shape == ws[0].shape and w.dtype == ws[0].dtype for w in ws)
        d, F = ws[0].shape
        w_dev, w_host = self._pointer_table("w", ws)
        cs = engine.decoder_tile_width(surv.T, d, F, ws[0].dtype) if self.tile_decoder_step else 0
        if cs and all(w.data_ptr() % 16 == 0 for w in ws):
            self._decoder_moments_to("tiles")
            dec._derived_copies = True      # the packed copy tells when the device may have repacked it
            if self._w_tiles is None or self._w_tiles_gen != dec.packed_generation():
                self._w_tiles = engine.tile_decoders(packed, d, out=self._w_tiles)
                self._w_tiles_gen = dec.packed_generation()
            m_w, v_w = self.state["dec_w"]
            engine.decoder_weight_grad_adam_tiled(lists, surv, g_model, self._w_tiles, m_w, v_w, self.lr, self.betas,
                                                  self.eps, self.step_count + 1, ws=self.model._workspace())
            if self.defer_parameter_sync:
                engine.untile_decoders(self._w_tiles, packed)
                dec.mark_parameters_behind()
            else:
                engine.untile_decoders(self._w_tiles, packed, w_dev, w_host)
                dec.note_parameters_written()
            return
        self._decoder_moments_to("rows")
        self._w_tiles_gen = None
        m_w, v_w = self.state["dec_w"]
        engine.decoder_weight_grad_adam(lists, surv, g_model, packed, m_w, v_w, self.lr, self.betas, self.eps,
                                        self.step_count + 1)
        if self.defer_parameter_sync:
            dec.mark_parameters_behind()
        else:
            engine.unpack_decoders(packed, w_dev, w_host, d, F)
            dec.note_parameters_written()

    @torch.no_grad()
    def step(self, raw) -> None:
        """``raw``: the gradient tensors of ``CrossLayerTranscoder._loss_and_raw_gradients``; ``dec_w`` is None
        when ``decoder_weight_step`` has already applied it."""
        model = self.model
        self.step_count += 1
        w_slab, b_slab = model.encoder_module.stacked()
        self._adam(w_slab, raw["enc_w"], *self.state["enc_w"])
        self._adam(b_slab, raw["enc_b"], *self.state["enc_b"])
        dec = model.decoder_module
        packed = dec.packed()
        decs = dec._ordered()
        lib = nat.load()
        m_w, v_w = self.state["dec_w"]
        m_b, v_b = self.state["dec_b"]
        # all decoder matrices in one launch, all decoder biases in another: the parameters are separate
        # tensors, so the kernels get their addresses as a device array (rebuilt only when one has moved)
        ws = [lin.weight.data for lin in decs]
        bs = [lin.bias_param.data for lin in decs]
        assert all(w.is_contiguous() and w.shape == ws[0].shape and w.dtype == ws[0].dtype for w in ws)
        assert all(b.is_contiguous() and b.numel() == bs[0].numel() and b.dtype == bs[0].dtype for b in bs)
        d, F = ws[0].shape
        if raw["dec_w"] is not None:
            dec.sync_parameters()         # the two-copy kernel below reads neither copy's old value from the other
            self._decoder_moments_to("rows")
            self._w_tiles_gen = None      # the slab is about to change under the tiled copy
            m_w, v_w = self.state["dec_w"]
            assert packed.is_contiguous() and raw["dec_w"].is_contiguous() and raw["dec_w"].dtype == torch.float32
            from . import engine
            assert tuple(raw["dec_w"].shape) == (len(ws), F, d)
            assert tuple(packed.shape) == (len(ws), F, engine.decoder_pitch(d, ws[0].dtype))
            w_dev, w_host = self._pointer_table("w", ws)
            code = lib.clt_adam_step_decoders(nat.ptr(w_dev), ctypes.addressof(w_host), len(ws), nat.ptr(packed),
                                              nat.ptr(raw["dec_w"]), nat.ptr(m_w), nat.ptr(v_w), d, F, self.lr,
                                              self.betas[0], self.betas[1], self.eps, self.step_count,
                                              nat.dtype_code(ws[0].dtype), nat.current_stream(ws[0].device))
            nat.check(code, "clt_adam_step_decoders")
        b_dev, _ = self._pointer_table("b", bs)
        assert raw["dec_b"].is_contiguous() and raw["dec_b"].dtype == torch.float32
        code = lib.clt_adam_step_many(nat.ptr(b_dev), nat.ptr(raw["dec_b"]), nat.ptr(m_b), nat.ptr(v_b), len(bs),
                                      bs[0].numel(), self.lr, self.betas[0], self.betas[1], self.eps, self.step_count,
                                      nat.dtype_code(bs[0].dtype), nat.current_stream(bs[0].device))
        nat.check(code, "clt_adam_step_many")
        if raw.get("theta") is not None and "theta" in self.state:
            self._adam(model.theta_manager.log_threshold.data, raw["theta"].contiguous(), *self.state["theta"])
        # skip matrices and per-target feature offset / scale: separate small tensors, one launch per family
        if dec.skip_weights is not None:
            skips = list(dec.skip_weights.values()) if hasattr(dec.skip_weights, "values") else list(dec.skip_weights)
        else:
            skips = None
        for key, params in (("skip", skips),
                            ("feat_offset", list(dec.feature_offset) if dec.feature_offset is not None else None),
                            ("feat_scale", list(dec.feature_scale) if dec.feature_scale is not None else None)):
            if params is None or raw.get(key) is None or key not in self.state:
                continue
            ps = [p.data for p in params]
            assert all(p.is_contiguous() and p.numel() == ps[0].numel() and p.dtype == ps[0].dtype for p in ps)
            grad = raw[key].contiguous()
            assert grad.dtype == torch.float32 and grad.numel() == len(ps) * ps[0].numel()
            p_dev, _ = self._pointer_table(key, ps)
            m_p, v_p = self.state[key]
            code = lib.clt_adam_step_many(nat.ptr(p_dev), nat.ptr(grad), nat.ptr(m_p), nat.ptr(v_p), len(ps), ps[0].numel(),
                                          self.lr, self.betas[0], self.betas[1], self.eps, self.step_count,
                                          nat.dtype_code(ps[0].dtype), nat.current_stream(ps[0].device))
            nat.check(code, "clt_adam_step_many")
        # the kernels wrote through .data: caches keyed on version counters would not notice
        dec._bias_cache.clear()
        dec._cached_decoder_norms = None
        dec.note_parameters_written()
