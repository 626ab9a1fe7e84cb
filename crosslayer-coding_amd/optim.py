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

    @torch.no_grad()
    def decoder_weight_step(self, lists, surv, g_model) -> None:
        """The decoder weights' part of the NEXT ``step`` (which must follow with ``raw["dec_w"] = None``), taken
        straight from the survivor lists: gradient rows go from registers into the update of the moments and
        of the packed copy; the checkpoint-layout parameters are then rewritten from the packed copy."""
        from . import engine
        dec = self.model.decoder_module
        packed = dec.packed()
        ws = [lin.weight.data for lin in dec._ordered()]
        assert all(w.is_contiguous() and w.shape == ws[0].shape and w.dtype == ws[0].dtype for w in ws)
        d, F = ws[0].shape
        m_w, v_w = self.state["dec_w"]
        engine.decoder_weight_grad_adam(lists, surv, g_model, packed, m_w, v_w, self.lr, self.betas, self.eps,
                                        self.step_count + 1)
        w_dev, w_host = self._pointer_table("w", ws)
        engine.unpack_decoders(packed, w_dev, w_host, d, F)

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
