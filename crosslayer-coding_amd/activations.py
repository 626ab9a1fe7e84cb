"""BatchTopK / TokenTopK / JumpReLU operators backed by the HIP selection kernels.

Same call surface as the reference's autograd Functions
(clt/models/activations.py:9-220): ``X.apply(...)`` and the static
``X._compute_mask(...)`` helpers.  Forward runs the radix-select / threshold kernels;
the backward rules are the reference's (straight-through mask for the top-k family,
rectangle-window threshold gradient for JumpReLU) written with elementwise torch ops.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _native as nat
from . import engine


def _mask_from_survivors(surv: engine.SurvivorList, shape) -> torch.Tensor:
    rows = engine.survivor_rows(surv)
    flat = rows * surv.F + surv.col.to(torch.int64)
    mask = torch.zeros(surv.L * surv.T * surv.F, dtype=torch.bool, device=surv.col.device)
    mask[flat] = True
    return mask.view(shape)


def _as_block(t: torch.Tensor) -> torch.Tensor:
    """[B, F] tensor as a one-layer [1, B, F] slab the kernels accept."""
    if t.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        t = t.to(torch.float32)
    return t.detach().contiguous().unsqueeze(0)


def resolve_token_k(k_float: float, f_total: int) -> int:
    """k rule of TokenTopK (activations.py:108-116): fraction -> ceil, count -> int, capped."""
    if f_total == 0 or k_float <= 0:
        return 0
    if 0 < k_float < 1:
        kk = int(torch.ceil(torch.tensor(k_float * f_total)).item())
    else:
        kk = int(k_float)
    return min(kk, f_total)


class BatchTopK(torch.autograd.Function):
    @staticmethod
    def _compute_mask(x: torch.Tensor, k_per_token: int,
                      x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Boolean mask of the min(k*B, numel) top entries of the whole block
        (activations.py:11-36); ties go to the lowest flat index."""
        if k_per_token <= 0 or x.numel() == 0:
            return torch.zeros_like(x, dtype=torch.bool)
        rank = x if x_for_ranking is None else x_for_ranking
        nat.require_device(rank, "BatchTopK")
        B = x.size(0)
        block = _as_block(rank.reshape(B, -1))
        surv = engine.batchtopk_select(block, int(k_per_token), global_mode=False)
        return _mask_from_survivors(surv, x.shape)

    @staticmethod
    def forward(ctx, x: torch.Tensor, k: float, straight_through: bool,
                x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
        mask = BatchTopK._compute_mask(x, int(k), x_for_ranking)
        ctx.save_for_backward(mask)
        ctx.straight_through = straight_through
        return x * mask.to(x.dtype)

    @staticmethod
    def backward(ctx, *grads: torch.Tensor):
        if len(grads) != 1:
            raise ValueError(f"BatchTopK backward expected 1 gradient tensor, got {len(grads)}")
        (mask,) = ctx.saved_tensors
        # both settings of straight_through use the mask gradient (activations.py:82-90)
        return grads[0] * mask.to(grads[0].dtype), None, None, None


class TokenTopK(torch.autograd.Function):
    @staticmethod
    def _compute_mask(x: torch.Tensor, k_float: float,
                      x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Row-wise top-k mask (activations.py:99-128)."""
        if x.numel() == 0:
            return torch.zeros_like(x, dtype=torch.bool)
        n_rows, f_total = x.shape
        kk = resolve_token_k(float(k_float), f_total)
        if kk <= 0:
            return torch.zeros_like(x, dtype=torch.bool)
        rank = x if x_for_ranking is None else x_for_ranking
        nat.require_device(rank, "TokenTopK")
        surv = engine.tokentopk_select(_as_block(rank), kk, global_mode=False)
        return _mask_from_survivors(surv, x.shape)

    @staticmethod
    def forward(ctx, x: torch.Tensor, k: float, straight_through: bool,
                x_for_ranking: Optional[torch.Tensor] = None) -> torch.Tensor:
        mask = TokenTopK._compute_mask(x, k, x_for_ranking)
        ctx.save_for_backward(mask)
        ctx.straight_through = straight_through
        return x * mask.to(x.dtype)

    @staticmethod
    def backward(ctx, *grads: torch.Tensor):
        if len(grads) != 1:
            raise ValueError(f"TokenTopK backward expected 1 gradient tensor, got {len(grads)}")
        (mask,) = ctx.saved_tensors
        return grads[0] * mask.to(grads[0].dtype), None, None, None


class JumpReLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input: torch.Tensor, threshold: torch.Tensor, bandwidth: float) -> torch.Tensor:
        """(input >= threshold).float() * input, fp32 result (activations.py:177-180)."""
        ctx.save_for_backward(input, threshold)
        ctx.bandwidth = bandwidth
        nat.require_device(input, "JumpReLU")
        feat = input.shape[-1] if input.dim() > 0 else 1
        x2 = input.detach().reshape(-1, feat)
        if x2.dtype not in (torch.float32, torch.bfloat16, torch.float16):
            x2 = x2.to(torch.float32)
        theta = threshold.detach().to(device=x2.device, dtype=x2.dtype)
        theta = torch.broadcast_to(theta.reshape(-1) if theta.dim() > 0 else theta, (feat,)).contiguous()
        surv = engine.threshold_select(x2.contiguous().unsqueeze(0), theta.unsqueeze(0), nat.PRED_GE_THETA)
        return engine.densify(surv, out_f32=True)[0].view(input.shape)

    @staticmethod
    def backward(ctx, *grads: torch.Tensor) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], None]:
        """STE for the input, rectangle window of width `bandwidth` for the threshold
        (activations.py:183-220)."""
        g = grads[0]
        x, theta = ctx.saved_tensors
        bw = ctx.bandwidth
        need_x, need_theta, _ = ctx.needs_input_grad
        gx = gtheta = None
        if need_x:
            gx = g * (x >= theta).type_as(g)
        if need_theta:
            window = (torch.abs(x - theta) <= (bw / 2.0)).type_as(x)
            per_elem = g * ((-x / bw) * window)
            extra = per_elem.dim() - theta.dim()
            if extra > 0:
                gtheta = per_elem.sum(dim=tuple(range(extra)))
            elif extra == 0:
                gtheta = per_elem
            else:
                gtheta = per_elem.sum()
            if gtheta.shape != theta.shape:
                gtheta = gtheta.reshape(theta.shape)
        return gx, gtheta, None


def token_k_from_config(k: float, f_total: int) -> int:
    """Integer per-token count for a config value (topk_k may be a fraction)."""
    return resolve_token_k(float(k), f_total)


__all__ = ["BatchTopK", "TokenTopK", "JumpReLU", "resolve_token_k", "token_k_from_config"]
