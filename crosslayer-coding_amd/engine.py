"""Tensor-level entry points over the C ABI: stacked encode, selection into survivor
lists, sparse decode.  torch supplies device memory and the current stream; every
computation is a HIP kernel of libclt_hip.so.

Layouts
    x          [L, T, d]      inputs, one slab per layer
    w_enc      [L, F, d]      encoder weights (nn.Linear layout)
    pre        [L, T, F]      pre-activations
    survivors  SurvivorList   rows r = layer * T + token; (col, val) sorted by col in a row
    w_packed   [n_dec, F, pitch]  decoder weights, feature-major; pitch = decoder_pitch(d, dtype) >= d
    out        [L, T, d]      reconstructions
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch

from . import _native as nat


@dataclass
class SurvivorList:
    """Compact activations of L layers x T tokens (CSR by row = layer*T + token).

    ``col`` / ``val`` may be longer than the list (threshold activations size them for any batch, see
    ``threshold_select``); every kernel walks the rows through ``row_ptr``, so the tail is never read."""

    row_ptr: torch.Tensor  # int32 [L*T + 1]
    col: torch.Tensor      # int32 [capacity >= nnz]   feature index
    val: torch.Tensor      # model dtype [capacity >= nnz]   raw pre-activation
    T: int
    F: int
    L: int
    dtype: torch.dtype
    # int32 [1] on the device when col / val were sized without reading the total back: 1 = the batch has more
    # survivors than a list can hold (2^31 - 1) and the list was emptied - whatever is computed from it must
    # be poisoned (``poison_if``) or refused (``trimmed``); None = sized from the exact total
    status: Optional[torch.Tensor] = None
    # host-side estimate of the survivor total where one is known without a read-back (cost models only)
    nnz_hint: Optional[int] = None

    @property
    def nnz(self) -> int:
        """Survivor total; reads one int back from the device (synchronises)."""
        return int(self.row_ptr[-1].item())

    @property
    def capacity(self) -> int:
        """Entries col / val hold: what buffers indexed by survivor are sized from, without a read-back."""
        return int(self.col.numel())

    def trimmed(self) -> "SurvivorList":
        """The same list with col / val cut to the exact total (one read-back): for consumers that size
        survivor-indexed buffers from ``capacity``.  Raises when the batch had no representable list."""
        if self.status is None:
            return self
        total, bad = int(self.row_ptr[-1].item()), int(self.status.item())
        if bad:
            raise nat.CLTNativeError("the batch has more active features than a survivor list can hold (2^31 - 1)")
        return SurvivorList(self.row_ptr, self.col[:total], self.val[:total], self.T, self.F, self.L, self.dtype,
                            None, total)


def max_list_entries(L: int, T: int, F: int) -> int:
    """Entries no survivor list of this shape exceeds: every element, or what an int32 row pointer addresses."""
    return min(int(L) * int(T) * int(F), 2 ** 31 - 1)


def poison_if(buf: torch.Tensor, flag: torch.Tensor) -> None:
    """NaN over ``buf`` when the device flag is set (decided on the device, nothing is read back)."""
    if buf.numel() == 0:
        return
    assert buf.is_contiguous()
    code = nat.load().clt_poison_if(nat.ptr(buf), buf.numel() * buf.element_size(), nat.ptr(flag),
                                    nat.current_stream(buf.device))
    nat.check(code, "clt_poison_if")


class Workspace:
    """Grow-only device buffers reused across calls on one stream."""

    def __init__(self, device: torch.device):
        self.device = device
        self._bufs: Dict[str, torch.Tensor] = {}

    def get(self, name: str, nbytes: int) -> torch.Tensor:
        buf = self._bufs.get(name)
        if buf is None or buf.numel() < nbytes:
            self._bufs.pop(name, None)
            buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=self.device)
            self._bufs[name] = buf
        return buf

    def typed(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        item = torch.empty((), dtype=dtype).element_size()
        buf = self.get(name, n * item)
        return buf[: n * item].view(dtype).view(*shape)

    def release(self) -> None:
        self._bufs.clear()


# below this many (token, target) rows one wavefront per row already underfills the GPU
SLICED_DECODE_MIN_ROWS = 8192
# ... or, whatever the batch, when the decoders are far larger than the caches: a short batch then spends its time
# fetching decoder rows from HBM, and the schedules that give each XCD its own part of a matrix fetch every row once
# instead of once per XCD that happens to need it (C1 with 64 tokens: 1.64 -> 1.29 ms, C0 with 256: 2.79 -> 1.87 ms)
SLICED_DECODE_MIN_SLAB_BYTES = 128 << 20


def _wants_sliced_decode(rows: int, slab_bytes: int) -> bool:
    return rows >= SLICED_DECODE_MIN_ROWS or slab_bytes >= SLICED_DECODE_MIN_SLAB_BYTES


# token rows of one tile of the matrix-core encoder: shorter batches are padded to it (see ``encode``)
ENCODE_MIN_TOKENS = 256
# widest d_model the gradient kernels that walk survivor lists take (a row is held by one wavefront, up to eight
# 16-byte pieces per lane in bf16); wider models get their gradients from the dense formulation
BACKWARD_MAX_D_MODEL = 4096
# below this many multiply-adds a shape the matrix-core encoder does not take stays on the generic kernel (about
# 0.2 ms there); above it the operands are zero-padded to a shape it takes (see ``encode``)
ENCODE_PAD_MIN_MACS = 5e7


def _stream(t: torch.Tensor) -> int:
    return nat.current_stream(t.device)


def encode(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor],
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """pre[l] = x[l] @ w[l].T + b[l] for stacked layers (parallel.py:286 per layer)."""
    nat.require_device(x, "encode")
    L, T, d = x.shape
    F = w.shape[1]
    assert w.shape == (L, F, d) and x.dtype == w.dtype
    assert x.stride(2) == 1 and x.stride(1) == d and w.stride(2) == 1 and w.stride(1) == d
    if out is None:
        out = torch.empty((L, T, F), dtype=x.dtype, device=x.device)
    assert out.shape == (L, T, F) and out.stride(2) == 1 and out.stride(1) == F
    if b is not None:
        assert b.shape == (L, F) and b.stride(1) == 1 and b.dtype == x.dtype
    lib = nat.load()
    dt = nat.dtype_code(x.dtype)

    def query(x_, w_, b_, out_):
        return bool(lib.clt_encode_fast_path(nat.ptr(x_), nat.ptr(w_), nat.ptr(b_), nat.ptr(out_), x_.shape[1], x_.shape[2],
                                             w_.shape[1], L, x_.stride(0), w_.stride(0),
                                             b_.stride(0) if b_ is not None else 0, out_.stride(0), dt))

    def run(x_, w_, b_, out_):
        code = lib.clt_encode(nat.ptr(x_), nat.ptr(w_), nat.ptr(b_), nat.ptr(out_), x_.shape[1], x_.shape[2], w_.shape[1], L,
                              x_.stride(0), w_.stride(0), b_.stride(0) if b_ is not None else 0, out_.stride(0),
                              dt, _stream(x))
        nat.check(code, "clt_encode")

    if T == 0 or query(x, w, b, out):
        run(x, w, b, out)
        return out
    # The matrix-core kernel works on whole 256 x 256 tiles and whole 128-byte stages along d; anything else falls
    # to the one-thread-per-output kernel, which is 30x slower on a short prompt and hundreds of times on a large
    # odd shape.  Such operands are handed over as zero-padded copies instead (zeros add nothing to the sums;
    # rows and columns past the real ones are dropped coming out): only the tokens of a short batch when nothing
    # else is in the way, the weights too (two passes over them, still far cheaper) when d or F is.
    stage = 128 // x.element_size()
    Tp, dp, Fp = max(T, ENCODE_MIN_TOKENS), -(-d // stage) * stage, max(256, -(-F // 8) * 8)
    if (dp != d or Fp != F) and L * T * F * d < ENCODE_PAD_MIN_MACS:
        run(x, w, b, out)
        return out
    xp, wp, bp = x, w, b
    if Tp != T or dp != d:
        xp = torch.zeros((L, Tp, dp), dtype=x.dtype, device=x.device)
        xp[:, :T, :d] = x
    if dp != d or Fp != F:
        wp = torch.zeros((L, Fp, dp), dtype=x.dtype, device=x.device)
        wp[:, :F, :d] = w
    if b is not None and Fp != F:
        bp = torch.zeros((L, Fp), dtype=x.dtype, device=x.device)
        bp[:, :F] = b
    outp = out if (Tp == T and Fp == F) else torch.empty((L, Tp, Fp), dtype=x.dtype, device=x.device)
    if not query(xp, wp, bp, outp):       # something else is in the way (an unaligned view, say)
        run(x, w, b, out)
        return out
    run(xp, wp, bp, outp)
    if outp is not out:
        out.copy_(outp[:, :T, :F])
    return out


def encode_segmented(x: torch.Tensor, w: torch.Tensor, n_seg: int, d_seg: int, x_seg_stride: int, x_row_stride: int,
                     w_seg_stride: int, w_row_stride: int, T: int, F: int,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[T, F] = sum over segments q of x_q[T, d_seg] @ w_q[F, d_seg].T, where segment q of either operand
    starts q * seg_stride elements after the tensor's first element and its rows are row_stride apart: the
    per-source product behind the JumpReLU threshold gradient (activations.py:183-220) taken from the
    gradient slab and the packed decoder slab in place."""
    nat.require_device(x, "encode_segmented")
    assert x.dtype == w.dtype and x.is_contiguous() and w.is_contiguous()
    assert (n_seg - 1) * x_seg_stride + (T - 1) * x_row_stride + d_seg <= x.numel()
    assert (n_seg - 1) * w_seg_stride + (F - 1) * w_row_stride + d_seg <= w.numel()
    if out is None:
        out = torch.empty((T, F), dtype=x.dtype, device=x.device)
    assert out.shape == (T, F) and out.is_contiguous()
    code = nat.load().clt_encode_segmented(nat.ptr(x), nat.ptr(w), nat.ptr(out), T, d_seg, n_seg, F, x_seg_stride,
                                           x_row_stride, w_seg_stride, w_row_stride, nat.dtype_code(x.dtype), _stream(x))
    nat.check(code, "clt_encode_segmented")
    return out


def colstats(pre: torch.Tensor):
    """(mean, denom) fp32 [L, F] of the global ranking z-score (activations.py:281-283)."""
    nat.require_device(pre, "colstats")
    L, T, F = pre.shape
    mean = torch.empty((L, F), dtype=torch.float32, device=pre.device)
    denom = torch.empty((L, F), dtype=torch.float32, device=pre.device)
    code = nat.load().clt_colstats(nat.ptr(pre), nat.ptr(mean), nat.ptr(denom), T, F, L, pre.stride(0),
                                   nat.dtype_code(pre.dtype), _stream(pre))
    nat.check(code, "clt_colstats")
    return mean, denom


def colstats_full(pre: torch.Tensor):
    """(mean, std, denom) fp32 [L, F]: colstats plus the unbiased std itself (theta.py:305-318)."""
    L, T, F = _check_pre(pre)
    mean = torch.empty((L, F), dtype=torch.float32, device=pre.device)
    std = torch.empty_like(mean)
    denom = torch.empty_like(mean)
    code = nat.load().clt_colstats_full(nat.ptr(pre), nat.ptr(mean), nat.ptr(std), nat.ptr(denom), T, F, L,
                                        pre.stride(0), nat.dtype_code(pre.dtype), _stream(pre))
    nat.check(code, "clt_colstats_full")
    return mean, std, denom


def selected_min_accumulate(surv: SurvivorList, mean: torch.Tensor, denom: torch.Tensor, sum_buf: torch.Tensor,
                            count_buf: torch.Tensor, ws: Optional[Workspace] = None) -> None:
    """sum_buf / count_buf [L, F] (model dtype) += the per-feature minimum z-score of the positive
    survivors of this batch / 1 (theta.py:82-173)."""
    L, F = surv.L, surv.F
    assert sum_buf.shape == (L, F) and count_buf.shape == (L, F)
    assert sum_buf.dtype == surv.dtype and count_buf.dtype == surv.dtype
    assert sum_buf.is_contiguous() and count_buf.is_contiguous()
    dev = surv.row_ptr.device
    wbuf = (ws or Workspace(dev)).get("selected_min", L * F * 4)
    code = nat.load().clt_selected_min_accumulate(
        nat.ptr(surv.row_ptr), nat.ptr(surv.col), nat.ptr(surv.val), nat.ptr(mean), nat.ptr(denom), surv.T, F, L,
        nat.dtype_code(surv.dtype), nat.ptr(sum_buf), nat.ptr(count_buf), nat.ptr(wbuf), wbuf.numel(),
        nat.current_stream(dev))
    nat.check(code, "clt_selected_min_accumulate")


def _check_pre(pre: torch.Tensor):
    nat.require_device(pre, "select")
    L, T, F = pre.shape
    assert pre.stride(2) == 1 and (pre.stride(1) == F or T <= 1)
    return L, T, F


def batchtopk_select(pre: torch.Tensor, k: int, global_mode: bool, ws: Optional[Workspace] = None,
                     stats=None) -> SurvivorList:
    """BatchTopK survivors of pre [L, T, F] (activations.py:11-36 per layer, 261-357 global)."""
    L, T, F = _check_pre(pre)
    dev = pre.device
    k = int(k)
    if global_mode:
        total = min(k * T, T * F * L) if k > 0 else 0
    else:
        total = L * min(k * T, T * F) if k > 0 else 0
    row_ptr = torch.empty(L * T + 1, dtype=torch.int32, device=dev)
    col = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
    val = torch.empty(max(total, 1), dtype=pre.dtype, device=dev)
    mode = nat.TOPK_GLOBAL if global_mode else nat.TOPK_PER_LAYER
    lib = nat.load()
    mean = denom = None
    if global_mode and total > 0:
        mean, denom = stats if stats is not None else colstats(pre)
    nbytes = lib.clt_batchtopk_workspace_bytes(T, F, L, max(k, 0), mode, nat.dtype_code(pre.dtype))
    wbuf = (ws or Workspace(dev)).get("select", nbytes)
    code = lib.clt_batchtopk_select(nat.ptr(pre), T, F, L, pre.stride(0), k, mode, nat.ptr(mean), nat.ptr(denom),
                                    nat.dtype_code(pre.dtype), nat.ptr(row_ptr), nat.ptr(col), nat.ptr(val),
                                    nat.ptr(wbuf), wbuf.numel(), _stream(pre))
    nat.check(code, "clt_batchtopk_select")
    return SurvivorList(row_ptr, col[:total], val[:total], T, F, L, pre.dtype)


def encode_collect_supported(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], k: int) -> bool:
    """True when encode_collect can run these shapes (else: encode, then batchtopk_select)."""
    if not x.is_cuda or k <= 0:
        return False
    L, T, d = x.shape
    F = w.shape[1]
    return bool(nat.load().clt_encode_collect_supported(
        nat.ptr(x), nat.ptr(w), nat.ptr(b), T, d, F, L, x.stride(0), w.stride(0),
        b.stride(0) if b is not None else 0, int(k), nat.dtype_code(x.dtype)))


def encode_collect(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], k: int, pre_scratch: torch.Tensor,
                   ws: Workspace):
    """First half of the fused per-layer BatchTopK path: the encoder projection whose epilogue
    keeps only the candidates above a sampled cut (encoder.py:151-162 + activations.py:11-36).
    Returns the handle that collect_select needs."""
    nat.require_device(x, "encode_collect")
    L, T, d = x.shape
    F = w.shape[1]
    assert w.shape == (L, F, d) and x.dtype == w.dtype and pre_scratch.shape == (L, T, F)
    assert pre_scratch.dtype == x.dtype and pre_scratch.stride(2) == 1 and pre_scratch.stride(1) == F
    lib = nat.load()
    dt = nat.dtype_code(x.dtype)
    nbytes = lib.clt_encode_collect_workspace_bytes(T, d, F, L, int(k), dt)
    wbuf = ws.get("collect", nbytes)
    code = lib.clt_encode_collect(nat.ptr(x), nat.ptr(w), nat.ptr(b), nat.ptr(pre_scratch), T, d, F, L,
                                  x.stride(0), w.stride(0), b.stride(0) if b is not None else 0,
                                  pre_scratch.stride(0), int(k), dt, nat.ptr(wbuf), wbuf.numel(), _stream(x))
    nat.check(code, "clt_encode_collect")
    return (pre_scratch, int(k), wbuf)


def collect_select(handle) -> SurvivorList:
    """Second half: exact per-layer BatchTopK on the collected candidates."""
    pre, k, wbuf = handle
    L, T, F = pre.shape
    dev = pre.device
    total = L * min(k * T, T * F)
    row_ptr = torch.empty(L * T + 1, dtype=torch.int32, device=dev)
    col = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
    val = torch.empty(max(total, 1), dtype=pre.dtype, device=dev)
    code = nat.load().clt_collect_select(nat.ptr(pre), T, F, L, pre.stride(0), k, nat.dtype_code(pre.dtype),
                                         nat.ptr(row_ptr), nat.ptr(col), nat.ptr(val), nat.ptr(wbuf), wbuf.numel(),
                                         _stream(pre))
    nat.check(code, "clt_collect_select")
    return SurvivorList(row_ptr, col[:total], val[:total], T, F, L, pre.dtype)


def tokentopk_select(pre: torch.Tensor, kk: int, global_mode: bool, ws: Optional[Workspace] = None,
                     stats=None) -> SurvivorList:
    """TokenTopK survivors, kk already resolved to a count (activations.py:99-128, 391-491)."""
    L, T, F = _check_pre(pre)
    dev = pre.device
    kk = int(kk)
    total = T * min(kk, L * F) if global_mode else L * T * min(kk, F)
    total = max(total, 0)
    row_ptr = torch.empty(L * T + 1, dtype=torch.int32, device=dev)
    col = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
    val = torch.empty(max(total, 1), dtype=pre.dtype, device=dev)
    mode = nat.TOPK_GLOBAL if global_mode else nat.TOPK_PER_LAYER
    lib = nat.load()
    mean = denom = None
    if global_mode and total > 0:
        mean, denom = stats if stats is not None else colstats(pre)
    nbytes = lib.clt_tokentopk_workspace_bytes(T, F, L, max(kk, 0), mode, nat.dtype_code(pre.dtype))
    wbuf = (ws or Workspace(dev)).get("select", nbytes)
    code = lib.clt_tokentopk_select(nat.ptr(pre), T, F, L, pre.stride(0), kk, mode, nat.ptr(mean), nat.ptr(denom),
                                    nat.dtype_code(pre.dtype), nat.ptr(row_ptr), nat.ptr(col), nat.ptr(val),
                                    nat.ptr(wbuf), wbuf.numel(), _stream(pre))
    nat.check(code, "clt_tokentopk_select")
    return SurvivorList(row_ptr, col[:total], val[:total], T, F, L, pre.dtype)


def _fit(row_ptr: torch.Tensor, capacity: int) -> torch.Tensor:
    """Device-side check that the survivor total fits ``capacity`` (else the list is emptied): the int32
    [1] status the emit call is gated on."""
    status = torch.empty(1, dtype=torch.int32, device=row_ptr.device)
    code = nat.load().clt_survivors_fit(nat.ptr(row_ptr), row_ptr.numel() - 1, int(capacity), nat.ptr(status),
                                        nat.current_stream(row_ptr.device))
    nat.check(code, "clt_survivors_fit")
    return status


def _read_total(row_ptr: torch.Tensor) -> int:
    total = int(row_ptr[-1].item())
    if total == -2:
        raise nat.CLTNativeError("the batch has more active features than a survivor list can hold (2^31 - 1)")
    return total


def threshold_dense(pre: torch.Tensor, theta: Optional[torch.Tensor], pred: int) -> torch.Tensor:
    """``pre`` [L, T, F] gated in place - x where the predicate holds, else 0 (activations.py:177-180,
    registry.py:30-33) - and the number of elements kept, as a one-element int64 tensor on the device."""
    L, T, F = _check_pre(pre)
    nat.require_device(pre, "threshold_dense")
    if theta is not None:
        assert theta.shape == (L, F) and theta.dtype == pre.dtype and theta.is_contiguous()
    total = torch.empty(1, dtype=torch.int64, device=pre.device)
    code = nat.load().clt_threshold_dense(nat.ptr(pre), T, F, L, pre.stride(0), nat.ptr(theta), int(pred),
                                          nat.dtype_code(pre.dtype), nat.ptr(total), _stream(pre))
    nat.check(code, "clt_threshold_dense")
    return total


def threshold_select(pre: torch.Tensor, theta: Optional[torch.Tensor], pred: int,
                     ws: Optional[Workspace] = None, read_back: bool = True) -> SurvivorList:
    """JumpReLU (x >= theta), ReLU (x > 0) or non-zero compaction of pre [L, T, F].

    Two kernels.  ``read_back``: one 4-byte read-back in between sizes col / val exactly.  Without it nothing
    is read back: col / val get ``max_list_entries`` entries, which every batch fits that a list can
    represent at all, and ``status`` says on the device whether this one could be (else it is empty)."""
    L, T, F = _check_pre(pre)
    dev = pre.device
    lib = nat.load()
    code_dt = nat.dtype_code(pre.dtype)
    if theta is not None:
        assert theta.shape == (L, F) and theta.dtype == pre.dtype and theta.is_contiguous()
    row_ptr = torch.empty(L * T + 1, dtype=torch.int32, device=dev)
    wbuf = (ws or Workspace(dev)).get("threshold", max(L * T * 4, 256))
    code = lib.clt_threshold_count(nat.ptr(pre), T, F, L, pre.stride(0), nat.ptr(theta), pred, code_dt,
                                   nat.ptr(row_ptr), nat.ptr(wbuf), wbuf.numel(), _stream(pre))
    nat.check(code, "clt_threshold_count")
    status = None
    if read_back:
        total = _read_total(row_ptr)
    else:
        total = max_list_entries(L, T, F)
        status = _fit(row_ptr, total)
    col = torch.empty(max(total, 1), dtype=torch.int32, device=dev)
    val = torch.empty(max(total, 1), dtype=pre.dtype, device=dev)
    code = lib.clt_threshold_emit(nat.ptr(pre), T, F, L, pre.stride(0), nat.ptr(theta), pred, code_dt,
                                  nat.ptr(row_ptr), nat.ptr(col), nat.ptr(val), nat.ptr(status), _stream(pre))
    nat.check(code, "clt_threshold_emit")
    return SurvivorList(row_ptr, col[:total], val[:total], T, F, L, pre.dtype, status, total if read_back else None)


def encode_threshold(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], theta: torch.Tensor,
                     ws: Workspace, density_ppm: int = 20000,
                     pre_scratch: Optional[torch.Tensor] = None) -> Optional[SurvivorList]:
    """Encoder projection + JumpReLU (x >= theta) without dense pre-activations
    (parallel.py:286 + theta.py:70-79).  Returns None when the shapes do not qualify.

    ``pre_scratch`` None: the total is read back once and col / val are sized exactly; None is returned when
    the survivors exceeded the pool ``density_ppm`` provides for (the caller then runs ``encode`` and
    ``threshold_select``).  With ``pre_scratch`` [L, T, F] nothing is read back: col / val get
    ``max_list_entries`` entries, and a pool that turns out too small makes the device itself take the
    dense route through ``pre_scratch`` (clt_encode_threshold_recover), so the list is exact whatever the
    density; ``status`` is set only for a batch no list can represent."""
    nat.require_device(x, "encode_threshold")
    L, T, d = x.shape
    F = w.shape[1]
    assert w.shape == (L, F, d) and x.dtype == w.dtype
    assert theta.shape == (L, F) and theta.dtype == x.dtype and theta.stride(1) == 1
    lib = nat.load()
    dt = nat.dtype_code(x.dtype)
    strides = (x.stride(0), w.stride(0), b.stride(0) if b is not None else 0, theta.stride(0))
    if not lib.clt_encode_threshold_supported(nat.ptr(x), nat.ptr(w), nat.ptr(b), nat.ptr(theta), T, d, F, L,
                                              *strides, int(density_ppm), dt):
        return None
    if pre_scratch is not None and theta.stride(0) != F:
        return None
    nbytes = lib.clt_encode_threshold_workspace_bytes(T, d, F, L, int(density_ppm), dt)
    wbuf = ws.get("collect_threshold", nbytes)
    row_ptr = torch.empty(L * T + 1, dtype=torch.int32, device=x.device)
    code = lib.clt_encode_threshold_count(nat.ptr(x), nat.ptr(w), nat.ptr(b), nat.ptr(theta), T, d, F, L, *strides,
                                          int(density_ppm), dt, nat.ptr(row_ptr), nat.ptr(wbuf), wbuf.numel(), _stream(x))
    nat.check(code, "clt_encode_threshold_count")
    flags = None
    if pre_scratch is None:
        total = _read_total(row_ptr)
        if total < 0:
            return None
    else:
        assert pre_scratch.shape == (L, T, F) and pre_scratch.dtype == x.dtype
        assert pre_scratch.stride(2) == 1 and pre_scratch.stride(1) == F
        total = max_list_entries(L, T, F)
        flags = torch.empty(3, dtype=torch.int32, device=x.device)
        code = lib.clt_encode_threshold_recover(nat.ptr(x), nat.ptr(w), nat.ptr(b), nat.ptr(theta), nat.ptr(pre_scratch),
                                                T, d, F, L, *strides, pre_scratch.stride(0), int(density_ppm), dt,
                                                nat.ptr(row_ptr), total, nat.ptr(flags), nat.ptr(wbuf), wbuf.numel(),
                                                _stream(x))
        nat.check(code, "clt_encode_threshold_recover")
    col = torch.empty(max(total, 1), dtype=torch.int32, device=x.device)
    val = torch.empty(max(total, 1), dtype=x.dtype, device=x.device)
    code = lib.clt_encode_threshold_emit(T, F, L, int(density_ppm), dt, nat.ptr(row_ptr), nat.ptr(col), nat.ptr(val),
                                         nat.ptr(flags), nat.ptr(wbuf), wbuf.numel(), _stream(x))
    nat.check(code, "clt_encode_threshold_emit")
    if flags is None:
        return SurvivorList(row_ptr, col[:total], val[:total], T, F, L, x.dtype, None, total)
    code = lib.clt_threshold_emit(nat.ptr(pre_scratch), T, F, L, pre_scratch.stride(0), nat.ptr(theta), nat.PRED_GE_THETA,
                                  dt, nat.ptr(row_ptr), nat.ptr(col), nat.ptr(val), flags[1:].data_ptr(), _stream(x))
    nat.check(code, "clt_threshold_emit")
    return SurvivorList(row_ptr, col[:total], val[:total], T, F, L, x.dtype, flags[2:3])


# ---- evaluation reductions ------------------------------------------------------------------------------
def survivor_metrics(surv: SurvivorList, fired_eps: float = 1e-6):
    """(entries != 0 per layer, int64 [L]; tokens with value > fired_eps per (layer, feature),
    int32 [L, F]) straight from the survivor list (evaluator.py:194-244, 350-405)."""
    nat.require_device(surv.row_ptr, "survivor_metrics")
    dev = surv.row_ptr.device
    nonzero = torch.empty(surv.L, dtype=torch.int64, device=dev)
    fired = torch.empty((surv.L, surv.F), dtype=torch.int32, device=dev)
    empty = surv.capacity == 0
    code = nat.load().clt_survivor_metrics(nat.ptr(surv.row_ptr), None if empty else nat.ptr(surv.col),
                                           None if empty else nat.ptr(surv.val), surv.T, surv.F, surv.L,
                                           nat.dtype_code(surv.dtype), fired_eps, nat.ptr(nonzero), nat.ptr(fired),
                                           _stream(surv.row_ptr))
    nat.check(code, "clt_survivor_metrics")
    return nonzero, fired


def dead_feature_update(fired: torch.Tensor, passes_since_fired: torch.Tensor) -> None:
    """In place: counters of features that fired go to 0, the others go up by one (trainer.py:711-712)."""
    nat.require_device(fired, "dead_feature_update")
    assert fired.dtype == torch.int32 and passes_since_fired.dtype == torch.int64
    assert fired.is_contiguous() and passes_since_fired.is_contiguous() and fired.numel() == passes_since_fired.numel()
    code = nat.load().clt_dead_feature_update(nat.ptr(fired), nat.ptr(passes_since_fired), fired.numel(), _stream(fired))
    nat.check(code, "clt_dead_feature_update")


DENORM_MODES = {"none": 0, "mean_std": 1, "sqrt_d_model": 2}


def reconstruction_stats(rec: torch.Tensor, target: torch.Tensor, mode: str = "none",
                         mean: Optional[torch.Tensor] = None, std: Optional[torch.Tensor] = None,
                         scale: float = 1.0, ws: Optional[Workspace] = None) -> torch.Tensor:
    """float64 [L, 3]: MSE, mean column variance of the target, mean column variance of the error,
    after de-normalising rec and target [L, T, d] in their dtype (evaluator.py:246-345)."""
    nat.require_device(rec, "reconstruction_stats")
    L, T, d = rec.shape
    assert target.shape == rec.shape and target.dtype == rec.dtype and rec.is_contiguous() and target.is_contiguous()
    if mode == "mean_std":
        assert mean is not None and std is not None and mean.shape == (L, d) and std.shape == (L, d)
        mean, std = mean.to(rec.dtype).contiguous(), std.to(rec.dtype).contiguous()
    stats = torch.empty((L, 3), dtype=torch.float64, device=rec.device)
    lib = nat.load()
    wbuf = (ws or Workspace(rec.device)).get("recon_stats", lib.clt_reconstruction_stats_workspace_bytes(d, L))
    code = lib.clt_reconstruction_stats(nat.ptr(rec), nat.ptr(target), T, d, L, nat.dtype_code(rec.dtype),
                                        DENORM_MODES[mode], nat.ptr(mean) if mode == "mean_std" else None,
                                        nat.ptr(std) if mode == "mean_std" else None, float(scale), nat.ptr(stats),
                                        nat.ptr(wbuf), wbuf.numel(), _stream(rec))
    nat.check(code, "clt_reconstruction_stats")
    return stats


# ---- backward pass (MSE reconstruction loss) ---------------------------------------------------------
def mse_loss_grad(rec: torch.Tensor, target: torch.Tensor, ws: Optional[Workspace] = None, mode: str = "none",
                  mean: Optional[torch.Tensor] = None, std: Optional[torch.Tensor] = None, scale: float = 1.0):
    """(loss per layer [L] fp32, g [L, T, d] fp32 = d loss / d rec, the same in the model dtype,
    bias_grad [L, d] fp32) for loss = sum over layers of mean((rec' - target')^2), ' being the reference's
    de-normalisation (losses.py:45-92): ``mode`` "mean_std" with the target statistics ``mean`` / ``std``
    [L, d], "sqrt_d_model" with ``scale`` = sqrt(d_model), or "none"."""
    nat.require_device(rec, "mse_loss_grad")
    L, T, d = rec.shape
    assert target.shape == rec.shape and target.dtype == rec.dtype and rec.is_contiguous() and target.is_contiguous()
    if mode == "mean_std":
        assert mean is not None and std is not None and mean.shape == (L, d) and std.shape == (L, d)
        mean, std = mean.to(rec.dtype).contiguous(), std.to(rec.dtype).contiguous()
    dev = rec.device
    loss = torch.empty(L, dtype=torch.float32, device=dev)
    g = torch.empty((L, T, d), dtype=torch.float32, device=dev)
    bias_grad = torch.empty((L, d), dtype=torch.float32, device=dev)
    g_model = g if rec.dtype == torch.float32 else torch.empty((L, T, d), dtype=rec.dtype, device=dev)
    lib = nat.load()
    wbuf = (ws or Workspace(dev)).get("mse", lib.clt_mse_workspace_bytes(T, d, L))
    code = lib.clt_mse_loss_grad(nat.ptr(rec), nat.ptr(target), T, d, L, nat.dtype_code(rec.dtype), DENORM_MODES[mode],
                                 nat.ptr(mean) if mode == "mean_std" else None, nat.ptr(std) if mode == "mean_std" else None,
                                 float(scale), nat.ptr(loss), nat.ptr(g), nat.ptr(g_model) if g_model is not g else None,
                                 nat.ptr(bias_grad), nat.ptr(wbuf), wbuf.numel(), _stream(rec))
    nat.check(code, "clt_mse_loss_grad")
    return loss, g, g_model, bias_grad


def decode_backward_values(surv: SurvivorList, w_packed: torch.Tensor, g: torch.Tensor, tying: str,
                           src_mask: Optional[int] = None, ws: Optional[Workspace] = None,
                           feat_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """d loss / d (kept activation) for every survivor, fp32 [capacity] (the straight-through gate hands
    it to the pre-activation unchanged, activations.py:66-96).  ``feat_scale`` [L, F]: the per-target
    feature scale of tied decoders, a factor on each target's share (decoder.py:228-285).  The per-target
    dot products stay in the "decode_backward" buffer of ``ws`` for ``feature_affine_grad``."""
    L, T, F = surv.L, surv.T, surv.F
    d = g.shape[2]
    assert g.shape == (L, T, d) and g.dtype == torch.float32 and g.is_contiguous()
    assert w_packed.dtype == surv.dtype and w_packed.is_contiguous()
    assert tuple(w_packed.shape[1:]) == (F, decoder_pitch(d, surv.dtype))
    assert feat_scale is None or (feat_scale.shape == (L, F) and feat_scale.dtype == surv.dtype and feat_scale.is_contiguous())
    if src_mask is None:
        src_mask = (1 << L) - 1
    cap = surv.capacity          # survivor-indexed buffers are sized from the arrays, not from a read-back
    dval = torch.empty(max(cap, 1), dtype=torch.float32, device=g.device)
    lib = nat.load()
    wbuf = (ws or Workspace(g.device)).get("decode_backward", lib.clt_decode_backward_workspace_bytes(T, L, cap))
    code = lib.clt_decode_backward_values(nat.ptr(surv.row_ptr), nat.ptr(surv.col), nat.ptr(surv.val), nat.ptr(w_packed),
                                          nat.ptr(feat_scale), nat.ptr(g), T, d, F, L, nat.TYING[tying],
                                          src_mask & ((1 << 64) - 1), cap, nat.dtype_code(surv.dtype), nat.ptr(dval),
                                          nat.ptr(wbuf), wbuf.numel(), _stream(g))
    nat.check(code, "clt_decode_backward_values")
    return dval[:cap]


def feature_affine_grad(lists, surv: SurvivorList, ws: Workspace, feat_offset: Optional[torch.Tensor],
                        feat_scale: Optional[torch.Tensor], src_mask: Optional[int] = None):
    """(d offset [L, F] or None, d scale [L, F] or None), fp32: gradients of the per-target feature offset /
    scale of tied decoders (decoder.py:228-285).  Must follow ``decode_backward_values`` on the same ``ws``."""
    L, T, F = surv.L, surv.T, surv.F
    ptr, _, src = lists
    dev = surv.row_ptr.device
    if src_mask is None:
        src_mask = (1 << L) - 1
    doff = torch.empty((L, F), dtype=torch.float32, device=dev) if feat_offset is not None else None
    dsc = torch.empty((L, F), dtype=torch.float32, device=dev) if feat_scale is not None else None
    lib = nat.load()
    cap = surv.capacity
    wbuf = ws.get("decode_backward", lib.clt_decode_backward_workspace_bytes(T, L, cap))
    code = lib.clt_feature_affine_grad(nat.ptr(ptr), nat.ptr(src), nat.ptr(surv.val), nat.ptr(feat_offset), nat.ptr(feat_scale),
                                       T, F, L, src_mask & ((1 << 64) - 1), cap, nat.dtype_code(surv.dtype), nat.ptr(doff),
                                       nat.ptr(dsc), nat.ptr(wbuf), wbuf.numel(), nat.current_stream(dev))
    nat.check(code, "clt_feature_affine_grad")
    return doff, dsc


def skip_weight_grad(g_t: torch.Tensor, x_s: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out [d, d] fp32 (+)= g_t.T @ x_s: gradient of one skip matrix (rec[t] += x[s] @ W_skip.T,
    decoder.py:297-338); g_t [T, d] fp32, x_s [T, d] in the model dtype."""
    nat.require_device(g_t, "skip_weight_grad")
    T, d = g_t.shape
    assert x_s.shape == (T, d) and g_t.dtype == torch.float32 and g_t.is_contiguous() and x_s.is_contiguous()
    assert out.shape == (d, d) and out.dtype == torch.float32 and out.is_contiguous()
    code = nat.load().clt_skip_weight_grad(nat.ptr(g_t), nat.ptr(x_s), nat.ptr(out), T, d, 1 if accumulate else 0,
                                           nat.dtype_code(x_s.dtype), _stream(g_t))
    nat.check(code, "clt_skip_weight_grad")


def feature_lists(surv: SurvivorList, ws: Optional[Workspace] = None):
    """The survivor list regrouped by (layer, feature): (ptr [L*F+1], token [nnz], source index [nnz])."""
    L, T, F = surv.L, surv.T, surv.F
    dev = surv.row_ptr.device
    ptr = torch.empty(L * F + 1, dtype=torch.int32, device=dev)
    tok = torch.empty(max(surv.capacity, 1), dtype=torch.int32, device=dev)
    src = torch.empty(max(surv.capacity, 1), dtype=torch.int32, device=dev)
    lib = nat.load()
    wbuf = (ws or Workspace(dev)).get("feature_lists", lib.clt_feature_lists_workspace_bytes(F, L))
    code = lib.clt_feature_lists(nat.ptr(surv.row_ptr), nat.ptr(surv.col), T, F, L, nat.ptr(ptr), nat.ptr(tok),
                                 nat.ptr(src), nat.ptr(wbuf), wbuf.numel(), nat.current_stream(dev))
    nat.check(code, "clt_feature_lists")
    return ptr, tok, src


def decoder_weight_grad(lists, surv: SurvivorList, g: torch.Tensor, tying: str,
                        feat_offset: Optional[torch.Tensor] = None, feat_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 [n_dec, F, d] gradient of the packed (feature-major) decoder weights (one matrix per
    (source, target) pair, per source or per target, as ``tying`` says); ``g`` is d loss / d rec in
    the model dtype; ``feat_offset`` / ``feat_scale`` [L, F]: the per-target affine terms the forward applied."""
    assert g.dtype == surv.dtype and g.is_contiguous()
    ptr, tok, src = lists
    L, T, F = surv.L, surv.T, surv.F
    d = g.shape[2]
    n_dec = L * (L + 1) // 2 if tying == "none" else L
    out = torch.empty((n_dec, F, d), dtype=torch.float32, device=g.device)
    code = nat.load().clt_decoder_weight_grad(nat.ptr(ptr), nat.ptr(tok), nat.ptr(src), nat.ptr(surv.val), nat.ptr(g),
                                              nat.ptr(feat_offset), nat.ptr(feat_scale), nat.ptr(out), T, d, F, L,
                                              nat.TYING[tying], nat.dtype_code(surv.dtype), _stream(g))
    nat.check(code, "clt_decoder_weight_grad")
    return out


def decoder_weight_grad_adam(lists, surv: SurvivorList, g: torch.Tensor, w_packed: torch.Tensor, m: torch.Tensor,
                             v: torch.Tensor, lr: float, betas, eps: float, step: int) -> None:
    """``decoder_weight_grad`` and the Adam step of the untied decoder weights in one pass: the moments
    [n_dec, F, d] and the packed working copy [n_dec, F, pitch] are updated in place, the gradient is never
    written (trainer.py:663-778 for the decoder weights).  The checkpoint-layout parameters follow with
    ``unpack_decoders``."""
    assert g.dtype == surv.dtype and g.is_contiguous() and w_packed.dtype == surv.dtype and w_packed.is_contiguous()
    ptr, tok, src = lists
    L, T, F = surv.L, surv.T, surv.F
    d = g.shape[2]
    n_dec = L * (L + 1) // 2
    assert tuple(w_packed.shape) == (n_dec, F, decoder_pitch(d, surv.dtype))
    assert m.shape == (n_dec, F, d) and v.shape == m.shape and m.dtype == torch.float32 and v.dtype == torch.float32
    assert m.is_contiguous() and v.is_contiguous()
    code = nat.load().clt_decoder_weight_grad_adam(nat.ptr(ptr), nat.ptr(tok), nat.ptr(src), nat.ptr(surv.val), nat.ptr(g),
                                                   nat.ptr(w_packed), nat.ptr(m), nat.ptr(v), T, d, F, L, lr, betas[0],
                                                   betas[1], eps, step, nat.dtype_code(surv.dtype), _stream(g))
    nat.check(code, "clt_decoder_weight_grad_adam")


def unpack_decoders(w_packed: torch.Tensor, w_refs_dev: torch.Tensor, w_refs_host, d: int, F: int) -> None:
    """Checkpoint-layout parameters [d, F] (their addresses in the device int64 tensor ``w_refs_dev`` and in the
    host ctypes array ``w_refs_host``) from the packed working copy [n_dec, F, pitch]."""
    import ctypes
    n_dec = w_packed.shape[0]
    assert w_refs_dev.dtype == torch.int64 and w_refs_dev.numel() == n_dec and w_packed.is_contiguous()
    code = nat.load().clt_unpack_decoders(nat.ptr(w_packed), nat.ptr(w_refs_dev), ctypes.addressof(w_refs_host), n_dec, d, F,
                                          nat.dtype_code(w_packed.dtype), _stream(w_packed))
    nat.check(code, "clt_unpack_decoders")


def decoder_fingerprint(w_refs_dev: torch.Tensor, d: int, F: int, dtype: torch.dtype, state: torch.Tensor,
                        changed: torch.Tensor, store_only: bool) -> None:
    """Hash a sample of every decoder parameter ([d, F] each, addresses in the device int64 tensor ``w_refs_dev``):
    ``changed[i]`` = 1 where it differs from the hash kept in ``state`` (int64 [16 n_dec], zeros before the first
    call), which is brought up to date; ``store_only`` records without comparing."""
    n_dec = w_refs_dev.numel()
    assert w_refs_dev.dtype == torch.int64 and state.dtype == torch.int64 and state.numel() == 16 * n_dec
    assert changed.dtype == torch.int32 and changed.numel() == n_dec and state.is_contiguous()
    code = nat.load().clt_decoder_fingerprint(nat.ptr(w_refs_dev), n_dec, d, F, nat.dtype_code(dtype), nat.ptr(state),
                                              nat.ptr(changed), 1 if store_only else 0, _stream(state))
    nat.check(code, "clt_decoder_fingerprint")


def pack_decoders_if(w_refs_dev: torch.Tensor, w_packed: torch.Tensor, d: int, F: int, changed: torch.Tensor) -> None:
    """Repack, on the device's own decision, the matrices of the slab [n_dec, F, pitch] whose ``changed`` flag is set."""
    n_dec = w_packed.shape[0]
    assert w_refs_dev.numel() == n_dec and changed.numel() == n_dec and w_packed.is_contiguous()
    code = nat.load().clt_pack_decoders_if(nat.ptr(w_refs_dev), nat.ptr(w_packed), n_dec, d, F,
                                           nat.dtype_code(w_packed.dtype), nat.ptr(changed), _stream(w_packed))
    nat.check(code, "clt_pack_decoders_if")


def bias_sum(b_refs_dev: torch.Tensor, d: int, L: int, tying: str, src_mask: int, dtype: torch.dtype) -> torch.Tensor:
    """fp32 [L, d]: per target the sum of the biases of the decoders that run for it (addresses of the n_dec bias
    vectors in the device int64 tensor ``b_refs_dev``), sources of ``src_mask`` in ascending order."""
    out = torch.empty((L, d), dtype=torch.float32, device=b_refs_dev.device)
    code = nat.load().clt_bias_sum(nat.ptr(b_refs_dev), b_refs_dev.numel(), d, L, nat.TYING[tying], int(src_mask),
                                   nat.dtype_code(dtype), nat.ptr(out), _stream(out))
    nat.check(code, "clt_bias_sum")
    return out


def decoder_tile_width(T: int, d: int, F: int, dtype: torch.dtype) -> int:
    """Columns per tile of the tiled decoder layout [n_dec, d // CS, F, CS] when the column-tile weight-gradient
    kernel takes this shape, else 0."""
    return int(nat.load().clt_decoder_tile_width(int(T), int(d), int(F), nat.dtype_code(dtype)))


def tile_decoders(w_packed: torch.Tensor, d: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Tiled copy [n_dec, d // CS, F, CS] of the feature-major slab [n_dec, F, pitch]."""
    n_dec, F, _ = w_packed.shape
    cs = 32 // w_packed.element_size()
    assert d % cs == 0 and w_packed.is_contiguous()
    if out is None:
        out = torch.empty((n_dec, d // cs, F, cs), dtype=w_packed.dtype, device=w_packed.device)
    assert out.is_contiguous() and tuple(out.shape) == (n_dec, d // cs, F, cs) and out.dtype == w_packed.dtype
    code = nat.load().clt_tile_decoders(nat.ptr(w_packed), nat.ptr(out), n_dec, d, F, nat.dtype_code(w_packed.dtype),
                                        _stream(w_packed))
    nat.check(code, "clt_tile_decoders")
    return out


def untile_decoders(w_tiles: torch.Tensor, w_packed: torch.Tensor, w_refs_dev: Optional[torch.Tensor] = None,
                    w_refs_host=None) -> None:
    """The feature-major slab [n_dec, F, pitch] and (when their addresses are given, as for ``unpack_decoders``)
    the checkpoint-layout parameters [d, F], rewritten from the tiled weights."""
    import ctypes
    n_dec, ns, F, cs = w_tiles.shape
    d = ns * cs
    assert w_tiles.is_contiguous() and w_packed.is_contiguous() and w_packed.dtype == w_tiles.dtype
    assert tuple(w_packed.shape) == (n_dec, F, decoder_pitch(d, w_tiles.dtype))
    assert (w_refs_dev is None) == (w_refs_host is None)
    if w_refs_dev is not None:
        assert w_refs_dev.dtype == torch.int64 and w_refs_dev.numel() == n_dec
    code = nat.load().clt_untile_decoders(nat.ptr(w_tiles), nat.ptr(w_packed), nat.ptr(w_refs_dev),
                                          ctypes.addressof(w_refs_host) if w_refs_host is not None else None, n_dec, d, F,
                                          nat.dtype_code(w_tiles.dtype), _stream(w_tiles))
    nat.check(code, "clt_untile_decoders")


def decoder_weight_grad_adam_tiled(lists, surv: SurvivorList, g: torch.Tensor, w_tiles: torch.Tensor, m_tiles: torch.Tensor,
                                   v_tiles: torch.Tensor, lr: float, betas, eps: float, step: int,
                                   ws: Optional[Workspace] = None) -> None:
    """``decoder_weight_grad_adam`` over column tiles: weights and moments [n_dec, d // CS, F, CS] are updated in
    place (equal to the row route up to the fp32 association of some gradient sums, repeatable bit for bit);
    ``untile_decoders`` brings the slab and the checkpoint-layout parameters up to date."""
    assert g.dtype == surv.dtype and g.is_contiguous() and w_tiles.dtype == surv.dtype and w_tiles.is_contiguous()
    ptr, tok, src = lists
    L, T, F = surv.L, surv.T, surv.F
    d = g.shape[2]
    n_dec = L * (L + 1) // 2
    cs = decoder_tile_width(T, d, F, surv.dtype)
    assert cs > 0, "shape not taken by the column-tile kernel"
    assert tuple(w_tiles.shape) == (n_dec, d // cs, F, cs)
    assert m_tiles.shape == w_tiles.shape and v_tiles.shape == w_tiles.shape and m_tiles.dtype == torch.float32
    assert v_tiles.dtype == torch.float32 and m_tiles.is_contiguous() and v_tiles.is_contiguous()
    lib = nat.load()
    cap = int(tok.numel())
    wbuf = (ws or Workspace(g.device)).get("decoder_tiles", lib.clt_decoder_tiles_workspace_bytes(cap, nat.dtype_code(surv.dtype)))
    code = lib.clt_decoder_weight_grad_adam_tiled(nat.ptr(ptr), nat.ptr(tok), nat.ptr(src), nat.ptr(surv.val), nat.ptr(g),
                                                  nat.ptr(w_tiles), nat.ptr(m_tiles), nat.ptr(v_tiles), T, d, F, L, cap, lr,
                                                  betas[0], betas[1], eps, step, nat.dtype_code(surv.dtype), nat.ptr(wbuf),
                                                  wbuf.numel(), _stream(g))
    nat.check(code, "clt_decoder_weight_grad_adam_tiled")


def encoder_weight_grad(lists, dval: torch.Tensor, x: torch.Tensor, F: int):
    """(fp32 [L, F, d], fp32 [L, F]): gradients of the stacked encoder weights and biases."""
    ptr, tok, src = lists
    L, T, d = x.shape
    assert x.is_contiguous() and dval.dtype == torch.float32
    dw = torch.empty((L, F, d), dtype=torch.float32, device=x.device)
    db = torch.empty((L, F), dtype=torch.float32, device=x.device)
    code = nat.load().clt_encoder_weight_grad(nat.ptr(ptr), nat.ptr(tok), nat.ptr(src), nat.ptr(dval), nat.ptr(x),
                                              nat.ptr(dw), nat.ptr(db), T, d, F, L, nat.dtype_code(x.dtype), _stream(x))
    nat.check(code, "clt_encoder_weight_grad")
    return dw, db


def scatter_survivor_values(surv: SurvivorList, src: torch.Tensor, layer: int, dense: torch.Tensor) -> None:
    """dense[tok, col] = src[j] for the survivors j of ``layer`` (decoder.py:228-285 with activations.py:183-220: the
    kept activations' share of d loss / d activation behind a per-target feature scale)."""
    assert dense.shape == (surv.T, surv.F) and dense.dtype == surv.dtype and dense.is_contiguous()
    assert src.dtype == torch.float32 and src.numel() >= surv.col.numel()
    code = nat.load().clt_scatter_survivor_values(nat.ptr(surv.row_ptr), nat.ptr(surv.col), nat.ptr(src), int(layer), surv.T,
                                                  surv.F, surv.L, nat.dtype_code(surv.dtype), nat.ptr(dense), _stream(dense))
    nat.check(code, "clt_scatter_survivor_values")


def jumprelu_theta_grad(pre: torch.Tensor, grad_out: torch.Tensor, theta: torch.Tensor, bandwidth: float,
                        out: torch.Tensor, ws: Optional[Workspace] = None) -> None:
    """out [F] fp32 = gradient of one layer's JumpReLU thresholds from dense pre-activations and dense
    d loss / d activation, both [T, F] in the model dtype (activations.py:196-199)."""
    nat.require_device(pre, "jumprelu_theta_grad")
    T, F = pre.shape
    assert grad_out.shape == pre.shape and grad_out.dtype == pre.dtype and theta.dtype == pre.dtype
    assert pre.is_contiguous() and grad_out.is_contiguous() and theta.is_contiguous() and theta.numel() == F
    assert out.dtype == torch.float32 and out.is_contiguous() and out.numel() == F
    lib = nat.load()
    wbuf = (ws or Workspace(pre.device)).get("theta_grad", lib.clt_jumprelu_theta_grad_workspace_bytes(F))
    code = lib.clt_jumprelu_theta_grad(nat.ptr(pre), nat.ptr(grad_out), nat.ptr(theta), T, F, float(bandwidth),
                                       nat.dtype_code(pre.dtype), nat.ptr(out), nat.ptr(wbuf), wbuf.numel(), _stream(pre))
    nat.check(code, "clt_jumprelu_theta_grad")


def decoder_pitch(d: int, dtype: torch.dtype) -> int:
    """Row pitch (elements) of the feature-major decoder slab: d, plus one 128-byte line when a row is an
    even number of lines (so that a column part of all rows spreads over every L2 channel)."""
    return int(nat.load().clt_decoder_pitch(int(d), nat.dtype_code(dtype)))


def alloc_packed(n_dec: int, F: int, d: int, dtype: torch.dtype, device) -> torch.Tensor:
    """Zeroed slab [n_dec, F, pitch] for feature-major decoders; ``slab[i, :, :d]`` is matrix i."""
    return torch.zeros((n_dec, F, decoder_pitch(d, dtype)), dtype=dtype, device=device)


def pack_decoder(w_ref: torch.Tensor, out: torch.Tensor) -> None:
    """[d, F] checkpoint layout -> feature-major rows of one matrix of the slab, out [F, pitch]."""
    nat.require_device(w_ref, "pack_decoder")
    d, F = w_ref.shape
    pitch = decoder_pitch(d, w_ref.dtype)
    assert w_ref.is_contiguous() and out.shape == (F, pitch) and out.is_contiguous() and out.dtype == w_ref.dtype
    code = nat.load().clt_pack_decoder(nat.ptr(w_ref), nat.ptr(out), d, F, 1, d * F, F * pitch,
                                       nat.dtype_code(w_ref.dtype), _stream(w_ref))
    nat.check(code, "clt_pack_decoder")


def decode_sparse(surv: SurvivorList, w_packed: torch.Tensor, tying: str, d: int,
                  bias_sum: Optional[torch.Tensor] = None, feat_offset: Optional[torch.Tensor] = None,
                  feat_scale: Optional[torch.Tensor] = None, skip_add: Optional[torch.Tensor] = None,
                  t_begin: int = 0, t_end: Optional[int] = None, src_mask: Optional[int] = None,
                  out: Optional[torch.Tensor] = None, out_f32: bool = False,
                  ws: Optional[Workspace] = None) -> torch.Tensor:
    """Reconstructions [L, T, d] for targets [t_begin, t_end) (decoder.py:176-340).

    With a workspace and a batch large enough to fill the GPU the XCD-sliced kernel is used."""
    nat.require_device(w_packed, "decode_sparse")
    L, T, F = surv.L, surv.T, surv.F
    t_end = L if t_end is None else t_end
    if src_mask is None:
        src_mask = (1 << L) - 1
    dev = w_packed.device
    odt = torch.float32 if out_f32 else surv.dtype
    if out is None:
        out = torch.empty((L, T, d), dtype=odt, device=dev)
    assert out.shape == (L, T, d) and out.is_contiguous() and out.dtype == odt
    assert w_packed.is_contiguous() and w_packed.dtype == surv.dtype
    assert tuple(w_packed.shape[1:]) == (F, decoder_pitch(d, surv.dtype))
    for a in (bias_sum, skip_add):
        assert a is None or (a.dtype == torch.float32 and a.is_contiguous())
    for a in (feat_offset, feat_scale):
        assert a is None or (a.dtype == surv.dtype and a.is_contiguous() and a.shape == (L, F))
    lib = nat.load()
    # the largest offset the kernels form, slot * F * d + f * d + column, is a 64-bit quantity (1.0e10
    # elements for 300 decoders of 32768 x 1024); it must lie inside the slab that was handed in
    need = lib.clt_decoder_slab_elems(d, F, L, nat.TYING[tying], nat.dtype_code(surv.dtype))
    if need < 0 or w_packed.numel() < need:
        raise nat.CLTNativeError(f"decode_sparse: packed decoders hold {w_packed.numel()} elements, the kernels index {need}")
    wbuf, wbytes = None, 0
    if ws is not None and _wants_sliced_decode(T * (t_end - t_begin), w_packed.numel() * w_packed.element_size()):
        wbytes = lib.clt_decode_workspace_bytes(T, d, F, L)
        wbuf = ws.get("decode", wbytes)
    code = lib.clt_decode_sparse(
        nat.ptr(surv.row_ptr), nat.ptr(surv.col), nat.ptr(surv.val), nat.ptr(w_packed), nat.ptr(bias_sum),
        nat.ptr(feat_offset), nat.ptr(feat_scale), nat.ptr(skip_add), nat.ptr(out), T, d, F, L,
        nat.TYING[tying], t_begin, t_end, src_mask & ((1 << 64) - 1), nat.dtype_code(surv.dtype),
        1 if out_f32 else 0, nat.ptr(wbuf), wbytes, _stream(w_packed))
    nat.check(code, "clt_decode_sparse")
    return out


def decode_route(T: int, d: int, F: int, L: int, tying: str, dtype: torch.dtype, rows: Optional[int] = None) -> int:
    """The schedule (``nat.ROUTE_*``) decode_sparse takes for these shapes when it is given a workspace
    and ``rows`` = tokens x targets of the call (default: all L targets)."""
    lib = nat.load()
    rows = T * L if rows is None else rows
    n_dec = L * (L + 1) // 2 if tying == "none" else L
    slab_bytes = n_dec * F * decoder_pitch(d, dtype) * torch.empty((), dtype=dtype).element_size()
    wbytes = lib.clt_decode_workspace_bytes(T, d, F, L) if _wants_sliced_decode(rows, slab_bytes) else 0
    code = lib.clt_decode_route(T, d, F, L, nat.TYING[tying], nat.dtype_code(dtype), wbytes)
    if code < 0:
        nat.check(code, "clt_decode_route")
    return code


def accumulate_dense(surv: SurvivorList, layer: int, acc: torch.Tensor, init: bool,
                     feat_offset: Optional[torch.Tensor] = None, feat_scale: Optional[torch.Tensor] = None) -> None:
    """acc [T, F] (model dtype) += the survivors of ``layer``, each addition rounded to the model dtype:
    the ``summed_activation`` a decoder tied per target multiplies (decoder.py:208-246).  ``feat_offset``
    / ``feat_scale`` [F]: the target layer's affine terms, applied to the non-zero entries."""
    nat.require_device(acc, "accumulate_dense")
    assert acc.shape == (surv.T, surv.F) and acc.is_contiguous() and acc.dtype == surv.dtype
    for a in (feat_offset, feat_scale):
        assert a is None or (a.dtype == surv.dtype and a.is_contiguous() and a.numel() == surv.F)
    code = nat.load().clt_accumulate_dense(nat.ptr(surv.row_ptr), nat.ptr(surv.col), nat.ptr(surv.val),
                                           nat.ptr(feat_offset), nat.ptr(feat_scale), nat.ptr(acc), surv.T, surv.F,
                                           int(layer), 1 if init else 0, nat.dtype_code(surv.dtype), _stream(acc))
    nat.check(code, "clt_accumulate_dense")


def densify(surv: SurvivorList, out_f32: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Dense [L, T, F] activations (value or 0) from a survivor list (activations.py:65, 347)."""
    dev = surv.row_ptr.device
    odt = torch.float32 if (out_f32 or surv.dtype == torch.float32) else surv.dtype
    if out is None:
        out = torch.empty((surv.L, surv.T, surv.F), dtype=odt, device=dev)
    assert out.stride(2) == 1 and (out.stride(1) == surv.F or surv.T <= 1) and out.dtype == odt
    code = nat.load().clt_densify(nat.ptr(surv.row_ptr), nat.ptr(surv.col), nat.ptr(surv.val), nat.ptr(out),
                                  surv.T, surv.F, surv.L, out.stride(0), nat.dtype_code(surv.dtype),
                                  1 if odt == torch.float32 else 0, nat.current_stream(dev))
    nat.check(code, "clt_densify")
    return out


def decoder_norms(w_packed: torch.Tensor, L: int, tying: str, d: int) -> torch.Tensor:
    """[L, F] per-feature decoder norms in the model dtype (decoder.py:374-485)."""
    nat.require_device(w_packed, "decoder_norms")
    F = w_packed.shape[1]
    assert w_packed.is_contiguous() and w_packed.shape[2] == decoder_pitch(d, w_packed.dtype)
    out = torch.empty((L, F), dtype=w_packed.dtype, device=w_packed.device)
    code = nat.load().clt_decoder_norms(nat.ptr(w_packed), nat.ptr(out), d, F, L, nat.TYING[tying],
                                        nat.dtype_code(w_packed.dtype), _stream(w_packed))
    nat.check(code, "clt_decoder_norms")
    return out


def survivor_rows(surv: SurvivorList) -> torch.Tensor:
    """Row index (layer*T + token) of every survivor, int64 [nnz]."""
    counts = (surv.row_ptr[1:] - surv.row_ptr[:-1]).to(torch.int64)
    return torch.repeat_interleave(torch.arange(surv.L * surv.T, device=counts.device), counts)
