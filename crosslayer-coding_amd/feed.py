"""Activation-store feed: from (chunk, row) indices to the normalised batch slabs on the device.

Host-side mirror of the batch assembly of the reference's manifest-driven stores
(clt/training/data/manifest_activation_store.py:328-958, local_activation_store.py:87-166) with
the file / HTTP transport left to the caller:

* `read_manifest` parses ``index.bin`` (legacy ``uint32[N, 2]`` rows of (chunk, row), or the
  16-byte (chunk_id, num_tokens, offset) records expanded to per-row entries);
* `prepare_normalization` turns ``norm_stats.json`` into fp32 ``[L, d]`` tables the way
  ``_prep_norm`` does (std + 1e-6, any malformed layer disables normalisation);
* `DeviceActivationFeed.parse_batch` is ``_fetch_and_parse_batch``: rows grouped by chunk in
  ascending chunk order, inside a chunk in the sampler's order, normalised in fp32 and cast once.
  Every chunk of a batch is one `clt_feed_gather` launch that writes all layers, inputs and
  targets into two ``[L, T, d]`` slabs - no per-layer tensors, no ``torch.cat``, no fp32 copy.
  Chunks can be made resident (288 GB of HBM hold whole datasets; pinned host memory works too,
  the kernel reads it in place) or arrive per batch as the bytes of ``_fetch_slice``.
"""

from __future__ import annotations

import logging
import math
from pathlib import Path
from typing import Any, Callable, Dict, List, Optional, Tuple, Union

import numpy as np
import torch

from . import _native as nat

logger = logging.getLogger(__name__)

NORM_MODES = {"none": 0, "mean_std": 1, "sqrt_d_model": 2}
_SRC_CODES = {torch.float32: nat.CLT_F32, torch.bfloat16: nat.CLT_BF16, torch.float16: nat.CLT_F16}


def read_manifest(path: Union[str, Path], total_tokens: Optional[int] = None) -> Optional[np.ndarray]:
    """``index.bin`` as ``uint32[N, 2]`` rows of (chunk_id, row) (local_activation_store.py:87-166).

    A file whose size is a multiple of 16 is first read as (int32 chunk_id, int32 num_tokens,
    int64 offset) records and expanded; when ``total_tokens`` is given and the records do not add
    up to it the file is read as legacy pairs instead.  Returns None when the file is missing or
    fits neither format."""
    path = Path(path)
    if not path.exists():
        logger.error(f"Manifest file not found: {path}")
        return None
    size = path.stat().st_size
    if size % 16 == 0:
        rec = np.fromfile(path, dtype=np.dtype([("chunk_id", np.int32), ("num_tokens", np.int32), ("offset", np.int64)]))
        chunk_ids = rec["chunk_id"].astype(np.uint32)
        counts = rec["num_tokens"].astype(np.uint32)
        if total_tokens is not None and total_tokens > 0 and int(counts.sum()) != total_tokens:
            logger.warning("3-field manifest parse produced total_rows=%d but metadata reports %d tokens. "
                           "Falling back to legacy 2-field manifest parsing.", int(counts.sum()), total_tokens)
            return np.fromfile(path, dtype=np.uint32).reshape(-1, 2)
        total = int(counts.sum())
        data = np.empty((total, 2), dtype=np.uint32)
        at = 0
        for cid, n in zip(chunk_ids, counts):
            n = int(n)
            if n == 0:
                continue
            data[at:at + n, 0] = cid
            data[at:at + n, 1] = np.arange(n, dtype=np.uint32)
            at += n
        return data
    if size % 8 == 0:
        return np.fromfile(path, dtype=np.uint32).reshape(-1, 2)
    logger.error(f"Manifest file size ({size} bytes) is not compatible with known formats (8 or 16 bytes per row).")
    return None


def prepare_normalization(norm_stats: Optional[Dict[str, Any]], layer_indices: List[int], d_model: int):
    """``_prep_norm`` (manifest_activation_store.py:563-690) for ``mean_std``: returns
    (apply, mean_in, std_in, mean_tg, std_tg) with fp32 ``[L, d]`` tables (std + 1e-6), or
    (False, None, ...) when the statistics are absent, malformed, non-positive or miss a layer."""
    off = (False, None, None, None, None)
    if not norm_stats:
        logger.warning("mean_std normalization requested but no stats data loaded.")
        return off
    L = len(layer_indices)
    pos = {l: i for i, l in enumerate(layer_indices)}
    tabs = [torch.zeros(L, d_model), torch.ones(L, d_model), torch.zeros(L, d_model), torch.ones(L, d_model)]
    missing = set(layer_indices)
    try:
        for key, stats in norm_stats.items():
            layer = int(key)
            if layer not in pos:
                logger.warning(f"Normalization stats contain unknown layer index {layer}. Skipping.")
                continue
            missing.discard(layer)
            for kind, (mt, st) in (("inputs", (tabs[0], tabs[1])), ("targets", (tabs[2], tabs[3]))):
                if not (kind in stats and "mean" in stats[kind] and "std" in stats[kind]):
                    return off
                try:
                    mean = torch.tensor(stats[kind]["mean"], dtype=torch.float32)
                    std = torch.tensor(stats[kind]["std"], dtype=torch.float32) + 1e-6
                except (ValueError, TypeError) as e:
                    logger.warning(f"Layer {layer} {kind} mean/std failed tensor conversion: {e}. Disabling normalization.")
                    return off
                if torch.any(std <= 0):
                    logger.warning(f"Layer {layer} {kind} std contains non-positive values after adding epsilon. "
                                   "Disabling normalization.")
                    return off
                mt[pos[layer]] = mean
                st[pos[layer]] = std
    except (KeyError, ValueError, TypeError, RuntimeError) as e:
        logger.error(f"Error processing normalization stats (e.g., invalid format, wrong keys): {e}. Disabling normalization.")
        return off
    if missing:
        logger.warning(f"Normalization stats missing for layers: {sorted(missing)}. Disabling normalization.")
        return off
    return (True, *tabs)


class _Chunk:
    __slots__ = ("data", "rows", "dtype", "layer_stride", "target_offset")

    def __init__(self, data: torch.Tensor, rows: int, dtype: torch.dtype, layer_stride: int, target_offset: int):
        self.data, self.rows, self.dtype = data, rows, dtype
        self.layer_stride, self.target_offset = layer_stride, target_offset


class DeviceActivationFeed:
    """Batch assembly of ManifestActivationStore on the device.

    ``dtype`` is both the stored element type the bytes are read as and the type of the batch,
    as in the reference (manifest_activation_store.py:881-886); ``out_dtype`` may name a
    different batch type (float32, bfloat16 or float16)."""

    def __init__(self, num_layers: int, d_model: int, dtype: Union[str, torch.dtype] = "bfloat16",
                 device: Union[str, torch.device] = "cuda:0", normalization_method: str = "none",
                 norm_stats: Optional[Dict[str, Any]] = None, out_dtype: Optional[torch.dtype] = None):
        if normalization_method not in NORM_MODES:
            raise ValueError(f"Invalid normalization_method: {normalization_method}. "
                             f"Must be one of ['none', 'mean_std', 'sqrt_d_model']")
        self.num_layers, self.d_model = num_layers, d_model
        self.layer_indices = list(range(num_layers))
        self.device = torch.device(device)
        self.dtype = getattr(torch, dtype) if isinstance(dtype, str) else dtype
        if self.dtype not in _SRC_CODES:
            raise ValueError(f"Unsupported store dtype {self.dtype}")
        self.out_dtype = out_dtype or self.dtype
        if self.out_dtype not in _SRC_CODES:
            raise ValueError(f"Unsupported batch dtype {self.out_dtype}: the kernels take float32, bfloat16 or float16")
        self.bytes_per_element = torch.finfo(self.dtype).bits // 8
        self.bytes_per_row = d_model * self.bytes_per_element
        self.normalization_method = normalization_method
        self.apply_normalization = False
        self._tables: Tuple[Optional[torch.Tensor], ...] = (None, None, None, None)
        if normalization_method == "mean_std":
            ok, *tabs = prepare_normalization(norm_stats, self.layer_indices, d_model)
            self.apply_normalization = ok
            if ok:
                self._tables = tuple(t.to(self.device).contiguous() for t in tabs)
        elif normalization_method == "sqrt_d_model":
            self.apply_normalization = True
        self._chunks: Dict[int, _Chunk] = {}
        self._staging: List[Optional[Tuple[torch.Tensor, torch.cuda.Event]]] = [None, None]
        self._slot = 0

    # ---- resident chunks ----
    def add_chunk(self, chunk_id: int, data: Union[torch.Tensor, np.ndarray, bytes], rows: Optional[int] = None,
                  where: str = "device") -> None:
        """Keep a whole chunk resident.  ``data``: ``[L, 2, rows, d]`` (inputs, targets per layer) as a
        tensor / array of the store dtype, or the same as raw bytes with ``rows`` given.  ``where``:
        "device" (HBM) or "pinned" (page-locked host memory the kernel reads in place)."""
        t = self._as_store_tensor(data, rows)
        n = t.shape[2]
        if where == "pinned":
            held = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
            held.copy_(t)
        elif where == "device":
            held = t.to(self.device).contiguous()
        else:
            raise ValueError("where must be 'device' or 'pinned'")
        self._chunks[int(chunk_id)] = _Chunk(held, n, self.dtype, 2 * n * self.d_model, n * self.d_model)

    def _as_store_tensor(self, data, rows: Optional[int]) -> torch.Tensor:
        L, d = self.num_layers, self.d_model
        if isinstance(data, (bytes, bytearray, memoryview)):
            if rows is None:
                raise ValueError("rows is required for raw bytes")
            want = rows * self.bytes_per_row * 2 * L
            if len(data) != want:
                raise ValueError(f"Incorrect byte size. Expected {want}, got {len(data)}")
            return torch.frombuffer(bytearray(data), dtype=self.dtype).reshape(L, 2, rows, d)
        t = torch.from_numpy(data) if isinstance(data, np.ndarray) else data
        if t.dim() != 4 or t.shape[0] != L or t.shape[1] != 2 or t.shape[3] != d:
            raise ValueError(f"chunk must be [L={L}, 2, rows, d={d}], got {tuple(t.shape)}")
        return t.to(self.dtype).contiguous()

    # ---- staging for fetched slices ----
    def _stage(self, nbytes: int) -> torch.Tensor:
        """A pinned buffer no launch still reads: two buffers take turns, each guarded by an event."""
        self._slot ^= 1
        held = self._staging[self._slot]
        if held is not None:
            held[1].synchronize()
        if held is None or held[0].numel() < nbytes:
            buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, pin_memory=True)
        else:
            buf = held[0]
        self._staging[self._slot] = (buf, torch.cuda.Event())
        return buf

    # ---- the batch ----
    def parse_batch(self, idxs: np.ndarray,
                    fetch_slice: Optional[Callable[[int, np.ndarray], bytes]] = None
                    ) -> Tuple[Dict[int, torch.Tensor], Dict[int, torch.Tensor]]:
        """``_fetch_and_parse_batch`` (manifest_activation_store.py:776-958).  ``idxs`` ``[N, 2]`` of
        (chunk, row).  Chunks added with `add_chunk` are read where they live; for the others
        ``fetch_slice(chunk_id, sorted_rows)`` must return the reference's wire bytes."""
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise nat.CLTNativeError("DeviceActivationFeed.parse_batch: the feed kernel runs on a ROCm GPU only and "
                                     "there is no CPU path")
        idxs = np.asarray(idxs)
        if idxs.ndim != 2 or idxs.shape[1] != 2:
            raise ValueError(f"idxs must be Nx2, got shape {idxs.shape}")
        N, L, d = idxs.shape[0], self.num_layers, self.d_model
        x = torch.empty((L, N, d), dtype=self.out_dtype, device=self.device)
        tg = torch.empty((L, N, d), dtype=self.out_dtype, device=self.device)
        if N == 0:
            return {l: x[l] for l in self.layer_indices}, {l: tg[l] for l in self.layer_indices}
        unique_chunks, inverse = np.unique(idxs[:, 0], return_inverse=True)
        pieces = []
        stage_bytes = 0
        for i, chunk_id in enumerate(unique_chunks):
            rows = idxs[inverse == i, 1].astype(np.int64)
            chunk = self._chunks.get(int(chunk_id))
            if chunk is not None:
                if rows.size and (rows.min() < 0 or rows.max() >= chunk.rows):
                    raise IndexError(f"row index out of range for chunk {int(chunk_id)} ({chunk.rows} rows)")
                pieces.append((chunk, rows.astype(np.int32), None))
                continue
            if fetch_slice is None:
                raise RuntimeError(f"Failed to fetch data for chunk(s): [{int(chunk_id)}]: not resident and no fetch_slice")
            sorted_rows = np.sort(rows)
            raw = fetch_slice(int(chunk_id), sorted_rows.astype(np.uint32))
            want = len(sorted_rows) * self.bytes_per_row * 2 * L
            if len(raw) != want:
                raise ValueError(f"Incorrect byte size fetched for chunk {int(chunk_id)}. Expected {want}, got {len(raw)}")
            reorder = np.searchsorted(sorted_rows, rows).astype(np.int32)
            pieces.append((None, reorder, raw))
            stage_bytes += (want + 255) & ~255
        stage = self._stage(stage_bytes) if stage_bytes else None
        lib = nat.load()
        stream = torch.cuda.current_stream(self.device).cuda_stream
        mode = NORM_MODES[self.normalization_method] if self.apply_normalization else 0
        tabs = [nat.ptr(t) if (t is not None and mode == 1) else None for t in self._tables]
        scale = math.sqrt(d) if mode == 2 else 1.0
        # all row indices of the batch go up in one copy; each piece points into it
        index_dev = torch.from_numpy(np.concatenate([p[1] for p in pieces])).to(self.device)
        out_row, at = 0, 0
        for chunk, index, raw in pieces:
            n = int(index.shape[0])
            if chunk is not None:
                src_ptr, src_rows = chunk.data.data_ptr(), chunk.rows
                layer_stride, target_offset = chunk.layer_stride, chunk.target_offset
            else:
                view = stage[at:at + len(raw)]
                view.numpy()[:] = np.frombuffer(raw, dtype=np.uint8)     # the one host copy, into pinned memory
                src_ptr, src_rows = view.data_ptr(), n
                layer_stride, target_offset = 2 * n * d, n * d
                at += (len(raw) + 255) & ~255
            code = lib.clt_feed_gather(src_ptr, _SRC_CODES[self.dtype], src_rows, layer_stride, target_offset,
                                       index_dev.data_ptr() + 4 * out_row, n, d, L, mode, *tabs, scale, nat.ptr(x),
                                       nat.ptr(tg), out_row, N, nat.dtype_code(self.out_dtype), stream)
            nat.check(code, "clt_feed_gather")
            out_row += n
        if stage is not None:
            self._staging[self._slot][1].record(torch.cuda.current_stream(self.device))
        return {l: x[l] for l in self.layer_indices}, {l: tg[l] for l in self.layer_indices}
