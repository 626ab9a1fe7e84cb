"""ctypes binding of libclt_hip.so (the C ABI declared in include/clt_hip.h).

torch is imported first so that the library binds to the HIP runtime torch has
already loaded: one runtime per process, so torch's streams and device pointers
are the library's streams and pointers.  There is no fallback: when the library is
missing, or a call is made without a ROCm device, this module raises.
"""

from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import build as _build

CLT_F32, CLT_BF16, CLT_F16 = 0, 1, 2
TYING = {"none": 0, "per_source": 1, "per_target": 2}
TOPK_PER_LAYER, TOPK_GLOBAL = 0, 1
PRED_GE_THETA, PRED_GT_ZERO, PRED_NONZERO = 0, 1, 2
ROUTE_GENERIC, ROUTE_SINGLE, ROUTE_SLICED, ROUTE_SLICED_ALL_SOURCES, ROUTE_QUARTER, ROUTE_LINE = 0, 1, 2, 3, 4, 5

_i64 = ctypes.c_int64
_vp = ctypes.c_void_p
_int = ctypes.c_int
_u64 = ctypes.c_uint64
_sz = ctypes.c_size_t
_f64 = ctypes.c_double

# name -> (restype, argtypes); mirrors include/clt_hip.h one to one
_SIGNATURES = {
    "clt_version": (_int, []),
    "clt_error_string": (ctypes.c_char_p, [_int]),
    "clt_encode": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "clt_encode_fast_path": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "clt_encode_segmented": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "clt_colstats": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "clt_colstats_full": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "clt_selected_min_accumulate": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp, _vp, _vp, _sz, _vp]),
    "clt_batchtopk_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _int, _int]),
    "clt_batchtopk_select": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp, _int, _vp, _vp, _vp, _vp, _sz, _vp]),
    "clt_encode_collect_supported": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "clt_encode_collect_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _int]),
    "clt_encode_collect": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "clt_collect_select": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _sz, _vp]),
    "clt_tokentopk_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _int, _int]),
    "clt_tokentopk_select": (_int, [_vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp, _int, _vp, _vp, _vp, _vp, _sz, _vp]),
    "clt_threshold_count": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, _int, _int, _vp, _vp, _sz, _vp]),
    "clt_threshold_count_static": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, _int, _int, _vp, _vp]),
    "clt_threshold_emit": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, _int, _int, _vp, _vp, _vp, _vp, _vp]),
    "clt_threshold_dense": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, _int, _int, _vp, _vp]),
    "clt_survivors_fit": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "clt_encode_threshold_supported": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "clt_encode_threshold_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64, _int]),
    "clt_encode_threshold_count": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int, _vp, _vp, _sz, _vp]),
    "clt_encode_threshold_emit": (_int, [_i64, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "clt_encode_threshold_recover": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _int,
                                            _vp, _i64, _vp, _vp, _sz, _vp]),
    "clt_poison_if": (_int, [_vp, _i64, _vp, _vp]),
    "clt_pack_decoder": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp]),
    "clt_decode_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "clt_decode_sparse": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _i64, _i64, _u64, _int, _int, _vp, _sz, _vp]),
    "clt_decode_route": (_int, [_i64, _i64, _i64, _i64, _int, _int, _sz]),
    "clt_decoder_pitch": (_i64, [_i64, _int]),
    "clt_decoder_slab_elems": (_i64, [_i64, _i64, _i64, _int, _int]),
    "clt_accumulate_dense": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "clt_densify": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "clt_mse_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "clt_mse_loss_grad": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _int, _vp, _vp, _f64, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "clt_decode_backward_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "clt_decode_backward_values": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _u64, _i64, _int, _vp, _vp, _sz, _vp]),
    "clt_feature_affine_grad": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _u64, _i64, _int, _vp, _vp, _vp, _sz, _vp]),
    "clt_skip_weight_grad": (_int, [_vp, _vp, _vp, _i64, _i64, _int, _int, _vp]),
    "clt_feature_lists_workspace_bytes": (_sz, [_i64, _i64]),
    "clt_feature_lists": (_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "clt_decoder_weight_grad": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "clt_encoder_weight_grad": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "clt_adam_step": (_int, [_vp, _vp, _vp, _vp, _i64, _f64, _f64, _f64, _f64, _i64, _int, _vp]),
    "clt_decoder_weight_grad_adam": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _f64, _f64, _f64, _f64, _i64, _int, _vp]),
    "clt_unpack_decoders": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "clt_decoder_fingerprint": (_int, [_vp, _i64, _i64, _i64, _int, _vp, _vp, _int, _vp]),
    "clt_pack_decoders_if": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _vp, _vp]),
    "clt_bias_sum": (_int, [_vp, _i64, _i64, _i64, _int, _u64, _int, _vp, _vp]),
    "clt_decoder_tile_width": (_int, [_i64, _i64, _i64, _int]),
    "clt_decoder_tiles_workspace_bytes": (_sz, [_i64, _int]),
    "clt_tile_decoders": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "clt_untile_decoders": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "clt_decoder_weight_grad_adam_tiled": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f64, _f64, _f64,
                                                  _f64, _i64, _int, _vp, _sz, _vp]),
    "clt_adam_step_decoder": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _f64, _f64, _f64, _f64, _i64, _int, _vp]),
    "clt_adam_step_decoders": (_int, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _f64, _f64, _f64, _f64, _i64, _int, _vp]),
    "clt_adam_step_many": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _f64, _f64, _f64, _f64, _i64, _int, _vp]),
    "clt_decoder_norms": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _int, _vp]),
    "clt_scatter_survivor_values": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _vp]),
    "clt_jumprelu_theta_grad_workspace_bytes": (_sz, [_i64]),
    "clt_jumprelu_theta_grad": (_int, [_vp, _vp, _vp, _i64, _i64, _f64, _int, _vp, _vp, _sz, _vp]),
    "clt_probe_gather": (_int, [_vp, _i64, _i64, _vp, _i64, _i64, _int, _vp, _vp]),
    "clt_feed_gather": (_int, [_vp, _int, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _int, _vp, _vp, _vp, _vp, _f64, _vp, _vp,
                              _i64, _i64, _int, _vp]),
    "clt_survivor_metrics": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, ctypes.c_float, _vp, _vp, _vp]),
    "clt_dead_feature_update": (_int, [_vp, _vp, _i64, _vp]),
    "clt_reconstruction_stats_workspace_bytes": (_sz, [_i64, _i64]),
    "clt_reconstruction_stats": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _int, _vp, _vp, _f64, _vp, _vp, _sz, _vp]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None


class CLTNativeError(RuntimeError):
    """A C-ABI call returned a negative code."""


def library_path() -> str:
    return _build.library_path()


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    """Load libclt_hip.so, building it first only when no built library exists."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        if not build_if_missing:
            raise CLTNativeError(f"{path} is missing; run crosslayer-coding_amd/build.py")
        _build.build()
    lib = ctypes.CDLL(path)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = library and header disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().clt_error_string(code).decode()
        raise CLTNativeError(f"{what} failed with code {code}: {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return CLT_F32
    if dtype == torch.bfloat16:
        return CLT_BF16
    if dtype == torch.float16:
        return CLT_F16      # forward-path entry points; the backward and optimiser kernels return CLT_ERR_DTYPE
    raise CLTNativeError(f"unsupported CLT dtype {dtype}; the HIP kernels implement float32, bfloat16 and float16")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def require_device(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise CLTNativeError(
            f"{what}: tensor is on {t.device}; the CLT kernels run on a ROCm GPU only and there is no CPU path")


def current_stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
