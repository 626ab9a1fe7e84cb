"""MI355X-native cross-layer-transcoder forward path.

``CrossLayerTranscoder`` mirrors the reference class for encode / decode / forward; the
work is done by hand-written gfx950 kernels in ``lib/libclt_hip.so`` (C ABI in
``include/clt_hip.h``), loaded with ctypes.  The directory name contains a hyphen, so
import it as ``crosslayer_coding_amd`` (the alias module next to this directory) or with
``importlib.import_module("crosslayer-coding_amd")``.
"""

from . import _native, engine  # noqa: F401
from . import activations, base, build, config, decoder, encoder, evaluator, feed, optim, parallel, registry, synth, theta  # noqa: F401
from .activations import BatchTopK, JumpReLU, TokenTopK
from .clt import CrossLayerTranscoder
from .config import CLTConfig
from .engine import SurvivorList
from .optim import CLTAdam
from .evaluator import CLTEvaluator, DeadFeatureTracker
from .feed import DeviceActivationFeed
from .registry import ACTIVATION_REGISTRY, get_activation_fn, register_activation_fn

__all__ = [
    "CrossLayerTranscoder", "CLTConfig", "CLTAdam", "CLTEvaluator", "DeadFeatureTracker", "DeviceActivationFeed", "BatchTopK", "TokenTopK", "JumpReLU", "SurvivorList",
    "ACTIVATION_REGISTRY", "get_activation_fn", "register_activation_fn",
]
