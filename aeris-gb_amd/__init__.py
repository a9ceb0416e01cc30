"""MI355X-native Swin denoiser hot path of AERIS window-partitioned inference.

The directory name carries a hyphen, so import it with
``importlib.import_module("aeris-gb_amd")``; all intra-package imports are relative.
"""
from . import _lib, ops  # noqa: F401
from ._lib import AerisError, LIB_PATH  # noqa: F401
from .model import (  # noqa: F401
    Attention,
    BlockOptions,
    FeedForward,
    InputStage,
    LocalAERIS,
    Mlp,
    ModulationLinear,
    OutputStage,
    PositionalEncoding2D,
    RoPE2D,
    SwinLayer,
    convert_inference_checkpoint,
    modulate,
    swin_shift,
    timestep_embedding,
)
from .sampler import TrigFlowSampler, sigma_schedule  # noqa: F401

__all__ = [n for n in dir() if not n.startswith("_")]
