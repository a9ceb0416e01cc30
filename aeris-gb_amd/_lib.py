"""ctypes binding of libaeris_hip.so (the C ABI declared in include/aeris_hip.h).

The library is loaded from ``csrc/`` next to this file.  There is no fallback: if the
library is missing, or a call fails, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes
import os

import torch  # noqa: F401  (imported first so that the HIP runtime torch ships is the one both sides use)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libaeris_hip.so")

OK, EINVAL, EUNSUPPORTED, ELAUNCH = 0, -1, -2, -3
BF16, F32 = 0, 1
NORM_LAYER, NORM_RMS = 0, 1
NORM_THEN_MOD, MOD_THEN_NORM = 0, 1
ACT_NONE, ACT_GELU, ACT_SWIGLU, ACT_SILU = 0, 1, 2, 3

_c_int, _c_i64, _c_f32, _c_vp = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

# name -> (restype, argtypes); must list every symbol include/aeris_hip.h declares
SIGNATURES = {
    "aeris_version": (_c_int, []),
    "aeris_last_error": (ctypes.c_char_p, []),
    "aeris_init": (_c_int, []),
    "aeris_window_index_map": (_c_int, [_c_int] * 7 + [_c_vp]),
    "aeris_relative_position_index": (_c_int, [_c_int, _c_int, _c_vp]),
    "aeris_shift_region_ids": (_c_int, [_c_int] * 6 + [_c_vp]),
    "aeris_window_attention_fwd": (_c_int, [_c_vp, _c_vp, _c_vp] + [_c_int] * 10 + [_c_f32, _c_vp]),
    "aeris_window_attention_heads_fwd": (_c_int, [_c_vp, _c_vp, _c_vp] + [_c_int] * 10 + [_c_f32, _c_int, _c_i64, _c_vp]),
    "aeris_qkv_attention_bias_bytes": (_c_i64, [_c_int, _c_int, _c_int]),
    "aeris_qkv_attention_prepare_bias": (_c_int, [_c_vp, _c_int, _c_int, _c_int, _c_vp, _c_vp]),
    "aeris_qkv_window_attention_fwd": (_c_int, [_c_vp, _c_vp, _c_vp, _c_vp, _c_vp] + [_c_int] * 11 + [_c_f32, _c_vp]),
    "aeris_norm_modulate_fwd": (_c_int, [_c_vp, _c_int, _c_vp, _c_int, _c_vp, _c_vp, _c_int, _c_vp, _c_vp, _c_i64, _c_i64,
                                         _c_i64, _c_int, _c_int, _c_int, _c_f32, _c_vp]),
    "aeris_output_stage_workspace_bytes": (_c_i64, [_c_int, _c_int, _c_int]),
    "aeris_output_stage_fwd": (_c_int, [_c_vp, _c_int, _c_vp, _c_vp, _c_int, _c_vp, _c_vp, _c_i64, _c_vp, _c_vp, _c_i64, _c_i64,
                                        _c_int, _c_int, _c_int, _c_f32, _c_vp, _c_i64, _c_vp]),
    "aeris_output_stage_noalloc_fwd": (_c_int, [_c_vp, _c_int, _c_vp, _c_vp, _c_int, _c_vp, _c_vp, _c_i64, _c_vp, _c_vp, _c_i64,
                                                _c_i64, _c_int, _c_int, _c_int, _c_f32, _c_vp]),
    "aeris_gemm_fwd": (_c_int, [_c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_int, _c_int, _c_i64, _c_int,
                                _c_int, _c_int, _c_i64, _c_i64, _c_vp]),
    "aeris_gemm_heads_fwd": (_c_int, [_c_vp, _c_vp, _c_vp, _c_vp, _c_i64, _c_int, _c_int, _c_int, _c_i64, _c_f32, _c_int,
                                      _c_vp]),
    "aeris_modulation_linear_fwd": (_c_int, [_c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_vp]),
    "aeris_timestep_embedding_fwd": (_c_int, [_c_vp, _c_vp, _c_int, _c_int, _c_f32, _c_vp]),
    "aeris_embed_prepare_fwd": (_c_int, [_c_vp, _c_vp, _c_vp, _c_i64, _c_i64, _c_int, _c_int, _c_int, _c_vp]),
    "aeris_embed_concat_fwd": (_c_int, [_c_vp, _c_int, _c_f32, _c_vp, _c_int, _c_vp, _c_vp, _c_i64, _c_i64, _c_int, _c_int,
                                        _c_vp]),
    "aeris_input_stage_weight_bytes": (_c_i64, [_c_int, _c_int]),
    "aeris_input_stage_pack_weight": (_c_int, [_c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_vp]),
    "aeris_input_stage_fwd": (_c_int, [_c_vp, _c_int, _c_f32, _c_vp, _c_int, _c_vp, _c_i64, _c_vp, _c_vp, _c_int, _c_i64,
                                       _c_int, _c_vp]),
}

_lib = None


class AerisError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"libaeris_hip error {code}: {msg}")
        self.code = code


def lib():
    """Load (once) and return the ctypes handle."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python aeris-gb_amd/build.py` "
                "(there is no fallback path for the HIP kernels)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().aeris_last_error().decode()


def check(code: int):
    if code != OK:
        raise AerisError(code, last_error())


def call(name, *args):
    check(getattr(lib(), name)(*args))
