"""ctypes binding of libm2_amd.so (the C ABI declared in include/m2_amd.h).

There is no CPU fallback: if the shared library has not been built, importing this module raises,
and every wrapper raises RuntimeError with the library's own message when a call fails.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libm2_amd.so")

M2_DTYPE_F32 = 0
M2_DTYPE_BF16 = 1
M2_HYENA_FILTER_STATIC_SCRATCH_BYTES = 20 << 20


class HyenaFilterParams(ctypes.Structure):
    """Mirror of `m2_hyena_filter_params`."""
    _fields_ = [(n, c_void_p) for n in (
        "z", "t", "freq", "deltas",
        "w0", "b0", "w1", "b1", "w2", "b2", "w3",
        "rw0", "rb0", "rw1", "rb1", "rw2", "rb2", "rw3")]


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python m2_amd/build.py` (hipcc, gfx950). "
            "m2_amd has no CPU or PyTorch fallback for its kernels.")
    lib = ctypes.CDLL(LIB_PATH)
    lib.m2_version.restype = c_int
    lib.m2_last_error.restype = c_char_p
    lib.m2_hyena_filter_workspace_bytes.restype = c_size_t
    lib.m2_hyena_filter_workspace_bytes.argtypes = [c_int, c_int, c_int, c_int]
    lib.m2_hyena_filter_fwd.restype = c_int
    lib.m2_hyena_filter_fwd.argtypes = [POINTER(HyenaFilterParams), c_int, c_int, c_int, c_int, c_int, c_float,
                                        c_float, c_void_p, c_void_p, c_void_p]
    lib.m2_hyena_filter_fwd_static.restype = c_int
    lib.m2_hyena_filter_fwd_static.argtypes = [POINTER(HyenaFilterParams), c_int, c_int, c_int, c_int, c_int, c_float,
                                               c_float, c_void_p, c_void_p]
    lib.m2_fftconv_supported_seqlen.restype = c_int
    lib.m2_fftconv_supported_seqlen.argtypes = [c_int]
    lib.m2_filter_spectrum_bytes.restype = c_size_t
    lib.m2_filter_spectrum_bytes.argtypes = [c_int, c_int]
    lib.m2_filter_spectrum_fwd.restype = c_int
    lib.m2_filter_spectrum_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p]
    lib.m2_mixer_core_fwd.restype = c_int
    lib.m2_mixer_core_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                      c_int, c_int, c_void_p]
    lib.m2_fftconv_fwd.restype = c_int
    lib.m2_fftconv_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
    lib.m2_mixer_filters_workspace_bytes.restype = ctypes.c_size_t
    lib.m2_mixer_filters_workspace_bytes.argtypes = [c_int] * 5
    lib.m2_mixer_filters_fwd.restype = c_int
    lib.m2_mixer_filters_fwd.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float,
                                         c_void_p, c_void_p, c_void_p]
    lib.m2_blockdiag_glu_fwd.restype = c_int
    lib.m2_blockdiag_glu_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
    lib.m2_blockdiag_linear_fwd.restype = c_int
    lib.m2_blockdiag_linear_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                            c_int, c_void_p]
    lib.m2_blockdiag_linear_f32_fwd.restype = c_int
    lib.m2_blockdiag_linear_f32_fwd.argtypes = [c_void_p] * 4 + [c_int] * 4 + [c_void_p]
    lib.m2_mlp_fused_supported.restype = c_int
    lib.m2_mlp_fused_supported.argtypes = [c_int, c_int, c_int]
    lib.m2_mlp_fused_fwd.restype = c_int
    lib.m2_mlp_fused_fwd.argtypes = [c_void_p] * 5 + [c_int] * 5 + [c_void_p]
    lib.m2_mlp_fused_packed_bytes.restype = ctypes.c_long
    lib.m2_mlp_fused_packed_bytes.argtypes = [c_int, c_int, c_int]
    lib.m2_mlp_fused_pack.restype = c_int
    lib.m2_mlp_fused_pack.argtypes = [c_void_p] * 3 + [c_int] * 3 + [c_void_p]
    lib.m2_glu_stream_supported.restype = c_int
    lib.m2_glu_stream_supported.argtypes = [c_int, c_int, c_int]
    lib.m2_glu_stream_packed_bytes.restype = ctypes.c_long
    lib.m2_glu_stream_packed_bytes.argtypes = [c_int, c_int, c_int]
    lib.m2_glu_stream_pack.restype = c_int
    lib.m2_glu_stream_pack.argtypes = [c_void_p] * 2 + [c_int] * 3 + [c_void_p]
    lib.m2_glu_stream_fwd.restype = c_int
    lib.m2_glu_stream_fwd.argtypes = [c_void_p] * 3 + [c_int] * 4 + [c_void_p]
    lib.m2_layernorm_bf16_fwd.restype = c_int
    lib.m2_layernorm_bf16_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                          c_void_p]
    lib.m2_layernorm_fwd.restype = c_int
    lib.m2_layernorm_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_void_p]
    lib.m2_blockdiag_linear_layernorm_supported.restype = c_int
    lib.m2_blockdiag_linear_layernorm_supported.argtypes = [c_int, c_int, c_int]
    lib.m2_blockdiag_linear_layernorm_fwd.restype = c_int
    lib.m2_blockdiag_linear_layernorm_fwd.argtypes = [c_void_p] * 6 + [c_float] + [c_void_p] * 3 + [c_int] * 4 + [c_void_p]
    lib.m2_embed_layernorm_fwd.restype = c_int
    lib.m2_embed_layernorm_fwd.argtypes = ([c_void_p] * 6 + [c_int] * 3 + [c_void_p] * 2 + [c_float] + [c_void_p] * 4
                                           + [c_int, c_int, c_int, c_void_p])
    return lib


lib = _load()

EXPORTS = ["m2_version", "m2_last_error", "m2_hyena_filter_workspace_bytes", "m2_hyena_filter_fwd", "m2_hyena_filter_fwd_static", "m2_mixer_filters_workspace_bytes", "m2_mixer_filters_fwd",
           "m2_fftconv_supported_seqlen", "m2_filter_spectrum_bytes", "m2_filter_spectrum_fwd", "m2_mixer_core_fwd",
           "m2_fftconv_fwd", "m2_blockdiag_glu_fwd", "m2_blockdiag_linear_fwd", "m2_blockdiag_linear_f32_fwd", "m2_mlp_fused_supported", "m2_mlp_fused_packed_bytes", "m2_mlp_fused_pack", "m2_mlp_fused_fwd", "m2_glu_stream_supported", "m2_glu_stream_packed_bytes", "m2_glu_stream_pack", "m2_glu_stream_fwd", "m2_layernorm_fwd", "m2_layernorm_bf16_fwd",
           "m2_embed_layernorm_fwd", "m2_blockdiag_linear_layernorm_supported", "m2_blockdiag_linear_layernorm_fwd"]


def check(rc: int) -> None:
    if rc != 0:
        msg = lib.m2_last_error()
        raise RuntimeError(f"libm2_amd error {rc}: {msg.decode() if msg else '?'}")
