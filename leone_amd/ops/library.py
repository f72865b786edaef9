"""Loads the gfx950 kernel library and declares its entry points for ctypes.

There is no substitute path: if the library cannot be built or loaded, the
first kernel call raises.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_double, c_float, c_int, c_void_p

from ..csrc import build as _build
from . import profile


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or failed to launch."""


_lock = threading.Lock()
_lib: ctypes.CDLL | None = None

P = c_void_p
_PROTOTYPES = {
    "leone_embed": [P, c_int, P, P, c_int, c_int, c_int, c_float, P],
    "leone_soft_cap": [P, ctypes.c_long, c_float, P],
    "leone_add_rmsnorm": [P, P, c_int, c_int, ctypes.c_long, P, c_int, c_float, P, c_int, P, c_int, c_int, P, P],
    "leone_swiglu": [P, P, c_int, c_int, c_int, P],
    "leone_rope_table": [P, P, c_double, c_int, c_int, P],
    "leone_qk_norm_rope_write": [P, c_int, c_int, ctypes.c_long, P, P, P, c_int, P, P, c_int, c_float, P, P, c_int, c_int, c_int,
                                 P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, P],
    "leone_attention_rows": [P, P, P, P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                             c_int, P],
    "leone_attention_decode_projected": [P, c_int, c_int, ctypes.c_long, P, P, c_int, c_float, P, P, c_int, c_int, c_int, P, P, P, c_int,
                                         P, P, P, c_int, P, P, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, P],
    "leone_attention_decode": [P, P, P, P, P, P, P, c_int, P, P, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                               c_int, P],
    "leone_attention_prefill": [P, P, P, P, P, P, c_int, P, c_int, c_int, c_int, c_int, c_int, c_float, c_int, P, P,
                                c_int, P],
    "leone_gemm_f32": [P, P, P, c_int, c_int, c_int, P],
    "leone_gemm_fused_bf16": [P, c_int, P, P, c_int, c_float, P, c_int, P, c_int, c_int, c_int, c_int, c_int, P, P, P, P,
                              c_int, P],
    "leone_gemm_rows_bf16": [P, P, c_int, P, c_int, c_int, c_int, c_int, c_int, c_int, ctypes.c_long, c_int, c_int, P],
    "leone_gemm_rows_shape_built": [c_int, c_int, c_int],
    "leone_argmax": [P, P, P, P, c_int, c_int, P],
    "leone_peak_read": [P, ctypes.c_long, P, c_int, P],
    "leone_peak_copy": [P, P, ctypes.c_long, c_int, P],
    "leone_peak_mfma": [c_int, c_int, c_int, P, P],
    "leone_library_product": [P, P, P, c_int, c_int, c_int, c_int, c_int, P],
    "leone_library_product_tune": [P, P, c_int, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, P, P, P, P],
    "leone_library_product_forget": [c_int, c_int, c_int, c_int, c_int],
    "leone_sample_temperature": [P, P, P, P, P, P, P, P, c_int, c_int, P],
    "leone_top_candidates": [P, P, P, P, c_int, c_int, c_int, P],
    "leone_sample_truncated": [P, P, P, c_int, c_int, P],
}


def library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            path = _build.library_path()
            if path is None:
                path = _build.build(verbose=True)
            lib = ctypes.CDLL(path)
            lib.leone_last_error.restype = c_char_p
            lib.leone_last_error.argtypes = []
            lib.leone_attention_prefill_tile_rows.restype = c_int
            lib.leone_attention_prefill_tile_rows.argtypes = []
            lib.leone_attention_prefill_group_tiles.restype = c_int
            lib.leone_attention_prefill_group_tiles.argtypes = []
            lib.leone_attention_prefill_max_splits.restype = c_int
            lib.leone_attention_prefill_max_splits.argtypes = []
            lib.leone_top_candidates_max.restype = c_int
            lib.leone_top_candidates_max.argtypes = []
            lib.leone_argmax_chunk.restype = c_int
            lib.leone_argmax_chunk.argtypes = []
            lib.leone_sample_truncated_stages.restype = c_int
            lib.leone_sample_truncated_stages.argtypes = []
            lib.leone_sample_truncated_params.restype = c_int
            lib.leone_sample_truncated_params.argtypes = []
            lib.leone_peak_mfma_flops.restype = ctypes.c_double
            lib.leone_peak_mfma_flops.argtypes = [c_int, c_int]
            lib.leone_gemm_rows_max_rows.restype = c_int
            lib.leone_gemm_rows_max_rows.argtypes = []
            lib.leone_gemm_rows_chunk.restype = c_int
            lib.leone_gemm_rows_chunk.argtypes = [c_int]
            lib.leone_library_product_available.restype = c_int
            lib.leone_library_product_available.argtypes = []
            lib.leone_library_product_tuned.restype = c_int
            lib.leone_library_product_tuned.argtypes = [c_int, c_int, c_int, c_int, c_int]
            for name, argtypes in _PROTOTYPES.items():
                fn = getattr(lib, name)
                fn.argtypes = argtypes
                fn.restype = c_int
            _lib = lib
    return _lib


def call(name: str, *args) -> None:
    lib = library()
    if profile.recording():
        with profile.span(profile.OPERATIONS.get(name, name)):
            status = getattr(lib, name)(*args)
    else:
        status = getattr(lib, name)(*args)
    if status != 0:
        raise KernelError(lib.leone_last_error().decode("utf-8", "replace"))
