"""Synthetic-model support: seeded normal weights and fp32 -> GGUF block quantizers.

Thin ctypes wrapper over ``lib/libslai_synth.so`` (host-only C++, OpenMP).  The
quantizers follow ggml's reference algorithms; the reference repository itself has no
quantizer, so these only generate inputs (the same bytes go to the device library and
to whatever checks it).
"""
import ctypes as C
import os

import numpy as np

from . import build as _build

GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 0, 1, 2, 8, 12, 13, 14
TYPE_NAMES = {"f32": 0, "f16": 1, "q4_0": 2, "q8_0": 8, "q4_k": 12, "q5_k": 13, "q6_k": 14}
BLOCK_ELEMS = {0: 1, 1: 1, 2: 32, 3: 32, 6: 32, 7: 32, 8: 32, 12: 256, 13: 256, 14: 256, 15: 256}
BLOCK_BYTES = {0: 4, 1: 2, 2: 18, 3: 20, 6: 22, 7: 24, 8: 34, 12: 144, 13: 176, 14: 210, 15: 292}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_build.SYNTH_LIB):
            _build.build_synth()
        L = C.CDLL(_build.SYNTH_LIB)
        L.slai_synth_set_threads.argtypes = [C.c_int]
        L.slai_synth_row_bytes.restype = C.c_size_t
        L.slai_synth_row_bytes.argtypes = [C.c_int, C.c_size_t]
        L.slai_synth_normal.argtypes = [C.c_uint64, C.c_float, C.c_void_p, C.c_size_t]
        L.slai_synth_quantize.restype = C.c_size_t
        L.slai_synth_quantize.argtypes = [C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        L.slai_synth_normal_quantized.restype = C.c_size_t
        L.slai_synth_normal_quantized.argtypes = [C.c_uint64, C.c_float, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p]
        L.slai_synth_f32_to_f16.restype = C.c_uint16
        L.slai_synth_f32_to_f16.argtypes = [C.c_float]
        _lib = L
    return _lib


def row_bytes(ggml_type, ncols):
    return lib().slai_synth_row_bytes(ggml_type, ncols)


def normal(seed, n, std=1.0):
    out = np.empty(n, dtype=np.float32)
    lib().slai_synth_normal(seed, std, out.ctypes.data, n)
    return out


def quantize(ggml_type, x):
    """x: float32 [nrows, ncols] -> uint8 array of packed GGUF blocks (row-major)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    nrows, ncols = x.shape
    rb = row_bytes(ggml_type, ncols)
    if rb == 0 or ncols % BLOCK_ELEMS[ggml_type]:
        raise ValueError("unsupported type/shape for quantize: %r %r" % (ggml_type, x.shape))
    out = np.empty(nrows * rb, dtype=np.uint8)
    n = lib().slai_synth_quantize(ggml_type, x.ctypes.data, nrows, ncols, out.ctypes.data)
    assert n == out.size
    return out


def normal_quantized(seed, ggml_type, nrows, ncols, std=0.02, out=None):
    """Packed blocks of a seeded std*N(0,1) [nrows, ncols] matrix, generated row by row."""
    rb = row_bytes(ggml_type, ncols)
    if rb == 0 or ncols % BLOCK_ELEMS[ggml_type]:
        raise ValueError("unsupported type/shape: %r (%d,%d)" % (ggml_type, nrows, ncols))
    if out is None:
        out = np.empty(nrows * rb, dtype=np.uint8)
    assert out.size == nrows * rb and out.dtype == np.uint8 and out.flags.c_contiguous
    lib().slai_synth_normal_quantized(seed, std, ggml_type, nrows, ncols, out.ctypes.data)
    return out
