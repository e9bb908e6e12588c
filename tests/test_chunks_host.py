"""CPU checks of the device-side layout and lane-chunk decoders (slai_amd/csrc/quant_formats.h),
built for the host: repack + element dequantisation must reproduce the oracle bit for bit, and
the per-chunk dot products must add up to W.x."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from helpers import random_blocks
from slai_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
TYPES = [0, 1, 2, 3, 6, 7, 8, 12, 13, 14, 15]


@pytest.fixture(scope="module")
def cc(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("cc") / "libchunk_check.so")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
                           "-I", os.path.join(ROOT, "slai_amd", "csrc"),
                           os.path.join(HERE, "native", "chunk_check.cpp"), "-o", out])
    L = C.CDLL(out)
    L.cc_row_stride.restype = C.c_size_t
    L.cc_row_stride.argtypes = [C.c_int, C.c_uint32]
    L.cc_repack.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
    L.cc_dequant.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
    L.cc_gemv.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
    L.cc_cover.restype = C.c_uint32
    L.cc_cover.argtypes = [C.c_int, C.c_uint32]
    L.cc_tiled_bytes.restype = C.c_size_t
    L.cc_tiled_bytes.argtypes = [C.c_int, C.c_uint32, C.c_uint32]
    L.cc_tiled_rows_log2.restype = C.c_uint32
    L.cc_tiled_rows_log2.argtypes = [C.c_int, C.c_uint32, C.c_uint32]
    L.cc_tiled_repack.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
    L.cc_tiled_dequant.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p]
    L.cc_tiled_gemv.argtypes = [C.c_int, C.c_void_p, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
    L.cc_encode_f16.restype = C.c_uint16
    L.cc_encode_f16.argtypes = [C.c_float]
    L.cc_decode_f16.restype = C.c_float
    L.cc_decode_f16.argtypes = [C.c_uint16]
    return L


def repack(cc, t, raw, nrows, ncols):
    dev = np.zeros(nrows * cc.cc_row_stride(t, ncols), np.uint8)
    cc.cc_repack(t, raw.ctypes.data, nrows, ncols, dev.ctypes.data)
    return dev


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("ncols", [256, 768, 2816])
def test_repack_dequant_bit_exact(cc, oracle_lib, t, ncols):
    nrows = 5
    be = oracle_lib.slo_block_elems(t)
    raw = random_blocks(t, nrows * ncols // be, seed=7 * t + ncols)
    ref = np.empty(nrows * ncols, np.float32)
    assert oracle_lib.slo_dequantize(t, raw.ctypes.data, nrows * ncols, ref.ctypes.data) == 0
    dev = repack(cc, t, raw, nrows, ncols)
    got = np.empty(nrows * ncols, np.float32)
    cc.cc_dequant(t, dev.ctypes.data, nrows, ncols, got.ctypes.data)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("ncols", [256, 2816, 11008])
def test_chunk_column_cover(cc, t, ncols):
    assert cc.cc_cover(t, ncols) == ncols


@pytest.mark.parametrize("t", TYPES)
def test_chunk_dots_sum_to_gemv(cc, oracle_lib, t):
    nrows, ncols = 9, 1280
    x = synth.normal(50 + t, nrows * ncols, 0.02).reshape(nrows, ncols)
    raw = synth.quantize(t, x)
    w = np.empty(nrows * ncols, np.float32)
    oracle_lib.slo_dequantize(t, raw.ctypes.data, nrows * ncols, w.ctypes.data)
    v = synth.normal(99, ncols, 1.0)
    ref = w.reshape(nrows, ncols).astype(np.float64) @ v.astype(np.float64)
    dev = repack(cc, t, raw, nrows, ncols)
    got = np.empty(nrows, np.float32)
    assert cc.cc_gemv(t, dev.ctypes.data, nrows, ncols, v.ctypes.data, got.ctypes.data) == 0
    scale = np.abs(w.reshape(nrows, ncols)).astype(np.float64) @ np.abs(v).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 2e-5 * scale), np.abs(got - ref) / scale


def test_f16_codec_host_side(cc):
    u = np.arange(65536, dtype=np.uint16)
    ref = u.view(np.float16).astype(np.float32)
    got = np.array([cc.cc_decode_f16(int(h)) for h in u[::7]], np.float32)
    r = ref[::7]
    nan = np.isnan(r)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(got[~nan].view(np.uint32), r[~nan].view(np.uint32))
    vals = np.random.Generator(np.random.PCG64(3)).normal(0, 1, 5000).astype(np.float32)
    enc = np.array([cc.cc_encode_f16(float(v)) for v in vals], np.uint16)
    assert np.array_equal(enc, vals.astype(np.float16).view(np.uint16))


TILED = [2, 8, 12, 13, 14]


@pytest.mark.parametrize("t", TILED)
@pytest.mark.parametrize("shape", [(5, 256), (70, 768), (33, 1024), (19, 2560), (40, 5632)])
def test_tiled_layout_dequant_bit_exact_and_dot(cc, oracle_lib, t, shape):
    """Tiled (row-per-lane) device layout: repack + element dequantisation reproduce the oracle bit for
    bit for every tile geometry (KQ = 1, 2, 4, with and without column padding), and the per-lane block
    dot products add up to W.x."""
    nrows, ncols = shape
    x = synth.normal(60 + t, nrows * ncols, 0.02).reshape(nrows, ncols)
    raw = synth.quantize(t, x)
    ref = np.empty(nrows * ncols, np.float32)
    oracle_lib.slo_dequantize(t, raw.ctypes.data, nrows * ncols, ref.ctypes.data)
    dev = np.zeros(cc.cc_tiled_bytes(t, nrows, ncols), np.uint8)
    cc.cc_tiled_repack(t, raw.ctypes.data, nrows, ncols, dev.ctypes.data)
    got = np.empty(nrows * ncols, np.float32)
    cc.cc_tiled_dequant(t, dev.ctypes.data, nrows, ncols, got.ctypes.data)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    v = synth.normal(98, ncols, 1.0)
    w = ref.reshape(nrows, ncols)
    out = np.empty(nrows, np.float32)
    assert cc.cc_tiled_gemv(t, dev.ctypes.data, nrows, ncols, v.ctypes.data, out.ctypes.data) == 0
    scale = np.abs(w).astype(np.float64) @ np.abs(v).astype(np.float64)
    assert np.all(np.abs(out - w.astype(np.float64) @ v.astype(np.float64)) <= 2e-5 * scale)


def test_tiled_geometry_choices(cc):
    assert cc.cc_tiled_rows_log2(12, 4096, 4096) == 4      # 16 cblocks -> 16 rows x 4
    assert cc.cc_tiled_rows_log2(12, 4096, 11008) == 4     # 43 cblocks -> padded to 44
    assert cc.cc_tiled_rows_log2(8, 768, 768) == 6         # 3 cblocks -> 64 rows x 1
    assert cc.cc_tiled_rows_log2(8, 768, 3072) == 4
    assert cc.cc_tiled_rows_log2(8, 64, 512) == 5
