"""Shared test helpers: oracle-side GGUF access and structured block inputs."""
import ctypes as C
import os

import numpy as np

import oracle
from oracle import np_oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


class OracleGguf:
    """Parses a GGUF byte array with the C oracle and exposes numpy views."""

    def __init__(self, data):
        self.L = oracle.load()
        self.L.slo_set_threads(min(8, os.cpu_count() or 1))   # row-parallel GEMV: same bits, less waiting
        self.data = np.ascontiguousarray(data, dtype=np.uint8)
        err = C.c_int(0)
        self.h = self.L.slo_gguf_parse(self.data.ctypes.data, self.data.size, C.byref(err))
        self.err = err.value
        if not self.h:
            raise ValueError("gguf parse error %d" % self.err)
        L, h = self.L, self.h
        self.tensors = {}
        for i in range(L.slo_gguf_n_tensors(h)):
            name = L.slo_gguf_tensor_name(h, i).decode()
            dims = [L.slo_gguf_tensor_dim(h, i, d) for d in range(4)]
            self.tensors[name] = dict(index=i, dims=dims, type=L.slo_gguf_tensor_type(h, i),
                                      offset=L.slo_gguf_tensor_offset(h, i), ndims=L.slo_gguf_tensor_ndims(h, i))
        self.meta = {}
        for i in range(L.slo_gguf_n_meta(h)):
            key = L.slo_gguf_meta_key(h, i).decode()
            t = L.slo_gguf_meta_type(h, i)
            if t == 8:
                v = L.slo_gguf_meta_str(h, i).decode()
            elif t == 9:
                v = ("array", L.slo_gguf_meta_arr_type(h, i), L.slo_gguf_meta_arr_len(h, i), L.slo_gguf_meta_arr_offset(h, i))
            elif t in (6, 12):
                v = L.slo_gguf_meta_f64(h, i)
            elif t in (1, 3, 5, 11):
                v = L.slo_gguf_meta_i64(h, i)
            else:
                v = L.slo_gguf_meta_u64(h, i)
            self.meta[key] = (t, v)

    def raw(self, name):
        t = self.tensors[name]
        n = int(np.prod(t["dims"]))
        nbytes = n // self.L.slo_block_elems(t["type"]) * self.L.slo_block_bytes(t["type"])
        return self.data[t["offset"]:t["offset"] + nbytes]

    def dequantize(self, name):
        t = self.tensors[name]
        n = int(np.prod(t["dims"]))
        out = np.empty(n, dtype=np.float32)
        rc = self.L.slo_gguf_tensor_dequantize(self.h, t["index"], out.ctypes.data)
        assert rc == 0
        return out

    def np_tensors(self):
        """name -> f32 array shaped [nrows, ncols] (or [n]) via the independent numpy dequantizers."""
        out = {}
        for name, t in self.tensors.items():
            n = int(np.prod(t["dims"]))
            a = np_oracle.dequantize(t["type"], self.raw(name), n)
            nrows, ncols = t["dims"][0], t["dims"][1]
            out[name] = a.reshape(ncols) if t["ndims"] == 1 else a.reshape(nrows, ncols)
        return out

    def close(self):
        if self.h:
            self.L.slo_gguf_free(self.h)
            self.h = None


def f16_bits(x):
    return int(np.float16(x).view(np.uint16))


def structured_blocks(ggml_type, n=16):
    """The deterministic block contents of the reference's (uncompiled) dequantization test,
    crates/slai/src/ops/quantization.rs:77-220: scale 1.234 / 5.678, byte ramps.  Known inputs
    only -- that test compares against the CPU dequantizer at run time and holds no outputs."""
    s1, s2 = f16_bits(1.234), f16_bits(5.678)
    out = bytearray()
    for i in range(n):
        k32 = np.arange(32)
        if ggml_type == 8:
            data = ((i * 16 - 128 + k32 + 128) % 256 - 128).astype(np.int8)
            out += np.uint16(s1).tobytes() + data.tobytes()
        elif ggml_type == 2:
            qs = ((i * 16 + np.arange(16)) % 256).astype(np.uint8)
            out += np.uint16(s1).tobytes() + qs.tobytes()
        elif ggml_type == 3:
            qs = ((i * 16 + np.arange(16)) % 256).astype(np.uint8)
            out += np.uint16(s1).tobytes() + np.uint16(3).tobytes() + qs.tobytes()
        elif ggml_type == 6:
            qs = ((i * 16 + np.arange(16)) % 256).astype(np.uint8)
            out += np.uint16(s1).tobytes() + bytes([1, 100, 200, 250]) + qs.tobytes()
        elif ggml_type == 7:
            qs = ((i * 16 + np.arange(16)) % 256).astype(np.uint8)
            out += np.uint16(s1).tobytes() + np.uint16(125).tobytes() + bytes([1, 100, 200, 250]) + qs.tobytes()
        elif ggml_type == 15:
            qs = np.clip(i * 8 - 127 + np.arange(256), -128, 127).astype(np.int8)
            out += np.float32(1.234).tobytes() + qs.tobytes() + bytes(32)
        elif ggml_type in (12, 13):
            scales = ((i * 16 + np.arange(12)) % 256).astype(np.uint8)
            qs = np.minimum(i * 16 + np.arange(128), 255).astype(np.uint8)
            qh = np.minimum(i * 16 + np.arange(32), 255).astype(np.uint8)
            out += np.uint16(s1).tobytes() + np.uint16(s2).tobytes() + scales.tobytes()
            if ggml_type == 13:
                out += qh.tobytes()
            out += qs.tobytes()
        elif ggml_type == 14:
            scales = ((i * 8 - 127 + np.arange(16) + 128) % 256 - 128).astype(np.int8)
            ql = ((i * 8 + np.arange(128)) % 256).astype(np.uint8)
            qh = ((i * 8 + np.arange(64)) % 256).astype(np.uint8)
            out += ql.tobytes() + qh.tobytes() + scales.tobytes() + np.uint16(123).tobytes()
        else:
            raise ValueError(ggml_type)
    return np.frombuffer(bytes(out), dtype=np.uint8).copy()


def random_blocks(ggml_type, n_blocks, seed, finite_scales=True):
    """Uniformly random block bytes (the reference's `Standard` distribution over raw bits,
    crates/slai/src/ops/gemv_quant.rs:81-99), with f16/f32 scale fields forced finite and
    moderate when `finite_scales` so that values are comparable."""
    from slai_amd.synth import BLOCK_BYTES
    rng = np.random.Generator(np.random.PCG64(seed))
    bb = BLOCK_BYTES[ggml_type]
    raw = rng.integers(0, 256, (n_blocks, bb), dtype=np.uint8)
    if finite_scales:
        def put_f16(col):
            v = rng.uniform(-2.0, 2.0, n_blocks).astype(np.float16)
            raw[:, col:col + 2] = v.view(np.uint8).reshape(n_blocks, 2)
        if ggml_type in (2, 6, 8):
            put_f16(0)
        elif ggml_type in (3, 7, 12, 13):
            put_f16(0); put_f16(2)
        elif ggml_type == 14:
            put_f16(208)
        elif ggml_type == 15:
            raw[:, 0:4] = rng.uniform(-2, 2, n_blocks).astype(np.float32).view(np.uint8).reshape(n_blocks, 4)
        elif ggml_type == 1:
            v = rng.uniform(-2.0, 2.0, n_blocks).astype(np.float16)
            raw[:, 0:2] = v.view(np.uint8).reshape(n_blocks, 2)
        elif ggml_type == 0:
            raw[:, 0:4] = rng.uniform(-2, 2, n_blocks).astype(np.float32).view(np.uint8).reshape(n_blocks, 4)
    return raw.reshape(-1)
