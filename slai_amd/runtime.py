"""Python face of the C ABI: contexts, tensors, quantized matrices, the ``LlmContext`` op
facade and the Llama-2 / GPT-2 model handles.

Class and method names follow the reference's Rust API for this path
(crates/slai/src/context.rs ``LlmContext``, stensor ``GpuTensor`` / ``GpuTensorView``,
crates/slai/src/quantized_matrix.rs ``GpuQuantMatrix``, crates/slai/src/gguf.rs ``Gguf``,
crates/slai/src/models/llama2/transformer.rs ``Llama2``), so tests read like the reference's.
Everything executes in libslai_hip.so; nothing here computes.
"""
import ctypes as C

import numpy as np

from . import _ffi
from ._ffi import AttnParams, RmsNormConfig, RopeConfig, View

_NP = {_ffi.DT_F32: np.float32, _ffi.DT_F16: np.float16, _ffi.DT_U8: np.uint8, _ffi.DT_I32: np.int32}
STORAGE = _ffi.USAGE_STORAGE | _ffi.USAGE_COPY_DST | _ffi.USAGE_COPY_SRC


class SlaiError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("slai error %d: %s" % (code, msg))
        self.code = code


class Backend:
    """One device + stream (slang_hal ``Backend``) with its kernels loaded (``LlmOps::new``)."""

    def __init__(self, device=0):
        self.L = _ffi.lib()
        h = C.c_void_p()
        rc = self.L.slai_ctx_create(device, C.byref(h))
        if rc:
            raise SlaiError(rc, "slai_ctx_create failed (is a GPU visible?)")
        self.h = h

    def check(self, rc):
        if rc:
            raise SlaiError(rc, self.L.slai_last_error(self.h).decode())

    def synchronize(self):
        self.check(self.L.slai_synchronize(self.h))

    def graph_begin_capture(self):
        self.check(self.L.slai_graph_begin_capture(self.h))

    def graph_end_capture(self):
        g = C.c_void_p()
        self.check(self.L.slai_graph_end_capture(self.h, C.byref(g)))
        return g

    def graph_launch(self, g):
        self.check(self.L.slai_graph_launch(self.h, g))

    def graph_destroy(self, g):
        self.L.slai_graph_destroy(self.h, g)

    def timer_begin(self):
        self.check(self.L.slai_timer_begin(self.h))

    def timer_end(self):
        ms = C.c_float()
        self.check(self.L.slai_timer_end(self.h, C.byref(ms)))
        return ms.value

    def close(self):
        if self.h:
            self.L.slai_ctx_destroy(self.h)
            self.h = None


class GpuTensor:
    """stensor ``GpuTensor<T>``: an owned device buffer with a column-major [nrows, ncols] shape."""

    def __init__(self, backend, nrows, ncols=1, dtype=_ffi.DT_F32, usage=STORAGE, data=None):
        self.b, self.nrows, self.ncols, self.dtype = backend, int(nrows), int(ncols), dtype
        esz = np.dtype(_NP[dtype]).itemsize
        self.nbytes = self.nrows * self.ncols * esz
        h = C.c_void_p()
        backend.check(backend.L.slai_buffer_create(backend.h, self.nbytes, dtype, usage, C.byref(h)))
        self.h = h
        if data is not None:
            self.write(data)

    @classmethod
    def vector(cls, backend, data, usage=STORAGE):
        data = np.ascontiguousarray(data, dtype=np.float32)
        return cls(backend, data.size, 1, _ffi.DT_F32, usage, data)

    @classmethod
    def matrix(cls, backend, data, usage=STORAGE):
        """data: numpy [nrows, ncols]; stored column-major like stensor's default ordering."""
        data = np.asarray(data, dtype=np.float32)
        return cls(backend, data.shape[0], data.shape[1], _ffi.DT_F32, usage, np.asfortranarray(data).T.copy())

    @classmethod
    def scalar(cls, backend, struct, usage=_ffi.USAGE_UNIFORM | _ffi.USAGE_COPY_DST):
        raw = np.frombuffer(bytes(struct), dtype=np.uint8)
        return cls(backend, raw.size, 1, _ffi.DT_U8, usage, raw)

    def write(self, data, offset_bytes=0):
        data = np.ascontiguousarray(data)
        self.b.check(self.b.L.slai_write_buffer(self.b.h, self.h, offset_bytes, data.ctypes.data, data.nbytes))

    def write_struct(self, struct):
        raw = np.frombuffer(bytes(struct), dtype=np.uint8)
        self.write(raw)

    def read(self):
        out = np.empty(self.nrows * self.ncols, dtype=_NP[self.dtype])
        self.b.check(self.b.L.slai_read_buffer(self.b.h, self.h, 0, out.ctypes.data, out.nbytes))
        return out

    def read_matrix(self):
        return self.read().reshape(self.ncols, self.nrows).T

    def view(self, offset=0, size=None, stride=None):
        n, m = self.nrows, self.ncols
        size = size or (n, m, 1, 1)
        stride = stride or (1, n, n * m, n * m)
        size = tuple(size) + (1,) * (4 - len(size))
        stride = tuple(stride) + (stride[-1],) * (4 - len(stride))
        return View(self.h, offset, (C.c_uint32 * 4)(*size), (C.c_uint32 * 4)(*stride))

    def as_view(self):
        return self.view()

    def column(self, i):
        return self.view(i * self.nrows, (self.nrows, 1, 1, 1), (1, self.nrows, self.nrows, self.nrows))

    def rows(self, start, n):
        return self.view(start, (n, 1, 1, 1), (1, n, n, n))

    def destroy(self):
        if self.h:
            self.b.L.slai_buffer_destroy(self.b.h, self.h)
            self.h = None


def _v(t):
    return t if isinstance(t, View) else t.as_view()


class GpuQuantMatrix:
    """crates/slai/src/quantized_matrix.rs ``GpuQuantMatrix``: packed GGUF rows resident on the device."""

    def __init__(self, backend, ggml_type, nrows, ncols, packed, layout=_ffi.LAYOUT_AUTO):
        self.b = backend
        packed = np.ascontiguousarray(packed).view(np.uint8).reshape(-1)
        h = C.c_void_p()
        backend.check(backend.L.slai_qmat_create_layout(backend.h, ggml_type, nrows, ncols, packed.ctypes.data, layout, C.byref(h)))
        self.h, self.ggml_type, self.nrows, self.ncols = h, ggml_type, nrows, ncols

    def shape(self):
        r, c, t = C.c_uint32(), C.c_uint32(), C.c_uint32()
        self.b.check(self.b.L.slai_qmat_shape(self.h, C.byref(r), C.byref(c), C.byref(t)))
        return r.value, c.value, t.value

    def device_bytes(self):
        return self.b.L.slai_qmat_device_bytes(self.h)

    def dequantize(self, row0=0, nrows=None):
        """``GgufTensorData::dequantize`` evaluated on the device; returns numpy [nrows, ncols]."""
        nrows = self.nrows - row0 if nrows is None else nrows
        out = GpuTensor(self.b, nrows * self.ncols)
        v = out.view(0, (nrows, self.ncols, 1, 1), (self.ncols, 1, nrows * self.ncols, nrows * self.ncols))
        self.b.check(self.b.L.slai_qmat_dequantize(self.b.h, self.h, row0, nrows, v))
        res = out.read().reshape(nrows, self.ncols)
        out.destroy()
        return res

    def destroy(self):
        if self.h:
            self.b.L.slai_qmat_destroy(self.b.h, self.h)
            self.h = None


class TensorCache:
    """crates/slai/src/tensor_cache.rs ``TensorCache``: idle temporaries keyed by element type, shape and usage."""

    def __init__(self, backend):
        self.b = backend
        h = C.c_void_p()
        backend.check(backend.L.slai_tensor_cache_create(backend.h, C.byref(h)))
        self.h = h

    def get_or_insert(self, nrows, ncols=1, dtype=_ffi.DT_F32, usage=STORAGE):
        """An idle tensor of this shape (contents as its last holder left them) or a new zero-filled one."""
        shape = (C.c_uint32 * 4)(int(nrows), int(ncols), 1, 1)
        h = C.c_void_p()
        self.b.check(self.b.L.slai_tensor_cache_get_or_insert(self.b.h, self.h, dtype, C.byref(shape), usage, C.byref(h)))
        t = GpuTensor.__new__(GpuTensor)
        t.b, t.nrows, t.ncols, t.dtype, t.h = self.b, int(nrows), int(ncols), dtype, h
        t.nbytes = t.nrows * t.ncols * np.dtype(_NP[dtype]).itemsize
        return t

    def reclaim(self, tensor):
        """What dropping a ``CachedTensor`` does: the tensor goes back into the pool; the handle must not be used after."""
        self.b.check(self.b.L.slai_tensor_cache_reclaim(self.b.h, self.h, tensor.h))
        tensor.h = None

    def clear(self):
        self.b.check(self.b.L.slai_tensor_cache_clear(self.b.h, self.h))

    def idle(self):
        return int(self.b.L.slai_tensor_cache_idle(self.h))

    def destroy(self):
        if self.h:
            self.b.L.slai_tensor_cache_destroy(self.b.h, self.h)
            self.h = None


class LlmContext:
    """crates/slai/src/context.rs ``LlmContext``: same method names and argument order (out first)."""

    def __init__(self, backend):
        self.backend = backend
        self.L, self.h = backend.L, backend.h

    def begin_submission(self):
        self.backend.check(self.L.slai_begin_submission(self.h))

    def submit(self):
        self.backend.check(self.L.slai_submit(self.h))

    def rms_norm_assign(self, config, out, value, weight):
        self.backend.check(self.L.slai_rms_norm_assign(self.h, config.h, _v(out), _v(value), _v(weight)))

    def layernorm_assign(self, out, value, eps=1e-5):
        self.backend.check(self.L.slai_layernorm_assign(self.h, _v(out), _v(value), eps))

    def matmul_quant_assign(self, out, a, b):
        self.backend.check(self.L.slai_matmul_quant_assign(self.h, _v(out), a.h, _v(b)))

    # fused forms (one kernel each) of the call sequences Llama2::launch issues
    def rms_norm_matmul_quant_assign(self, out, m, x, norm_weight, eps):
        self.backend.check(self.L.slai_rms_norm_matmul_quant_assign(self.h, _v(out), m.h, _v(x), _v(norm_weight), eps))

    def ffn_gate_up_silu(self, out_hb, gate, up, x, norm_weight, eps):
        self.backend.check(self.L.slai_ffn_gate_up_silu(self.h, _v(out_hb), gate.h, up.h, _v(x), _v(norm_weight), eps))

    def matmul_quant_add_assign(self, in_out_x, m, v):
        self.backend.check(self.L.slai_matmul_quant_add_assign(self.h, _v(in_out_x), m.h, _v(v)))

    def matmul_quant_columns(self, out, m, x, accumulate=False):
        """out[:, t] (+)= m * x[:, t] for up to 32 columns, on the matrix cores (tiled layouts only)."""
        self.backend.check(self.L.slai_matmul_quant_columns(self.h, _v(out), m.h, _v(x), 1 if accumulate else 0))

    def matmul_quant_assign_prepared(self, out, m, prepared):
        self.backend.check(self.L.slai_matmul_quant_assign_prepared(self.h, _v(out), m.h, _v(prepared)))

    def rms_norm_prepare(self, out_prepared, x, norm_weight):
        self.backend.check(self.L.slai_rms_norm_prepare(self.h, _v(out_prepared), _v(x), _v(norm_weight)))

    def rms_norm_matmul_quant_assign_prepared(self, out, m, x, prepared, eps):
        self.backend.check(self.L.slai_rms_norm_matmul_quant_assign_prepared(self.h, _v(out), m.h, _v(x), _v(prepared), eps))

    def ffn_gate_up_silu_prepared(self, out_hb, gate, up, x, prepared, eps):
        self.backend.check(self.L.slai_ffn_gate_up_silu_prepared(self.h, _v(out_hb), gate.h, up.h, _v(x), _v(prepared), eps))

    def matmul_quant_add_assign_emit(self, in_out_x, m, v, next_norm_weight, out_prepared):
        self.backend.check(self.L.slai_matmul_quant_add_assign_emit(self.h, _v(in_out_x), m.h, _v(v), _v(next_norm_weight), _v(out_prepared)))

    def matmul_assign(self, out, a, b, a_mode, b_mode):
        self.backend.check(self.L.slai_matmul_assign(self.h, _v(out), _v(a), _v(b), a_mode, b_mode))

    def add_assign(self, in_out_a, b):
        self.backend.check(self.L.slai_add_assign(self.h, _v(in_out_a), _v(b)))

    def mul_assign(self, in_out_a, b):
        self.backend.check(self.L.slai_mul_assign(self.h, _v(in_out_a), _v(b)))

    def copy(self, in_, out):
        self.backend.check(self.L.slai_copy(self.h, _v(in_), _v(out)))

    def rope(self, variant, config, in_out_q, in_out_k):
        self.backend.check(self.L.slai_rope(self.h, variant, config.h, _v(in_out_q), _v(in_out_k)))

    def silu(self, in_out_h1, in_h2):
        self.backend.check(self.L.slai_silu(self.h, _v(in_out_h1), _v(in_h2)))

    def gelu_inplace(self, x):
        self.backend.check(self.L.slai_gelu_inplace(self.h, _v(x)))

    def attn_mask(self, params, params_gpu, attn):
        self.backend.check(self.L.slai_attn_mask(self.h, C.byref(params), params_gpu.h, attn.h))

    def softmax_cols(self, in_out_mat):
        self.backend.check(self.L.slai_softmax_cols(self.h, _v(in_out_mat)))

    def attention(self, params, params_gpu, q, key_cache, value_cache, att, xb):
        """``BatchedMultiqueryAttention::launch`` (ops/batched_multiquery_attention.rs:32-100)."""
        self.backend.check(self.L.slai_attention(self.h, C.byref(params), params_gpu.h, _v(q), _v(key_cache), _v(value_cache),
                                                 _v(att), _v(xb)))

    def attention_static(self, params, params_gpu, q, key_cache, value_cache, att, xb):
        """``attention`` with the split partials in the library's static device array: allocates nothing."""
        self.backend.check(self.L.slai_attention_static(self.h, C.byref(params), params_gpu.h, _v(q), _v(key_cache), _v(value_cache),
                                                        _v(att), _v(xb)))

    def argmax(self, logits, out_index):
        self.backend.check(self.L.slai_argmax(self.h, _v(logits), out_index.h))

    def sample(self, logits, temperature, topp, coin, out_index):
        """models/sampler.rs:33-53 ``Sampler::sample`` with the draw `coin` in [0, 1) passed in."""
        self.backend.check(self.L.slai_sample(self.h, _v(logits), temperature, topp, coin, out_index.h))


def sampler_coin(seed, pos):
    """The draw the device-side sampling loops use at position `pos`."""
    return float(_ffi.lib().slai_sampler_coin(seed, pos))


class Gguf:
    """crates/slai/src/gguf.rs ``Gguf::from_bytes``; keeps the bytes alive for the handle."""

    def __init__(self, data):
        self.L = _ffi.lib()
        self.data = np.ascontiguousarray(data, dtype=np.uint8)
        h = C.c_void_p()
        err = C.create_string_buffer(512)
        rc = self.L.slai_gguf_parse(self.data.ctypes.data, self.data.size, C.byref(h), err, 512)
        if rc:
            raise SlaiError(rc, err.value.decode(errors="replace"))
        self.h = h

    @classmethod
    def open(cls, path):
        """Maps the file read-only (crates/slai-chat/src/cli.rs:43-57); the handle owns the mapping."""
        self = cls.__new__(cls)
        self.L = _ffi.lib()
        self.data = None
        h = C.c_void_p()
        err = C.create_string_buffer(512)
        rc = self.L.slai_gguf_open_file(str(path).encode(), C.byref(h), err, 512)
        if rc:
            raise SlaiError(rc, err.value.decode(errors="replace"))
        self.h = h
        return self

    @property
    def version(self):
        return self.L.slai_gguf_version(self.h)

    def metadata_debug_strings(self):
        """gguf.rs:686-695."""
        out = []
        for i in range(self.L.slai_gguf_metadata_count(self.h)):
            buf = C.create_string_buffer(512)
            if self.L.slai_gguf_meta_describe(self.h, i, buf, 512) == 0:
                out.append(buf.value.decode(errors="replace"))
        return out

    def meta_array_str(self, key):
        """gguf.rs:316-322 ``as_string_array`` (as bytes objects)."""
        n = self.meta_array_len(key)
        ptrs, lens, cnt = (C.c_void_p * max(n, 1))(), (C.c_uint64 * max(n, 1))(), C.c_uint64()
        rc = self.L.slai_gguf_meta_array_str(self.h, key.encode(), ptrs, lens, n, C.byref(cnt))
        if rc:
            raise SlaiError(rc, "metadata string array '%s'" % key)
        return [C.string_at(ptrs[i], lens[i]) if lens[i] else b"" for i in range(n)]

    def meta_array_f32(self, key):
        """gguf.rs:324-330 ``as_f32_array``."""
        n = self.meta_array_len(key)
        out, cnt = np.zeros(max(n, 1), dtype=np.float32), C.c_uint64()
        rc = self.L.slai_gguf_meta_array_f32(self.h, key.encode(), out.ctypes.data_as(C.POINTER(C.c_float)), n, C.byref(cnt))
        if rc:
            raise SlaiError(rc, "metadata f32 array '%s'" % key)
        return out[:n]

    def tensors(self):
        out = {}
        for i in range(self.L.slai_gguf_tensor_count(self.h)):
            name, dims, t, off = C.c_char_p(), (C.c_uint64 * 4)(), C.c_uint32(), C.c_uint64()
            self.L.slai_gguf_tensor_info(self.h, i, C.byref(name), C.byref(dims), C.byref(t), C.byref(off))
            out[name.value.decode(errors="replace")] = dict(dims=list(dims), type=t.value, offset=off.value)
        return out

    def meta_u32(self, key):
        v = C.c_uint32()
        rc = self.L.slai_gguf_meta_u32(self.h, key.encode(), C.byref(v))
        if rc:
            raise SlaiError(rc, "metadata u32 '%s'" % key)
        return v.value

    def meta_f32(self, key):
        v = C.c_float()
        rc = self.L.slai_gguf_meta_f32(self.h, key.encode(), C.byref(v))
        if rc:
            raise SlaiError(rc, "metadata f32 '%s'" % key)
        return v.value

    def meta_str(self, key):
        v = C.c_char_p()
        rc = self.L.slai_gguf_meta_str(self.h, key.encode(), C.byref(v))
        if rc:
            raise SlaiError(rc, "metadata string '%s'" % key)
        return v.value.decode()

    def meta_array_len(self, key):
        v = C.c_uint64()
        rc = self.L.slai_gguf_meta_array_len(self.h, key.encode(), C.byref(v))
        if rc:
            raise SlaiError(rc, "metadata array '%s'" % key)
        return v.value

    def to_gpu_matrix(self, backend, name):
        h = C.c_void_p()
        backend.check(self.L.slai_gguf_tensor_to_qmat(backend.h, self.h, name.encode(), C.byref(h)))
        m = GpuQuantMatrix.__new__(GpuQuantMatrix)
        m.b, m.h = backend, h
        m.nrows, m.ncols, m.ggml_type = m.shape()
        return m

    def check_llama2(self, model_type=_ffi.MODEL_LLAMA):
        """Host-only check of every tensor a Llama-2 / Qwen2 load would read; raises SlaiError on the first mismatch."""
        err = C.create_string_buffer(512)
        rc = self.L.slai_llama2_check_gguf(self.h, model_type, err, 512)
        if rc:
            raise SlaiError(rc, err.value.decode(errors="replace"))

    def check_gpt2(self):
        err = C.create_string_buffer(512)
        rc = self.L.slai_gpt2_check_gguf(self.h, err, 512)
        if rc:
            raise SlaiError(rc, err.value.decode(errors="replace"))

    def close(self):
        if self.h:
            self.L.slai_gguf_free(self.h)
            self.h = None


class Tokenizer:
    """``AnyTokenizer`` (crates/slai-chat/src/llm.rs:100-164): the Llama or GPT-2 tokenizer of a GGUF file."""

    def __init__(self, gguf, kind=_ffi.TOKENIZER_AUTO):
        self.L = _ffi.lib()
        h = C.c_void_p()
        err = C.create_string_buffer(512)
        rc = self.L.slai_tokenizer_from_gguf(gguf.h, kind, C.byref(h), err, 512)
        if rc:
            raise SlaiError(rc, err.value.decode(errors="replace"))
        self.h = h
        self.kind = self.L.slai_tokenizer_kind(h)
        self.bos, self.eos, self.unk = (self.L.slai_tokenizer_bos(h), self.L.slai_tokenizer_eos(h), self.L.slai_tokenizer_unk(h))
        self.vocab_size = self.L.slai_tokenizer_vocab_size(h)

    def _fail(self, rc):
        raise SlaiError(rc, (self.L.slai_tokenizer_last_error(self.h) or b"").decode(errors="replace"))

    def token_bytes(self, token):
        ptr, n = C.c_void_p(), C.c_size_t()
        rc = self.L.slai_tokenizer_token_str(self.h, token, C.byref(ptr), C.byref(n))
        if rc:
            raise SlaiError(rc, "token id outside the vocabulary")
        return C.string_at(ptr, n.value) if n.value else b""

    def bos_str(self):
        return self.token_bytes(self.bos).decode()

    def eos_str(self):
        return self.token_bytes(self.eos).decode()

    def encode(self, text, bos=False, eos=False):
        raw = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        cap = 4 * len(raw) + 8
        out, cnt = (C.c_int32 * cap)(), C.c_size_t()
        rc = self.L.slai_tokenizer_encode(self.h, raw, len(raw), int(bos), int(eos), out, cap, C.byref(cnt))
        if rc:
            self._fail(rc)
        return list(out[:cnt.value])

    def decode_bytes(self, tokens, prev_token=0):
        tokens = list(tokens)
        arr = (C.c_int32 * max(len(tokens), 1))(*tokens)
        n = C.c_size_t()
        cap = 64
        while True:
            buf = C.create_string_buffer(cap)
            rc = self.L.slai_tokenizer_decode(self.h, arr, len(tokens), prev_token, buf, cap, C.byref(n))
            if rc == _ffi.E_SHAPE and n.value > cap:
                cap = n.value
                continue
            if rc:
                self._fail(rc)
            return buf.raw[:n.value]

    def decode(self, tokens, prev_token=0):
        return self.decode_bytes(tokens, prev_token).decode("utf-8", errors="replace")

    def close(self):
        if self.h:
            self.L.slai_tokenizer_free(self.h)
            self.h = None


class Llama2:
    """``ChatLlama2`` without the tokenizer: config + weights + state + the per-token driver."""

    def __init__(self, backend, gguf, model_type=_ffi.MODEL_LLAMA, kv_dtype=_ffi.KV_F32):
        self.b = backend
        h = C.c_void_p()
        backend.check(backend.L.slai_llama2_from_gguf(backend.h, gguf.h, model_type, kv_dtype, C.byref(h)))
        self.h = h
        cfg = _ffi.Llama2Config()
        backend.check(backend.L.slai_llama2_get_config(h, C.byref(cfg)))
        self.config = cfg

    def weight_bytes(self):
        return self.b.L.slai_llama2_weight_bytes(self.h)

    def forward_logits(self, pos, token, fused=True):
        out = np.empty(self.config.vocab_size, dtype=np.float32)
        self.b.check(self.b.L.slai_llama2_forward_logits(self.h, pos, token, 1 if fused else 0, out.ctypes.data))
        return out

    def generate(self, prompt, n_steps, start_pos=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(n_steps, dtype=np.int32)
        ms = C.c_float()
        self.b.check(self.b.L.slai_llama2_generate(self.h, prompt.ctypes.data, prompt.size, start_pos, n_steps, out.ctypes.data, C.byref(ms)))
        return out, ms.value

    def generate_sampled(self, prompt, n_steps, temperature, topp, seed, start_pos=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(n_steps, dtype=np.int32)
        ms = C.c_float()
        self.b.check(self.b.L.slai_llama2_generate_sampled(self.h, prompt.ctypes.data, prompt.size, start_pos, n_steps, temperature, topp,
                                                           seed, out.ctypes.data, C.byref(ms)))
        return out, ms.value

    def decode_form(self):
        """0: one launch per step of the layer loop, 1: the whole layer stack in one resident launch per token."""
        return int(self.b.L.slai_llama2_decode_form(self.h))

    def trace_token(self, pos, token):
        """In-kernel time stamps of one token through the resident launch: uint64 [workgroups, 16 * n_layers + 8], ticks of
        the 100 MHz clock (see slai_llama2_trace_token)."""
        grid, stride = C.c_uint32(), C.c_uint32()
        cap = 4096 * (16 * self.config.n_layers + 8)
        out = np.zeros(cap, dtype=np.uint64)
        self.b.check(self.b.L.slai_llama2_trace_token(self.h, pos, token, out.ctypes.data, cap, C.byref(grid), C.byref(stride)))
        return out[:grid.value * stride.value].reshape(grid.value, stride.value)

    def time_steps(self, pos, token, reps=8):
        """[(step name, microseconds per launch inside a token with an event after every launch, launches per token,
        microseconds per launch of the step alone)] of the launch-per-step form (see slai_llama2_time_steps)."""
        cap = 32
        names = C.create_string_buffer(4096)
        us = np.zeros(cap, np.float32)
        alone = np.zeros(cap, np.float32)
        per = np.zeros(cap, np.uint32)
        n = C.c_uint32()
        self.b.check(self.b.L.slai_llama2_time_steps(self.h, pos, token, reps, C.cast(names, C.c_void_p), 4096, us.ctypes.data, alone.ctypes.data,
                                                     per.ctypes.data, cap, C.byref(n)))
        labels = names.value.decode().split("\n")[:n.value]
        return [(labels[i], float(us[i]), int(per[i]), float(alone[i])) for i in range(n.value)]

    def prefill_path(self):
        """2: matrix-core GEMM, 1: per-token workgroups over shared weights, 0: the token-by-token loop."""
        return int(self.b.L.slai_llama2_prefill_supported(self.h))

    def prefill_fp32_repeats(self):
        """Prefill calls that were repeated with fp32 MFMA because an activation was beyond the f16 range."""
        return int(self.b.L.slai_llama2_prefill_fp32_repeats(self.h))

    def prefill(self, tokens, start_pos=0, chunk=0):
        """Fill the caches for positions start_pos .. start_pos+len(tokens)-1, `chunk` tokens per pass over the
        weights (0 = the library's default); returns the stream time in ms."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        ms = C.c_float()
        self.b.check(self.b.L.slai_llama2_prefill(self.h, tokens.ctypes.data, tokens.size, start_pos, chunk, C.byref(ms)))
        return ms.value

    def kv_buffers(self, layer):
        k, v = C.c_void_p(), C.c_void_p()
        self.b.check(self.b.L.slai_llama2_kv_buffers(self.h, layer, C.byref(k), C.byref(v)))
        return k, v

    def write_kv(self, layer, k, v):
        """Fills positions [0, n) of layer `layer`'s caches from [n, kv_dim] arrays (cache dtype)."""
        kb, vb = self.kv_buffers(layer)
        for buf, arr in ((kb, k), (vb, v)):
            arr = np.ascontiguousarray(arr)
            self.b.check(self.b.L.slai_write_buffer(self.b.h, buf, 0, arr.ctypes.data, arr.nbytes))

    def destroy(self):
        if self.h:
            self.b.L.slai_llama2_destroy(self.h)
            self.h = None


class Gpt2:
    def __init__(self, backend, gguf, kv_dtype=_ffi.KV_F32):
        self.b = backend
        h = C.c_void_p()
        backend.check(backend.L.slai_gpt2_from_gguf(backend.h, gguf.h, kv_dtype, C.byref(h)))
        self.h = h
        p = _ffi.Gpt2Params()
        backend.check(backend.L.slai_gpt2_get_params(h, C.byref(p)))
        self.params = p

    def weight_bytes(self):
        return self.b.L.slai_gpt2_weight_bytes(self.h)

    def forward_logits(self, pos, token):
        out = np.empty(self.params.n_vocab, dtype=np.float32)
        self.b.check(self.b.L.slai_gpt2_forward_logits(self.h, pos, token, out.ctypes.data))
        return out

    def generate(self, prompt, n_steps, start_pos=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(n_steps, dtype=np.int32)
        ms = C.c_float()
        self.b.check(self.b.L.slai_gpt2_generate(self.h, prompt.ctypes.data, prompt.size, start_pos, n_steps, out.ctypes.data, C.byref(ms)))
        return out, ms.value

    def generate_sampled(self, prompt, n_steps, temperature, topp, seed, start_pos=0):
        prompt = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.zeros(n_steps, dtype=np.int32)
        ms = C.c_float()
        self.b.check(self.b.L.slai_gpt2_generate_sampled(self.h, prompt.ctypes.data, prompt.size, start_pos, n_steps, temperature, topp,
                                                         seed, out.ctypes.data, C.byref(ms)))
        return out, ms.value

    def prefill_path(self):
        """2: matrix-core GEMM, 0: the token-by-token loop."""
        return int(self.b.L.slai_gpt2_prefill_supported(self.h))

    def prefill_fp32_repeats(self):
        """Prefill calls that were repeated with fp32 MFMA because an activation was beyond the f16 range."""
        return int(self.b.L.slai_gpt2_prefill_fp32_repeats(self.h))

    def prefill(self, tokens, start_pos=0, chunk=0):
        """Fill the caches for positions start_pos .. start_pos+len(tokens)-1; returns the stream time in ms."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        ms = C.c_float()
        self.b.check(self.b.L.slai_gpt2_prefill(self.h, tokens.ctypes.data, tokens.size, start_pos, chunk, C.byref(ms)))
        return ms.value

    def destroy(self):
        if self.h:
            self.b.L.slai_gpt2_destroy(self.h)
            self.h = None
