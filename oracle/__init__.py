"""CPU oracle for the slai decode path -- TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this package.  The shipped library (``slai_amd``) never does.

``load()`` returns a ctypes handle on ``oracle/liboracle.so`` (the C restatement of
the reference's CPU path, see ``slai_oracle.c``); ``build()`` compiles it.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_lib = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        build()
    lib = C.CDLL(_LIB)
    u8p, f32p, i32p = C.POINTER(C.c_uint8), C.POINTER(C.c_float), C.POINTER(C.c_int)
    vp, sz = C.c_void_p, C.c_size_t
    sig = {
        "slo_set_threads": (None, [C.c_int]),
        "slo_get_threads": (C.c_int, []),
        "slo_decode_f16": (C.c_float, [C.c_uint16]),
        "slo_decode_f16_n": (None, [vp, sz, vp]),
        "slo_encode_f16": (C.c_uint16, [C.c_float]),
        "slo_block_elems": (C.c_int, [C.c_int]),
        "slo_block_bytes": (C.c_int, [C.c_int]),
        "slo_get_scale_min_k4": (None, [C.c_int, vp, vp, vp]),
        "slo_dequantize": (C.c_int, [C.c_int, vp, sz, vp]),
        "slo_dot": (C.c_float, [vp, vp, sz]),
        "slo_gemv": (None, [vp, vp, vp, sz, sz]),
        "slo_rms_norm": (None, [vp, vp, vp, sz, C.c_float]),
        "slo_softmax": (None, [vp, sz]),
        "slo_rope": (None, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int]),
        "slo_silu": (None, [vp, vp, sz]),
        "slo_layernorm": (None, [vp, vp, sz, C.c_float]),
        "slo_gelu": (C.c_float, [C.c_float]),
        "slo_gelu_n": (None, [vp, sz]),
        "slo_argmax": (C.c_int, [vp, sz]),
        "slo_attention": (None, [C.c_int] * 6 + [vp] * 5),
        "slo_gguf_parse": (vp, [vp, sz, i32p]),
        "slo_gguf_free": (None, [vp]),
        "slo_gguf_version": (C.c_uint32, [vp]),
        "slo_gguf_alignment": (C.c_uint32, [vp]),
        "slo_gguf_data_start": (C.c_uint64, [vp]),
        "slo_gguf_n_meta": (C.c_uint64, [vp]),
        "slo_gguf_n_tensors": (C.c_uint64, [vp]),
        "slo_gguf_meta_key": (C.c_char_p, [vp, C.c_uint64]),
        "slo_gguf_meta_type": (C.c_uint32, [vp, C.c_uint64]),
        "slo_gguf_meta_arr_type": (C.c_uint32, [vp, C.c_uint64]),
        "slo_gguf_meta_arr_len": (C.c_uint64, [vp, C.c_uint64]),
        "slo_gguf_meta_arr_offset": (C.c_uint64, [vp, C.c_uint64]),
        "slo_gguf_meta_u64": (C.c_uint64, [vp, C.c_uint64]),
        "slo_gguf_meta_i64": (C.c_int64, [vp, C.c_uint64]),
        "slo_gguf_meta_f64": (C.c_double, [vp, C.c_uint64]),
        "slo_gguf_meta_str": (C.c_char_p, [vp, C.c_uint64]),
        "slo_gguf_tensor_name": (C.c_char_p, [vp, C.c_uint64]),
        "slo_gguf_tensor_type": (C.c_uint32, [vp, C.c_uint64]),
        "slo_gguf_tensor_ndims": (C.c_uint32, [vp, C.c_uint64]),
        "slo_gguf_tensor_dim": (C.c_uint64, [vp, C.c_uint64, C.c_int]),
        "slo_gguf_tensor_offset": (C.c_uint64, [vp, C.c_uint64]),
        "slo_gguf_tensor_dequantize": (C.c_int, [vp, C.c_uint64, vp]),
        "slo_llama2_from_gguf": (vp, [vp, C.c_char_p, C.c_int, C.c_int, C.c_int]),
        "slo_llama2_free": (None, [vp]),
        "slo_llama2_forward": (None, [vp, C.c_int, C.c_int]),
        "slo_llama2_logits": (f32p, [vp]),
        "slo_llama2_x": (f32p, [vp]),
        "slo_llama2_config": (None, [vp, vp]),
        "slo_llama2_fill_kv": (None, [vp, sz, sz, vp, vp]),
        "slo_llama2_generate": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, vp]),
        "slo_gpt2_from_gguf": (vp, [vp, C.c_int]),
        "slo_gpt2_free": (None, [vp]),
        "slo_gpt2_forward": (None, [vp, C.c_int, C.c_int]),
        "slo_gpt2_logits": (f32p, [vp]),
        "slo_gpt2_config": (None, [vp, vp]),
        "slo_gpt2_generate": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
