"""ctypes binding of lib/libslai_hip.so (the C ABI declared in include/slai_hip.h).

The library is loaded lazily and must already be built (``slai_amd.build.build_hip()`` or
``__graft_entry__.build()``); there is no CPU fallback -- a missing library is an error.
"""
import ctypes as C
import os

from . import build as _build

OK, E_HIP, E_SHAPE, E_TYPE, E_ARG, E_PARSE, E_MISSING, E_STATE, E_IO = 0, -1, -2, -3, -4, -5, -6, -7, -8
TOKENIZER_AUTO, TOKENIZER_LLAMA, TOKENIZER_GPT2 = -1, 0, 1
DT_F32, DT_F16, DT_U8, DT_I32 = 0, 1, 2, 3
USAGE_MAP_READ, USAGE_COPY_SRC, USAGE_COPY_DST, USAGE_UNIFORM, USAGE_STORAGE = 0x1, 0x4, 0x8, 0x40, 0x80
ROPE_ORIGINAL, ROPE_NEOX = 0, 1
MODE_N, MODE_T = 0, 1
MODEL_LLAMA, MODEL_QWEN2 = 0, 1
KV_F32, KV_F16 = 0, 1
LAYOUT_AUTO, LAYOUT_ROWS, LAYOUT_TILE16, LAYOUT_TILE64 = 0, 1, 2, 3


class View(C.Structure):
    _fields_ = [("buf", C.c_void_p), ("offset", C.c_uint64), ("size", C.c_uint32 * 4), ("stride", C.c_uint32 * 4)]


class RmsNormConfig(C.Structure):
    _fields_ = [("nudge_factor", C.c_float), ("_padding", C.c_uint32 * 3)]


class RopeConfig(C.Structure):
    _fields_ = [("head_size", C.c_uint32), ("kv_dim", C.c_uint32), ("pos", C.c_uint32), ("base_freq", C.c_float)]


class AttnParams(C.Structure):
    _fields_ = [("seq_len", C.c_uint32), ("kv_dim", C.c_uint32), ("kv_mul", C.c_uint32), ("n_heads", C.c_uint32),
                ("head_size", C.c_uint32), ("pos", C.c_uint32), ("_padding", C.c_uint32 * 2)]


class Llama2Config(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("dim", "hidden_dim", "n_layers", "n_q_heads", "n_kv_heads", "vocab_size", "seq_len")] + \
               [("rope_base_freq", C.c_float), ("rms_norm_eps", C.c_float)]


class Gpt2Params(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("n_vocab", "n_seq", "n_embd", "n_head", "n_layer", "ff_len", "attn_b")]


vp, sz, u32, u64, i32 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64, C.c_int
P = C.POINTER

# name -> (restype, argtypes); every symbol include/slai_hip.h declares
SIGNATURES = {
    "slai_ctx_create": (i32, [i32, P(vp)]),
    "slai_ctx_destroy": (None, [vp]),
    "slai_last_error": (C.c_char_p, [vp]),
    "slai_ctx_stream": (vp, [vp]),
    "slai_begin_submission": (i32, [vp]),
    "slai_submit": (i32, [vp]),
    "slai_synchronize": (i32, [vp]),
    "slai_buffer_create": (i32, [vp, sz, i32, u32, P(vp)]),
    "slai_buffer_destroy": (None, [vp, vp]),
    "slai_buffer_size": (sz, [vp]),
    "slai_buffer_device_ptr": (vp, [vp]),
    "slai_write_buffer": (i32, [vp, vp, sz, vp, sz]),
    "slai_read_buffer": (i32, [vp, vp, sz, vp, sz]),
    "slai_copy_buffer": (i32, [vp, vp, sz, vp, sz, sz]),
    "slai_qmat_create": (i32, [vp, u32, u32, u32, vp, P(vp)]),
    "slai_qmat_create_layout": (i32, [vp, u32, u32, u32, vp, i32, P(vp)]),
    "slai_qmat_destroy": (None, [vp, vp]),
    "slai_qmat_shape": (i32, [vp, P(u32), P(u32), P(u32)]),
    "slai_qmat_device_bytes": (sz, [vp]),
    "slai_qmat_dequantize": (i32, [vp, vp, u32, u32, View]),
    "slai_rms_norm_assign": (i32, [vp, vp, View, View, View]),
    "slai_layernorm_assign": (i32, [vp, View, View, C.c_float]),
    "slai_matmul_quant_assign": (i32, [vp, View, vp, View]),
    "slai_matmul_assign": (i32, [vp, View, View, View, i32, i32]),
    "slai_rms_norm_matmul_quant_assign": (i32, [vp, View, vp, View, View, C.c_float]),
    "slai_ffn_gate_up_silu": (i32, [vp, View, vp, vp, View, View, C.c_float]),
    "slai_matmul_quant_add_assign": (i32, [vp, View, vp, View]),
    "slai_rms_norm_prepare": (i32, [vp, View, View, View]),
    "slai_matmul_quant_columns": (i32, [vp, View, vp, View, C.c_int]),
    "slai_matmul_quant_assign_prepared": (i32, [vp, View, vp, View]),
    "slai_rms_norm_matmul_quant_assign_prepared": (i32, [vp, View, vp, View, View, C.c_float]),
    "slai_ffn_gate_up_silu_prepared": (i32, [vp, View, vp, vp, View, View, C.c_float]),
    "slai_matmul_quant_add_assign_emit": (i32, [vp, View, vp, View, View, View]),
    "slai_add_assign": (i32, [vp, View, View]),
    "slai_mul_assign": (i32, [vp, View, View]),
    "slai_copy": (i32, [vp, View, View]),
    "slai_rope": (i32, [vp, i32, vp, View, View]),
    "slai_silu": (i32, [vp, View, View]),
    "slai_gelu_inplace": (i32, [vp, View]),
    "slai_attn_mask": (i32, [vp, P(AttnParams), vp, vp]),
    "slai_softmax_cols": (i32, [vp, View]),
    "slai_attention": (i32, [vp, P(AttnParams), vp, View, View, View, View, View]),
    "slai_attention_static": (i32, [vp, P(AttnParams), vp, View, View, View, View, View]),
    "slai_argmax": (i32, [vp, View, vp]),
    "slai_sample": (i32, [vp, View, C.c_float, C.c_float, C.c_float, vp]),
    "slai_sampler_coin": (C.c_float, [u64, u32]),
    "slai_tensor_cache_create": (i32, [vp, P(vp)]),
    "slai_tensor_cache_destroy": (None, [vp, vp]),
    "slai_tensor_cache_get_or_insert": (i32, [vp, vp, i32, P(u32 * 4), u32, P(vp)]),
    "slai_tensor_cache_reclaim": (i32, [vp, vp, vp]),
    "slai_tensor_cache_clear": (i32, [vp, vp]),
    "slai_tensor_cache_idle": (sz, [vp]),
    "slai_timer_begin": (i32, [vp]),
    "slai_timer_end": (i32, [vp, P(C.c_float)]),
    "slai_graph_begin_capture": (i32, [vp]),
    "slai_graph_end_capture": (i32, [vp, P(vp)]),
    "slai_graph_launch": (i32, [vp, vp]),
    "slai_graph_destroy": (None, [vp, vp]),
    "slai_gguf_parse": (i32, [vp, sz, P(vp), C.c_char_p, sz]),
    "slai_gguf_free": (None, [vp]),
    "slai_gguf_version": (u32, [vp]),
    "slai_gguf_tensor_count": (u64, [vp]),
    "slai_gguf_metadata_count": (u64, [vp]),
    "slai_gguf_data_start": (u64, [vp]),
    "slai_gguf_tensor_info": (i32, [vp, u64, P(C.c_char_p), P(u64 * 4), P(u32), P(u64)]),
    "slai_gguf_find_tensor": (i32, [vp, C.c_char_p, P(u64)]),
    "slai_gguf_meta_u32": (i32, [vp, C.c_char_p, P(u32)]),
    "slai_gguf_meta_f32": (i32, [vp, C.c_char_p, P(C.c_float)]),
    "slai_gguf_meta_str": (i32, [vp, C.c_char_p, P(C.c_char_p)]),
    "slai_gguf_meta_array_len": (i32, [vp, C.c_char_p, P(u64)]),
    "slai_gguf_meta_describe": (i32, [vp, u64, C.c_char_p, sz]),
    "slai_gguf_open_file": (i32, [C.c_char_p, P(vp), C.c_char_p, sz]),
    "slai_gguf_meta_array_str": (i32, [vp, C.c_char_p, P(vp), P(u64), u64, P(u64)]),
    "slai_gguf_meta_array_f32": (i32, [vp, C.c_char_p, P(C.c_float), u64, P(u64)]),
    "slai_tokenizer_from_gguf": (i32, [vp, i32, P(vp), C.c_char_p, sz]),
    "slai_tokenizer_free": (None, [vp]),
    "slai_tokenizer_kind": (i32, [vp]),
    "slai_tokenizer_bos": (u32, [vp]),
    "slai_tokenizer_eos": (u32, [vp]),
    "slai_tokenizer_unk": (u32, [vp]),
    "slai_tokenizer_vocab_size": (u32, [vp]),
    "slai_tokenizer_last_error": (C.c_char_p, [vp]),
    "slai_tokenizer_token_str": (i32, [vp, u32, P(vp), P(sz)]),
    "slai_tokenizer_encode": (i32, [vp, C.c_char_p, sz, i32, i32, P(C.c_int32), sz, P(sz)]),
    "slai_tokenizer_decode": (i32, [vp, P(C.c_int32), sz, C.c_int32, C.c_char_p, sz, P(sz)]),
    "slai_gguf_tensor_to_qmat": (i32, [vp, vp, C.c_char_p, P(vp)]),
    "slai_gguf_tensor_to_qmat_layout": (i32, [vp, vp, C.c_char_p, i32, P(vp)]),
    "slai_llama2_from_gguf": (i32, [vp, vp, i32, i32, P(vp)]),
    "slai_llama2_check_gguf": (i32, [vp, i32, C.c_char_p, sz]),
    "slai_gpt2_check_gguf": (i32, [vp, C.c_char_p, sz]),
    "slai_llama2_decode_form": (i32, [vp]),
    "slai_llama2_trace_token": (i32, [vp, u32, u32, vp, sz, P(u32), P(u32)]),
    "slai_llama2_time_steps": (i32, [vp, u32, u32, u32, vp, sz, vp, vp, vp, u32, P(u32)]),
    "slai_llama2_destroy": (None, [vp]),
    "slai_llama2_get_config": (i32, [vp, P(Llama2Config)]),
    "slai_llama2_weight_bytes": (sz, [vp]),
    "slai_llama2_forward_logits": (i32, [vp, u32, u32, i32, vp]),
    "slai_llama2_generate": (i32, [vp, vp, u32, u32, u32, vp, P(C.c_float)]),
    "slai_llama2_generate_sampled": (i32, [vp, vp, u32, u32, u32, C.c_float, C.c_float, u64, vp, P(C.c_float)]),
    "slai_llama2_kv_buffers": (i32, [vp, u32, P(vp), P(vp)]),
    "slai_llama2_logits_buffer": (i32, [vp, P(vp)]),
    "slai_gpt2_from_gguf": (i32, [vp, vp, i32, P(vp)]),
    "slai_gpt2_destroy": (None, [vp]),
    "slai_gpt2_get_params": (i32, [vp, P(Gpt2Params)]),
    "slai_gpt2_weight_bytes": (sz, [vp]),
    "slai_gpt2_forward_logits": (i32, [vp, u32, u32, vp]),
    "slai_gpt2_generate": (i32, [vp, vp, u32, u32, u32, vp, P(C.c_float)]),
    "slai_llama2_prefill": (i32, [vp, vp, u32, u32, u32, P(C.c_float)]),
    "slai_llama2_prefill_supported": (i32, [vp]),
    "slai_llama2_prefill_fp32_repeats": (C.c_uint32, [vp]),
    "slai_gpt2_prefill": (i32, [vp, vp, u32, u32, u32, P(C.c_float)]),
    "slai_gpt2_prefill_supported": (i32, [vp]),
    "slai_gpt2_prefill_fp32_repeats": (C.c_uint32, [vp]),
    "slai_gpt2_generate_sampled": (i32, [vp, vp, u32, u32, u32, C.c_float, C.c_float, u64, vp, P(C.c_float)]),
}

_lib = None


def lib():
    """Loads libslai_hip.so.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        path = _build.HIP_LIB
        if not os.path.exists(path):
            raise RuntimeError("%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` first "
                               "(the decode path has no CPU fallback)" % path)
        L = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib
