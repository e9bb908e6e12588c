"""GGUF v3 writer and synthetic Llama-2 / GPT-2 model files.

The container layout is the one the loader reads (reference parser:
crates/slai/src/gguf.rs:504-679): magic, version, counts, metadata KVs, tensor infos
(name, ndims, dims with ne0 = ncols first, ggml type, offset), then aligned data.
Synthetic models follow the tensor names and metadata keys of
crates/slai/src/models/llama2/transformer.rs:208-219,270-272,
crates/slai/src/models/llama2/cpu.rs:79-109 and crates/slai/src/models/gpt2/cpu.rs:37-48,118-131.
"""
import struct

import numpy as np

from . import synth

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f",
        T_BOOL: "<B", T_U64: "<Q", T_I64: "<q", T_F64: "<d"}


def _str(s):
    b = s.encode("utf-8") if isinstance(s, str) else bytes(s)
    return struct.pack("<Q", len(b)) + b


class GgufWriter:
    def __init__(self, version=3, alignment=32):
        self.version = version
        self.alignment = alignment
        self.meta = []      # (key, type, payload-bytes)
        self.tensors = []   # (name, dims(ne order), ggml_type, data: np.uint8 array)
        self.tensor_hook = None   # optional f(name, ne_dims, ggml_type, data) -> (ne_dims, ggml_type, data) or None to drop

    def add_meta(self, key, vtype, value, elem_type=None):
        if vtype == T_STR:
            payload = _str(value)
        elif vtype == T_ARR:
            if elem_type == T_STR:
                body = b"".join(_str(v) for v in value)
            else:
                body = b"".join(struct.pack(_FMT[elem_type], v) for v in value)
            payload = struct.pack("<IQ", elem_type, len(value)) + body
        else:
            payload = struct.pack(_FMT[vtype], value)
        self.meta.append((key, vtype, payload))

    def add_tensor(self, name, ne_dims, ggml_type, data):
        """ne_dims: GGUF order (ne0 = ncols first).  data: bytes-like of packed blocks."""
        data = np.frombuffer(data, dtype=np.uint8) if not isinstance(data, np.ndarray) else data.view(np.uint8).reshape(-1)
        if self.tensor_hook is not None:
            r = self.tensor_hook(name, list(ne_dims), ggml_type, data)
            if r is None:
                return
            ne_dims, ggml_type, data = r
        self.tensors.append((name, list(ne_dims), ggml_type, data))

    def to_bytes(self):
        head = struct.pack("<IIQQ", 0x46554747, self.version, len(self.tensors), len(self.meta))
        parts = [head]
        for key, vtype, payload in self.meta:
            parts.append(_str(key) + struct.pack("<I", vtype) + payload)
        a = self.alignment
        offsets, off = [], 0
        for _, _, _, data in self.tensors:
            offsets.append(off)
            off += data.size
            off += (a - off % a) % a
        for (name, dims, t, _), o in zip(self.tensors, offsets):
            parts.append(_str(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
                         + struct.pack("<IQ", t, o))
        header = b"".join(parts)
        start = len(header) + (a - len(header) % a) % a
        out = np.zeros(start + off, dtype=np.uint8)
        out[:len(header)] = np.frombuffer(header, dtype=np.uint8)
        for (_, _, _, data), o in zip(self.tensors, offsets):
            out[start + o:start + o + data.size] = data
        return out


def add_tokenizer_meta(w, tok):
    """tokenizer.* keys read by crates/slai/src/models/{llama2,gpt2}/tokenizer.rs and slai-chat/src/{llm,chat_template}.rs."""
    w.add_meta("tokenizer.ggml.model", T_STR, tok["model"])
    w.add_meta("tokenizer.ggml.tokens", T_ARR, list(tok["tokens"]), elem_type=T_STR)
    if "scores" in tok:
        w.add_meta("tokenizer.ggml.scores", T_ARR, [float(x) for x in tok["scores"]], elem_type=T_F32)
    if "merges" in tok:
        w.add_meta("tokenizer.ggml.merges", T_ARR, list(tok["merges"]), elem_type=T_STR)
    w.add_meta("tokenizer.ggml.bos_token_id", T_U32, tok["bos"])
    w.add_meta("tokenizer.ggml.eos_token_id", T_U32, tok["eos"])
    if "unk" in tok:
        w.add_meta("tokenizer.ggml.unknown_token_id", T_U32, tok["unk"])
    if tok.get("chat_template"):
        w.add_meta("tokenizer.chat_template", T_STR, tok["chat_template"])


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint8).reshape(-1)


def llama_gguf(dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab, seq_len, wtype, seed=1234,
               std=0.02, rope_base=10000.0, rms_eps=1e-5, out_type=None, v_type=None, embd_type=None,
               with_output=True, arch="llama", bias=False, norm_random=False, distinct_layers=None, tokenizer=None,
               ffn_norm_scale=1.0, tensor_hook=None, tensor_types=None):
    """Synthetic Llama-2-shape model file (uint8 numpy array).

    Weights are seeded std*N(0,1) quantized to `wtype` (`v_type` for attn_v, `out_type` for
    output.weight, `embd_type` for token_embd); norm weights are 1.0 unless norm_random.
    `distinct_layers`: when set, only that many layers are generated from scratch and the
    others reuse their packed bytes with the rows rotated (still distinct memory and the same
    value distribution; used to bound set-up time of the largest benchmark model).
    `ffn_norm_scale`: factor on the ffn_norm weights (large values push the normalised rows beyond the f16 range).
    `tokenizer`: optional dict(model=, tokens=, scores=|merges=, bos=, eos=, unk=, chat_template=) written as the
    tokenizer.* metadata a chat front end reads; `vocab` must then equal len(tokens).
    `tensor_hook`: see GgufWriter.tensor_hook (tests use it to write malformed files).
    """
    out_type = wtype if out_type is None else out_type
    v_type = wtype if v_type is None else v_type
    embd_type = wtype if embd_type is None else embd_type
    kv_dim = dim * n_kv_heads // n_heads
    w = GgufWriter()
    w.tensor_hook = tensor_hook
    w.add_meta("general.architecture", T_STR, arch)
    w.add_meta("general.alignment", T_U32, 32)
    w.add_meta(arch + ".embedding_length", T_U32, dim)
    w.add_meta(arch + ".feed_forward_length", T_U32, hidden_dim)
    w.add_meta(arch + ".block_count", T_U32, n_layers)
    w.add_meta(arch + ".attention.head_count", T_U32, n_heads)
    w.add_meta(arch + ".attention.head_count_kv", T_U32, n_kv_heads)
    w.add_meta(arch + ".context_length", T_U32, seq_len)
    w.add_meta(arch + ".rope.freq_base", T_F32, rope_base)
    w.add_meta(arch + ".attention.layer_norm_rms_epsilon", T_F32, rms_eps)
    if tokenizer is None:
        w.add_meta("tokenizer.ggml.tokens", T_ARR, [""] * vocab, elem_type=T_STR)
    else:
        assert len(tokenizer["tokens"]) == vocab
        add_tokenizer_meta(w, tokenizer)
    rng = np.random.Generator(np.random.PCG64(seed))
    ctr = [seed * 1000003]

    def qmat(nrows, ncols, t):
        ctr[0] += 1
        return synth.normal_quantized(ctr[0], t, nrows, ncols, std)

    def norm_vec(n, scale=1.0):
        if norm_random:
            return _f32(rng.normal(1.0, 0.02, n) * scale)
        return _f32(np.ones(n) * scale)

    def rot(packed, nrows, shift):
        rb = packed.size // nrows
        return np.roll(packed.reshape(nrows, rb), shift, axis=0).reshape(-1)

    w.add_tensor("token_embd.weight", [dim, vocab], embd_type, qmat(vocab, dim, embd_type))
    base = {}
    for l in range(n_layers):
        p = "blk.%d." % l
        src = None if distinct_layers is None or l < distinct_layers else l % distinct_layers
        shapes = [("attn_q", dim, dim, wtype), ("attn_k", kv_dim, dim, wtype), ("attn_v", kv_dim, dim, v_type),
                  ("attn_output", dim, dim, wtype), ("ffn_gate", hidden_dim, dim, wtype),
                  ("ffn_up", hidden_dim, dim, wtype), ("ffn_down", dim, hidden_dim, wtype)]
        if tensor_types:     # e.g. {"ffn_down": 14}: the mixes of real K-quant files (Q6_K down / v in half of the layers)
            shapes = [(nm, nr, nc, tensor_types.get(nm, t)) for nm, nr, nc, t in shapes]
        w.add_tensor(p + "attn_norm.weight", [dim], 0, norm_vec(dim))
        for nm, nr, nc, t in shapes:
            if src is None:
                data = qmat(nr, nc, t)
                base[(l, nm)] = data
            else:
                data = rot(base[(src, nm)], nr, 1 + l // distinct_layers)
            w.add_tensor(p + nm + ".weight", [nc, nr], t, data)
            if bias and nm in ("attn_q", "attn_k", "attn_v"):
                w.add_tensor(p + nm + ".bias", [nr], 0, _f32(rng.normal(0.0, std, nr)))
        w.add_tensor(p + "ffn_norm.weight", [dim], 0, norm_vec(dim, ffn_norm_scale))
    w.add_tensor("output_norm.weight", [dim], 0, norm_vec(dim))
    if with_output:
        w.add_tensor("output.weight", [dim, vocab], out_type, qmat(vocab, dim, out_type))
    return w.to_bytes()


def gpt2_gguf(n_embd=768, n_layer=12, n_head=12, ff_len=3072, vocab=50257, n_seq=1024, wtype=8, seed=1234,
              std=0.02, ffn_norm_scale=1.0, tensor_hook=None):
    """Synthetic GPT-2-shape model file: LayerNorm g~N(1,.02), b~N(0,.02), biases N(0,.02); `ffn_norm_scale`: factor on
    the ffn_norm gains (large values push the normalised rows beyond the f16 range)."""
    w = GgufWriter()
    w.tensor_hook = tensor_hook
    w.add_meta("general.architecture", T_STR, "gpt2")
    w.add_meta("general.file_type", T_U32, 7)
    w.add_meta("gpt2.context_length", T_U32, n_seq)
    w.add_meta("gpt2.embedding_length", T_U32, n_embd)
    w.add_meta("gpt2.attention.head_count", T_U32, n_head)
    w.add_meta("gpt2.block_count", T_U32, n_layer)
    w.add_meta("gpt2.feed_forward_length", T_U32, ff_len)
    w.add_meta("tokenizer.ggml.tokens", T_ARR, [""] * vocab, elem_type=T_STR)
    rng = np.random.Generator(np.random.PCG64(seed))
    ctr = [seed * 1000003]

    def qmat(nrows, ncols, t):
        ctr[0] += 1
        return synth.normal_quantized(ctr[0], t, nrows, ncols, std)

    def vec(mean, n, scale=1.0):
        return _f32(rng.normal(mean, 0.02, n) * scale)

    w.add_tensor("token_embd.weight", [n_embd, vocab], wtype, qmat(vocab, n_embd, wtype))
    w.add_tensor("position_embd.weight", [n_embd, n_seq], 0, _f32(rng.normal(0.0, std, (n_seq, n_embd))))
    for l in range(n_layer):
        p = "blk.%d." % l
        w.add_tensor(p + "attn_norm.weight", [n_embd], 0, vec(1.0, n_embd))
        w.add_tensor(p + "attn_norm.bias", [n_embd], 0, vec(0.0, n_embd))
        w.add_tensor(p + "attn_qkv.weight", [n_embd, 3 * n_embd], wtype, qmat(3 * n_embd, n_embd, wtype))
        w.add_tensor(p + "attn_qkv.bias", [3 * n_embd], 0, vec(0.0, 3 * n_embd))
        w.add_tensor(p + "attn_output.weight", [n_embd, n_embd], wtype, qmat(n_embd, n_embd, wtype))
        w.add_tensor(p + "attn_output.bias", [n_embd], 0, vec(0.0, n_embd))
        w.add_tensor(p + "ffn_norm.weight", [n_embd], 0, vec(1.0, n_embd, ffn_norm_scale))
        w.add_tensor(p + "ffn_norm.bias", [n_embd], 0, vec(0.0, n_embd))
        w.add_tensor(p + "ffn_up.weight", [n_embd, ff_len], wtype, qmat(ff_len, n_embd, wtype))
        w.add_tensor(p + "ffn_up.bias", [ff_len], 0, vec(0.0, ff_len))
        w.add_tensor(p + "ffn_down.weight", [ff_len, n_embd], wtype, qmat(n_embd, ff_len, wtype))
        w.add_tensor(p + "ffn_down.bias", [n_embd], 0, vec(0.0, n_embd))
    w.add_tensor("output_norm.weight", [n_embd], 0, vec(1.0, n_embd))
    w.add_tensor("output_norm.bias", [n_embd], 0, vec(0.0, n_embd))
    return w.to_bytes()


def tiny_llama_gguf(seed=1234, wtype=8, **kw):
    """BASELINE configuration 1: dim 288, 6 layers, 6 heads, hidden 768, vocab 32000, seq 256, Q8_0."""
    args = dict(dim=288, hidden_dim=768, n_layers=6, n_heads=6, n_kv_heads=6, vocab=32000, seq_len=256,
                wtype=wtype, seed=seed)
    args.update(kw)
    return llama_gguf(**args)
