"""Independent numpy twin of the C oracle -- TEST INFRASTRUCTURE ONLY.

Written separately from ``slai_oracle.c`` (vectorised, from the public ggml block
layouts and the textbook definitions of the ops) so that a slip in one of the two
restatements shows up as a disagreement.  Summation order differs from the C oracle
(numpy pairwise / BLAS), so whole-forward comparisons use a tolerance; dequantizers
are compared bit for bit.

Reference files restated: crates/slai/src/quantization.rs (block layouts),
crates/slai/src/models/llama2/cpu.rs:379-564, crates/slai/src/models/gpt2/cpu.rs:225-383.
"""
import numpy as np

F32 = np.float32


def decode_f16(u16):
    return np.asarray(u16, dtype=np.uint16).view(np.float16).astype(F32)


def _scale_min_k4(scales):
    """scales: [nb, 12] uint8 -> (sc [nb, 8], m [nb, 8]) uint8 (ggml get_scale_min_k4)."""
    s = scales.astype(np.uint8)
    sc = np.empty(s.shape[:-1] + (8,), dtype=np.uint8)
    mn = np.empty_like(sc)
    sc[..., :4] = s[..., 0:4] & 63
    mn[..., :4] = s[..., 4:8] & 63
    sc[..., 4:] = (s[..., 8:12] & 0xF) | ((s[..., 0:4] >> 6) << 4)
    mn[..., 4:] = (s[..., 8:12] >> 4) | ((s[..., 4:8] >> 6) << 4)
    return sc, mn


def dequantize(ggml_type, raw, n_elems):
    raw = np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw.view(np.uint8).reshape(-1)
    if ggml_type == 0:
        return raw[:n_elems * 4].view(F32).copy()
    if ggml_type == 1:
        return decode_f16(raw[:n_elems * 2].view(np.uint16))
    if ggml_type == 8:  # Q8_0: f16 d, 32 x i8
        b = raw[:n_elems // 32 * 34].reshape(-1, 34)
        d = decode_f16(b[:, 0:2].copy().view(np.uint16))
        q = b[:, 2:].view(np.int8).astype(F32)
        return (q * d).reshape(-1)
    if ggml_type == 2:  # Q4_0
        b = raw[:n_elems // 32 * 18].reshape(-1, 18)
        d = decode_f16(b[:, 0:2].copy().view(np.uint16))
        qs = b[:, 2:]
        lo = (qs & 0xF).astype(np.int32) - 8
        hi = (qs >> 4).astype(np.int32) - 8
        return (np.concatenate([lo, hi], axis=1).astype(F32) * d).reshape(-1)
    if ggml_type == 3:  # Q4_1
        b = raw[:n_elems // 32 * 20].reshape(-1, 20)
        d = decode_f16(b[:, 0:2].copy().view(np.uint16)); m = decode_f16(b[:, 2:4].copy().view(np.uint16))
        qs = b[:, 4:]
        q = np.concatenate([qs & 0xF, qs >> 4], axis=1).astype(F32)
        return (q * d + m).reshape(-1)
    if ggml_type in (6, 7):  # Q5_0 / Q5_1
        has_m = ggml_type == 7
        bs = 24 if has_m else 22
        b = raw[:n_elems // 32 * bs].reshape(-1, bs)
        d = decode_f16(b[:, 0:2].copy().view(np.uint16))
        o = 4 if has_m else 2
        qh = b[:, o:o + 4].copy().view(np.uint32)  # [nb,1]
        qs = b[:, o + 4:]
        j = np.arange(16, dtype=np.uint32)
        h0 = ((qh >> j) & 1).astype(np.int32) << 4
        h1 = ((qh >> (j + 16)) & 1).astype(np.int32) << 4
        lo = (qs & 0xF).astype(np.int32) | h0
        hi = (qs >> 4).astype(np.int32) | h1
        q = np.concatenate([lo, hi], axis=1)
        if has_m:
            m = decode_f16(b[:, 2:4].copy().view(np.uint16))
            return (q.astype(F32) * d + m).reshape(-1)
        return ((q - 16).astype(F32) * d).reshape(-1)
    if ggml_type == 15:  # Q8_K
        b = raw[:n_elems // 256 * 292].reshape(-1, 292)
        d = b[:, 0:4].copy().view(F32)
        q = b[:, 4:260].view(np.int8).astype(F32)
        return (d * q).reshape(-1)
    if ggml_type in (12, 13):  # Q4_K / Q5_K
        bs = 144 if ggml_type == 12 else 176
        b = raw[:n_elems // 256 * bs].reshape(-1, bs)
        d = decode_f16(b[:, 0:2].copy().view(np.uint16)); dmin = decode_f16(b[:, 2:4].copy().view(np.uint16))
        sc, mn = _scale_min_k4(b[:, 4:16])
        dsc = d * sc.astype(F32)          # [nb, 8]
        dmn = dmin * mn.astype(F32)
        if ggml_type == 12:
            qs = b[:, 16:].reshape(-1, 4, 32)
            hbit_lo = hbit_hi = 0
        else:
            qh = b[:, 16:48]                         # [nb, 32]
            qs = b[:, 48:].reshape(-1, 4, 32)
            c = np.arange(4).reshape(1, 4, 1)
            hbit_lo = ((qh[:, None, :] >> (2 * c)) & 1).astype(np.uint8) * 16
            hbit_hi = ((qh[:, None, :] >> (2 * c + 1)) & 1).astype(np.uint8) * 16
        lo = ((qs & 0xF) + hbit_lo).astype(F32)      # sub-block 2c
        hi = ((qs >> 4) + hbit_hi).astype(F32)       # sub-block 2c+1
        q = np.stack([lo, hi], axis=2).reshape(-1, 8, 32)
        return (dsc[:, :, None] * q - dmn[:, :, None]).astype(F32).reshape(-1)
    if ggml_type == 14:  # Q6_K: ql[128] qh[64] scales[16] d
        b = raw[:n_elems // 256 * 210].reshape(-1, 210)
        ql = b[:, :128].reshape(-1, 2, 64)
        qh = b[:, 128:192].reshape(-1, 2, 32)
        sc = b[:, 192:208].view(np.int8).reshape(-1, 2, 8).astype(F32)
        d = decode_f16(b[:, 208:210].copy().view(np.uint16)).reshape(-1, 1, 1)
        q1 = ((ql[:, :, :32] & 0xF) | (((qh >> 0) & 3) << 4)).astype(np.int32) - 32
        q2 = ((ql[:, :, 32:] & 0xF) | (((qh >> 2) & 3) << 4)).astype(np.int32) - 32
        q3 = ((ql[:, :, :32] >> 4) | (((qh >> 4) & 3) << 4)).astype(np.int32) - 32
        q4 = ((ql[:, :, 32:] >> 4) | (((qh >> 6) & 3) << 4)).astype(np.int32) - 32
        q = np.stack([q1, q2, q3, q4], axis=2).astype(F32)        # [nb, 2, 4, 32]
        isx = (np.arange(32) // 16)                               # l/16
        scale_idx = isx[None, :] + 2 * np.arange(4)[:, None]      # [4, 32]
        s = sc[:, :, scale_idx]                                   # [nb, 2, 4, 32]
        return ((d[..., None] * s).astype(F32) * q).astype(F32).reshape(-1)
    raise ValueError("no dequantizer for ggml type %d" % ggml_type)


def rms_norm(x, w, eps):
    x = x.astype(F32)
    ms = F32(np.dot(x.astype(np.float64), x.astype(np.float64)) / x.size)
    return (x * F32(1.0 / np.sqrt(ms + F32(eps)))).astype(F32) * w


def softmax(v):
    e = np.exp(v - v.max())
    return (e / e.sum()).astype(F32)


def rope_adjacent(v, head_size, pos, base=10000.0, limit=None):
    v = v.copy()
    n = v.size if limit is None else limit
    i = np.arange(0, n, 2)
    theta = np.power(F32(base), -(i % head_size).astype(F32) / F32(head_size)).astype(F32)
    ang = (F32(pos) * theta).astype(F32)
    c, s = np.cos(ang), np.sin(ang)
    x, y = v[i], v[i + 1]
    v[i], v[i + 1] = c * x - s * y, s * x + c * y
    return v


def attention(q, kc, vc, n_heads, kv_mul, head_size, pos):
    """kc, vc: [seq, kv_dim] arrays (position-major)."""
    out = np.zeros(n_heads * head_size, dtype=F32)
    for h in range(n_heads):
        o = (h // kv_mul) * head_size
        k = kc[:pos + 1, o:o + head_size]
        v = vc[:pos + 1, o:o + head_size]
        s = (k @ q[h * head_size:(h + 1) * head_size]) / F32(np.sqrt(F32(head_size)))
        out[h * head_size:(h + 1) * head_size] = softmax(s.astype(F32)) @ v
    return out


def gelu(x):
    x = x.astype(F32)
    return (F32(0.5) * x * (F32(1.0) + np.tanh(F32(0.7978846) * x * (F32(1.0) + F32(0.044715) * x * x)))).astype(F32)


def layernorm(v, eps=1e-5):
    v = v.astype(F32)
    c = v - v.mean(dtype=np.float64).astype(F32)
    var = F32(np.dot(c.astype(np.float64), c.astype(np.float64)) / v.size)
    return (c * F32(1.0 / np.sqrt(var + F32(eps)))).astype(F32)


class NpLlama:
    """cpu.rs Transformer::forward on dequantized f32 numpy weights (dict name -> array)."""

    def __init__(self, cfg, tensors, eps=1e-5, base=10000.0):
        self.cfg, self.t, self.eps, self.base = cfg, tensors, eps, base
        kv_dim = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
        self.kc = [np.zeros((cfg["seq_len"], kv_dim), dtype=F32) for _ in range(cfg["n_layers"])]
        self.vc = [np.zeros((cfg["seq_len"], kv_dim), dtype=F32) for _ in range(cfg["n_layers"])]

    def forward(self, token, pos):
        c, t = self.cfg, self.t
        hs = c["dim"] // c["n_heads"]
        kv_dim = c["dim"] * c["n_kv_heads"] // c["n_heads"]
        x = t["token_embd.weight"][token].copy()
        for l in range(c["n_layers"]):
            p = "blk.%d." % l
            xb = rms_norm(x, t[p + "attn_norm.weight"], self.eps)
            q = t[p + "attn_q.weight"] @ xb
            k = t[p + "attn_k.weight"] @ xb
            v = t[p + "attn_v.weight"] @ xb
            q = rope_adjacent(q, hs, pos, self.base)
            k = rope_adjacent(k, hs, pos, self.base, limit=kv_dim)
            self.kc[l][pos], self.vc[l][pos] = k, v
            a = attention(q, self.kc[l], self.vc[l], c["n_heads"], c["n_heads"] // c["n_kv_heads"], hs, pos)
            x = x + t[p + "attn_output.weight"] @ a
            xb = rms_norm(x, t[p + "ffn_norm.weight"], self.eps)
            g = t[p + "ffn_gate.weight"] @ xb
            u = t[p + "ffn_up.weight"] @ xb
            h = u * (g / (F32(1.0) + np.exp(-g)))
            x = x + t[p + "ffn_down.weight"] @ h.astype(F32)
        xb = rms_norm(x, t["output_norm.weight"], self.eps)
        out = t.get("output.weight", t["token_embd.weight"])
        return (out @ xb).astype(F32)


class NpGpt2:
    """gpt2/cpu.rs Transformer::forward on dequantized f32 numpy weights."""

    def __init__(self, cfg, tensors):
        self.cfg, self.t = cfg, tensors
        E = cfg["n_embd"]
        self.kc = [np.zeros((cfg["n_seq"], E), dtype=F32) for _ in range(cfg["n_layer"])]
        self.vc = [np.zeros((cfg["n_seq"], E), dtype=F32) for _ in range(cfg["n_layer"])]

    def forward(self, token, pos):
        c, t = self.cfg, self.t
        E = c["n_embd"]
        hs = E // c["n_head"]
        x = t["token_embd.weight"][token] + t["position_embd.weight"][pos]
        for l in range(c["n_layer"]):
            p = "blk.%d." % l
            cur = layernorm(x) * t[p + "attn_norm.weight"] + t[p + "attn_norm.bias"]
            qkv = t[p + "attn_qkv.weight"] @ cur + t[p + "attn_qkv.bias"]
            self.kc[l][pos], self.vc[l][pos] = qkv[E:2 * E], qkv[2 * E:]
            a = attention(qkv[:E], self.kc[l], self.vc[l], c["n_head"], 1, hs, pos)
            x = x + (t[p + "attn_output.weight"] @ a + t[p + "attn_output.bias"])
            cur = layernorm(x) * t[p + "ffn_norm.weight"] + t[p + "ffn_norm.bias"]
            h = gelu(t[p + "ffn_up.weight"] @ cur + t[p + "ffn_up.bias"])
            x = x + (t[p + "ffn_down.weight"] @ h + t[p + "ffn_down.bias"])
        cur = layernorm(x) * t["output_norm.weight"] + t["output_norm.bias"]
        return (t["token_embd.weight"] @ cur).astype(F32)
