"""Pins the oracle's ops against closed forms, library routines (torch CPU, numpy)
and invariants.  LEN 1757 as in the reference's op tests (ops/silu.rs:97 etc.)."""
import math

import numpy as np
import pytest
import torch

LEN = 1757


def rnd(seed, n, scale=1.0):
    return (np.random.Generator(np.random.PCG64(seed)).normal(0, scale, n)).astype(np.float32)


def test_gemv_vs_float64(oracle_lib):
    w, x = rnd(1, 37 * 300).reshape(37, 300), rnd(2, 300)
    out = np.empty(37, np.float32)
    oracle_lib.slo_gemv(out.ctypes.data, w.ctypes.data, x.ctypes.data, 37, 300)
    ref = w.astype(np.float64) @ x.astype(np.float64)
    assert np.abs(out - ref).max() < 300 * 2 ** -23 * np.abs(w).max() * np.abs(x).max() * 4
    # a transposed operand or a dropped column fails these exact cases
    w2 = np.zeros((3, 4), np.float32); w2[1, 2] = 2.0; w2[2, 3] = -1.0
    x2 = np.array([1, 10, 100, 1000], np.float32); o2 = np.empty(3, np.float32)
    oracle_lib.slo_gemv(o2.ctypes.data, w2.ctypes.data, x2.ctypes.data, 3, 4)
    assert o2.tolist() == [0.0, 200.0, -1000.0]
    # sequential accumulation order (nalgebra gemv = column axpys): 1e8 + 1 - 1e8 in f32
    w3 = np.array([[1e8, 1.0, -1e8]], np.float32); x3 = np.ones(3, np.float32); o3 = np.empty(1, np.float32)
    oracle_lib.slo_gemv(o3.ctypes.data, w3.ctypes.data, x3.ctypes.data, 1, 3)
    assert o3[0] == 0.0


def test_dot_order_and_value(oracle_lib):
    a, b = rnd(3, 1003), rnd(4, 1003)
    got = oracle_lib.slo_dot(a.ctypes.data, b.ctypes.data, 1003)
    assert abs(got - float(a.astype(np.float64) @ b.astype(np.float64))) < 1e-3
    # 8-lane interleave: lanes 0 and 4 are folded together first
    a = np.zeros(16, np.float32); b = np.ones(16, np.float32)
    a[0], a[4], a[8] = 1e8, -1e8, 1.0      # lane0 = (1e8 + 1) -> 1e8 ; lane4 = -1e8 ; (lane0+lane4) = 0
    assert oracle_lib.slo_dot(a.ctypes.data, b.ctypes.data, 16) == 0.0


def test_rms_norm_vs_torch(oracle_lib):
    x, w = rnd(5, LEN), rnd(6, LEN)
    out = np.empty(LEN, np.float32)
    oracle_lib.slo_rms_norm(out.ctypes.data, x.ctypes.data, w.ctypes.data, LEN, 1e-5)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x), (LEN,), torch.from_numpy(w), 1e-5).numpy()
    np.testing.assert_allclose(out, ref, rtol=2e-6, atol=1e-7)
    # eps matters: tiny input
    x2 = (x * 1e-4).astype(np.float32)
    o5 = np.empty(LEN, np.float32); o6 = np.empty(LEN, np.float32)
    oracle_lib.slo_rms_norm(o5.ctypes.data, x2.ctypes.data, w.ctypes.data, LEN, 1e-5)
    oracle_lib.slo_rms_norm(o6.ctypes.data, x2.ctypes.data, w.ctypes.data, LEN, 1e-6)
    assert np.abs(o5 - o6).max() > 1e-3


def test_softmax_vs_torch(oracle_lib):
    v = rnd(7, LEN, 3.0)
    got = v.copy()
    oracle_lib.slo_softmax(got.ctypes.data, LEN)
    ref = torch.softmax(torch.from_numpy(v).double(), 0).numpy()
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-9)
    assert abs(got.sum(dtype=np.float64) - 1.0) < 1e-5
    big = np.array([1000.0, 1000.0, -1000.0], np.float32)
    oracle_lib.slo_softmax(big.ctypes.data, 3)
    assert big.tolist() == [0.5, 0.5, 0.0]


def test_silu_gelu_layernorm_vs_torch(oracle_lib):
    a, b = rnd(8, LEN, 2.0), rnd(9, LEN)
    got = a.copy()
    oracle_lib.slo_silu(got.ctypes.data, b.ctypes.data, LEN)
    ref = (torch.nn.functional.silu(torch.from_numpy(a).double()) * torch.from_numpy(b).double()).numpy()
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-7)
    g = a.copy()
    oracle_lib.slo_gelu_n(g.ctypes.data, LEN)
    refg = torch.nn.functional.gelu(torch.from_numpy(a).double(), approximate="tanh").numpy()
    np.testing.assert_allclose(g, refg, rtol=1e-5, atol=2e-7)
    ln = np.empty(LEN, np.float32)
    oracle_lib.slo_layernorm(ln.ctypes.data, a.ctypes.data, LEN, 1e-5)
    refl = torch.nn.functional.layer_norm(torch.from_numpy(a).double(), (LEN,), eps=1e-5).numpy()
    np.testing.assert_allclose(ln, refl, rtol=1e-5, atol=1e-6)


def test_argmax_first_max(oracle_lib):
    v = rnd(10, 5000)
    assert oracle_lib.slo_argmax(v.ctypes.data, 5000) == int(np.argmax(v))
    t = np.array([1.0, 3.0, 3.0, 2.0, 3.0], np.float32)
    assert oracle_lib.slo_argmax(t.ctypes.data, 5) == 1


@pytest.mark.parametrize("neox", [0, 1])
def test_rope_invariants_and_closed_form(oracle_lib, neox):
    hs, nq, nk, pos = 128, 13, 9, 10     # shapes of the reference test ops/rope.rs:160-170
    dim, kv_dim = hs * nq, hs * nk
    q0, k0 = rnd(11, dim), rnd(12, kv_dim)
    q, k = q0.copy(), k0.copy()
    oracle_lib.slo_rope(q.ctypes.data, k.ctypes.data, hs, dim, kv_dim, 0, 10000.0, neox)
    assert np.array_equal(q, q0) and np.array_equal(k, k0)          # identity at pos 0
    q, k = q0.copy(), k0.copy()
    oracle_lib.slo_rope(q.ctypes.data, k.ctypes.data, hs, dim, kv_dim, pos, 10000.0, neox)
    for v, v0, n in ((q, q0, nq), (k, k0, nk)):
        a, a0 = v.reshape(n, hs).astype(np.float64), v0.reshape(n, hs).astype(np.float64)
        np.testing.assert_allclose((a ** 2).sum(1), (a0 ** 2).sum(1), rtol=1e-5)   # norm preserving
        j = np.arange(hs // 2)
        ang = pos * 10000.0 ** (-(2 * j) / hs)
        if neox:
            x, y = a0[:, :hs // 2], a0[:, hs // 2:]
            exp = np.concatenate([np.cos(ang) * x - np.sin(ang) * y, np.sin(ang) * x + np.cos(ang) * y], axis=1)
        else:
            x, y = a0[:, 0::2], a0[:, 1::2]
            exp = np.empty_like(a0)
            exp[:, 0::2] = np.cos(ang) * x - np.sin(ang) * y
            exp[:, 1::2] = np.sin(ang) * x + np.cos(ang) * y
        np.testing.assert_allclose(a, exp, rtol=0, atol=2e-5)
    # keys beyond kv_dim untouched: kv_dim < dim and a longer k buffer
    kbig = rnd(13, dim); kb0 = kbig.copy(); q = q0.copy()
    oracle_lib.slo_rope(q.ctypes.data, kbig.ctypes.data, hs, dim, kv_dim, pos, 10000.0, neox)
    assert np.array_equal(kbig[kv_dim:], kb0[kv_dim:]) and not np.array_equal(kbig[:kv_dim], kb0[:kv_dim])


def test_attention_invariants(oracle_lib):
    n_heads, kv_mul, hs, seq = 6, 2, 48, 32
    kv_dim = n_heads // kv_mul * hs
    q = rnd(14, n_heads * hs)
    kc = rnd(15, seq * kv_dim).reshape(seq, kv_dim); vc = rnd(16, seq * kv_dim).reshape(seq, kv_dim)
    att = np.zeros(seq * n_heads, np.float32); xb = np.empty(n_heads * hs, np.float32)

    def run(pos, kc_, vc_):
        oracle_lib.slo_attention(n_heads, kv_mul, hs, pos, seq, kv_dim, q.ctypes.data, kc_.ctypes.data,
                                 vc_.ctypes.data, att.ctypes.data, xb.ctypes.data)
        return xb.copy()

    out0 = run(0, kc, vc)      # pos 0 -> V[0] of the matching kv head
    for h in range(n_heads):
        o = (h // kv_mul) * hs
        assert np.array_equal(out0[h * hs:(h + 1) * hs], vc[0, o:o + hs])
    ke = np.tile(kc[0], (seq, 1)).copy()   # equal keys -> mean of V
    oute = run(9, ke, vc)
    for h in range(n_heads):
        o = (h // kv_mul) * hs
        np.testing.assert_allclose(oute[h * hs:(h + 1) * hs], vc[:10, o:o + hs].mean(0), rtol=1e-5, atol=1e-6)
    # general case vs float64 softmax attention
    pos = 20
    out = run(pos, kc, vc)
    for h in range(n_heads):
        o = (h // kv_mul) * hs
        s = kc[:pos + 1, o:o + hs].astype(np.float64) @ q[h * hs:(h + 1) * hs].astype(np.float64) / math.sqrt(hs)
        p = np.exp(s - s.max()); p /= p.sum()
        np.testing.assert_allclose(out[h * hs:(h + 1) * hs], p @ vc[:pos + 1, o:o + hs].astype(np.float64), rtol=1e-4, atol=1e-6)
        np.testing.assert_allclose(att[h * seq:h * seq + pos + 1], p, rtol=1e-4, atol=1e-7)
