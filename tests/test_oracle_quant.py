"""Pins the oracle's f16 decoder and block dequantizers (CPU only).

Checks are chosen so a plausible slip (wrong nibble half, wrong scale index, a
dropped -8/-32 offset, d*q-m fused or reordered) fails at least one of them."""
import numpy as np
import pytest

from helpers import random_blocks, structured_blocks
from oracle import np_oracle

ALL_TYPES = [0, 1, 2, 3, 6, 7, 8, 12, 13, 14, 15]


def deq(L, t, raw, n):
    out = np.empty(n, dtype=np.float32)
    assert L.slo_dequantize(t, raw.ctypes.data, n, out.ctypes.data) == 0
    return out


def test_decode_f16_exhaustive(oracle_lib):
    u = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, dtype=np.float32)
    oracle_lib.slo_decode_f16_n(u.ctypes.data, 65536, out.ctypes.data)
    ref = u.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(out), nan)
    assert np.array_equal(out[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    # the reference yields the canonical f32::NAN with the sign applied last (quantization.rs:401-408)
    assert set(np.unique(out[nan].view(np.uint32))) == {0x7fc00000, 0xffc00000}


def test_encode_f16_matches_ieee(oracle_lib):
    rng = np.random.Generator(np.random.PCG64(5))
    vals = np.concatenate([rng.normal(0, 1, 20000), rng.normal(0, 1e-6, 5000), rng.normal(0, 3e4, 5000),
                           [0.0, -0.0, 65504.0, 65520.0, 65519.99, 1e-8, 6e-8, 2.98e-8, 2.99e-8, np.inf, -np.inf]]).astype(np.float32)
    # exact ties
    ties = (np.arange(1024, 2048, dtype=np.float32) + 0.5) / 1024.0
    vals = np.concatenate([vals, ties.astype(np.float32)])
    with np.errstate(over="ignore"):
        ref = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle_lib.slo_encode_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, ref)


def test_get_scale_min_k4_bruteforce(oracle_lib):
    """All byte values at every position, against the 6-bit packing written out longhand."""
    import ctypes as C
    rng = np.random.Generator(np.random.PCG64(1))
    for trial in range(64):
        q = rng.integers(0, 256, 12, dtype=np.uint8)
        for pos in range(12):
            for val in range(0, 256, 5):
                q2 = q.copy(); q2[pos] = val
                for j in range(8):
                    d, m = C.c_uint8(0), C.c_uint8(0)
                    oracle_lib.slo_get_scale_min_k4(j, q2.ctypes.data, C.byref(d), C.byref(m))
                    if j < 4:
                        ed, em = q2[j] % 64, q2[j + 4] % 64
                    else:
                        ed = (q2[j + 4] % 16) + 16 * (q2[j - 4] // 64)
                        em = (q2[j + 4] // 16) + 16 * (q2[j] // 64)
                    assert (d.value, m.value) == (ed, em)
            break  # positions x values once; remaining trials below vary the whole array
        sc, mn = np_oracle._scale_min_k4(q[None, :])
        for j in range(8):
            d, m = C.c_uint8(0), C.c_uint8(0)
            oracle_lib.slo_get_scale_min_k4(j, q.ctypes.data, C.byref(d), C.byref(m))
            assert (d.value, m.value) == (sc[0, j], mn[0, j])


def test_hand_computable_blocks(oracle_lib):
    L = oracle_lib
    one = np.uint16(0x3C00).tobytes()  # f16 1.0
    # Q8_0 with scale 1.0: output == the int8 payload
    q = np.arange(-16, 16, dtype=np.int8)
    out = deq(L, 8, np.frombuffer(one + q.tobytes(), dtype=np.uint8).copy(), 32)
    assert np.array_equal(out, q.astype(np.float32))
    # Q4_0 all 0x88 -> zeros; byte j = j | (15-j)<<4 -> low half j-8, high half 7-j
    out = deq(L, 2, np.frombuffer(one + bytes([0x88] * 16), dtype=np.uint8).copy(), 32)
    assert np.array_equal(out, np.zeros(32, np.float32))
    qs = bytes([j | ((15 - j) << 4) for j in range(16)])
    out = deq(L, 2, np.frombuffer(one + qs, dtype=np.uint8).copy(), 32)
    assert np.array_equal(out, np.concatenate([np.arange(16) - 8, 7 - np.arange(16)]).astype(np.float32))
    # Q4_K with d=1, dmin=1, sc=[1..8], m=[8..1]: element (sub-block s, l) = sc_s*nibble - m_s
    sc = np.arange(1, 9); mn = np.arange(8, 0, -1)
    scales = np.zeros(12, np.uint8)
    scales[0:4] = sc[:4]; scales[4:8] = mn[:4]
    scales[8:12] = (sc[4:] & 0xF) | ((mn[4:] & 0xF) << 4)
    nib = (np.arange(256) * 7 + 3) % 16
    qs = np.zeros(128, np.uint8)
    for c in range(4):
        qs[32 * c:32 * c + 32] = nib[64 * c:64 * c + 32] | (nib[64 * c + 32:64 * c + 64] << 4)
    raw = np.frombuffer(one + one + scales.tobytes() + qs.tobytes(), dtype=np.uint8).copy()
    out = deq(L, 12, raw, 256)
    exp = (np.repeat(sc, 32) * nib - np.repeat(mn, 32)).astype(np.float32)
    assert np.array_equal(out, exp)
    # Q5_K: same block with qh bit (2c) set for even l, bit (2c+1) for l%3==0 -> +16
    qh = np.zeros(32, np.uint8)
    for c in range(4):
        for l in range(32):
            if l % 2 == 0: qh[l] |= 1 << (2 * c)
            if l % 3 == 0: qh[l] |= 2 << (2 * c)
    raw5 = np.frombuffer(one + one + scales.tobytes() + qh.tobytes() + qs.tobytes(), dtype=np.uint8).copy()
    out5 = deq(L, 13, raw5, 256)
    add = np.zeros(256)
    for c in range(4):
        l = np.arange(32)
        add[64 * c:64 * c + 32] = 16 * (l % 2 == 0)
        add[64 * c + 32:64 * c + 64] = 16 * (l % 3 == 0)
    exp5 = (np.repeat(sc, 32) * (nib + add) - np.repeat(mn, 32)).astype(np.float32)
    assert np.array_equal(out5, exp5)
    # Q6_K with d=1, scales[k]=k+1, six-bit value v(e) = (5e+1)%64 for element e -> (k+1)*(v-32)
    v = (np.arange(256) * 5 + 1) % 64
    ql = np.zeros(128, np.uint8); qh6 = np.zeros(64, np.uint8)
    for i in range(2):
        for l in range(32):
            e = [128 * i + l, 128 * i + l + 32, 128 * i + l + 64, 128 * i + l + 96]
            ql[64 * i + l] = (v[e[0]] & 0xF) | ((v[e[2]] & 0xF) << 4)
            ql[64 * i + l + 32] = (v[e[1]] & 0xF) | ((v[e[3]] & 0xF) << 4)
            qh6[32 * i + l] = (v[e[0]] >> 4) | ((v[e[1]] >> 4) << 2) | ((v[e[2]] >> 4) << 4) | ((v[e[3]] >> 4) << 6)
    sc6 = np.arange(1, 17, dtype=np.int8)
    raw6 = np.frombuffer(ql.tobytes() + qh6.tobytes() + sc6.tobytes() + one, dtype=np.uint8).copy()
    out6 = deq(L, 14, raw6, 256)
    exp6 = (np.repeat(sc6.astype(np.int32), 16) * (v - 32)).astype(np.float32)
    assert np.array_equal(out6, exp6)


@pytest.mark.parametrize("t", [2, 3, 6, 7, 8, 12, 13, 14, 15])
def test_structured_inputs_c_vs_numpy(oracle_lib, t):
    raw = structured_blocks(t)
    be = oracle_lib.slo_block_elems(t)
    n = raw.size // oracle_lib.slo_block_bytes(t) * be
    a = deq(oracle_lib, t, raw, n)
    b = np_oracle.dequantize(t, raw, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("t", ALL_TYPES)
def test_random_blocks_c_vs_numpy_bit_exact(oracle_lib, t):
    nb = 4096 if oracle_lib.slo_block_elems(t) > 1 else 65536
    raw = random_blocks(t, nb, seed=100 + t)
    n = nb * oracle_lib.slo_block_elems(t)
    a = deq(oracle_lib, t, raw, n)
    b = np_oracle.dequantize(t, raw, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("t", [1, 2, 8, 12, 13, 14])
def test_quantizer_roundtrip_error(oracle_lib, t):
    """The synthetic-model quantizers are input generators; they must still land near the source."""
    from slai_amd import synth
    x = synth.normal(3, 64 * 1024, 0.02).reshape(64, 1024)
    raw = synth.quantize(t, x)
    y = deq(oracle_lib, t, raw, x.size).reshape(x.shape)
    rel = np.abs(y - x).max() / np.abs(x).max()
    bound = {1: 1e-3, 2: 0.08, 8: 5e-3, 12: 0.08, 13: 0.04, 14: 0.02}[t]
    assert rel < bound, rel
    a = synth.normal_quantized(11, t, 8, 512)
    b = synth.quantize(t, synth.normal(11, 8 * 512, 0.02).reshape(8, 512))
    assert np.array_equal(a, b)
