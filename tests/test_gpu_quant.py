"""GPU parity: device-layout upload + dequantisation (bit-exact) and dequant-fused GEMV per format."""
import numpy as np
import pytest

from gpu_common import backend, rel_err  # noqa: F401
from helpers import random_blocks, structured_blocks
from slai_amd import synth

pytestmark = pytest.mark.gpu
TYPES = [0, 1, 2, 8, 12, 13, 14]
NAMES = {0: "f32", 1: "f16", 2: "q4_0", 8: "q8_0", 12: "q4_k", 13: "q5_k", 14: "q6_k"}


def oracle_deq(L, t, raw, n):
    out = np.empty(n, np.float32)
    assert L.slo_dequantize(t, raw.ctypes.data, n, out.ctypes.data) == 0
    return out


@pytest.mark.parametrize("t", TYPES, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("shape", [(5, 256), (3, 2816), (64, 1024)])
def test_dequantize_bit_exact_random_blocks(backend, oracle_lib, t, shape):
    from slai_amd.runtime import GpuQuantMatrix
    nrows, ncols = shape
    print("case", NAMES[t], shape, flush=True)
    raw = random_blocks(t, nrows * ncols // oracle_lib.slo_block_elems(t), seed=31 * t + ncols)
    ref = oracle_deq(oracle_lib, t, raw, nrows * ncols).reshape(nrows, ncols)
    m = GpuQuantMatrix(backend, t, nrows, ncols, raw)
    assert m.shape() == (nrows, ncols, t)
    got = m.dequantize()
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    # a row range
    part = m.dequantize(1, 2)
    assert np.array_equal(part.view(np.uint32), ref[1:3].view(np.uint32))
    m.destroy()


@pytest.mark.parametrize("t", [2, 8, 12, 13, 14], ids=lambda t: NAMES[t])
def test_dequantize_structured_reference_inputs(backend, oracle_lib, t):
    from slai_amd.runtime import GpuQuantMatrix
    raw = structured_blocks(t, 16)
    be = oracle_lib.slo_block_elems(t)
    ncols = be * 4 if be == 32 else be * 2
    nrows = 16 * be // ncols
    ref = oracle_deq(oracle_lib, t, raw, nrows * ncols).reshape(nrows, ncols)
    m = GpuQuantMatrix(backend, t, nrows, ncols, raw)
    assert np.array_equal(m.dequantize().view(np.uint32), ref.view(np.uint32))
    m.destroy()


def test_dequantize_f16_specials(backend, oracle_lib):
    from slai_amd.runtime import GpuQuantMatrix
    u = np.arange(65536, dtype=np.uint16)
    ref = oracle_deq(oracle_lib, 1, u.view(np.uint8), 65536)
    m = GpuQuantMatrix(backend, 1, 64, 1024, u.view(np.uint8))
    got = m.dequantize().reshape(-1)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))   # includes subnormals, infinities and canonical NaNs
    m.destroy()


GEMV_SHAPES = [(64, 256), (37, 768), (8, 11008), (1027, 4096), (4096, 4096)]


@pytest.mark.parametrize("t", TYPES, ids=lambda t: NAMES[t])
@pytest.mark.parametrize("shape", GEMV_SHAPES)
def test_gemv_vs_oracle(backend, oracle_lib, t, shape):
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    nrows, ncols = shape
    print("case", NAMES[t], shape, flush=True)
    raw = synth.normal_quantized(1000 + t, t, nrows, ncols, 0.02)
    w = oracle_deq(oracle_lib, t, raw, nrows * ncols).reshape(nrows, ncols)
    x = synth.normal(77, ncols, 1.0)
    ref = np.empty(nrows, np.float32)
    oracle_lib.slo_gemv(ref.ctypes.data, w.ctypes.data, x.ctypes.data, nrows, ncols)
    ctxt = LlmContext(backend)
    m = GpuQuantMatrix(backend, t, nrows, ncols, raw)
    v = GpuTensor.vector(backend, x)
    out = GpuTensor(backend, nrows)
    ctxt.matmul_quant_assign(out, m, v)
    got = out.read()
    scale = np.abs(w).astype(np.float64) @ np.abs(x).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 3e-5 * scale + 1e-12), float((np.abs(got - ref) / scale).max())
    assert rel_err(got, ref) < 1e-3
    ref64 = w.astype(np.float64) @ x.astype(np.float64)
    assert rel_err(got, ref64) < 1e-4
    for o in (m, v, out):
        o.destroy()


def test_gemv_writes_into_a_cache_column_view(backend, oracle_lib):
    """`matmul_quant_assign(k_cache.column(pos), wk, xb)` (transformer.rs:329-334)."""
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    nrows, ncols, seq, pos = 96, 512, 8, 5
    raw = synth.normal_quantized(5, 8, nrows, ncols, 0.02)
    w = oracle_deq(oracle_lib, 8, raw, nrows * ncols).reshape(nrows, ncols)
    x = synth.normal(6, ncols, 1.0)
    m = GpuQuantMatrix(backend, 8, nrows, ncols, raw)
    v = GpuTensor.vector(backend, x)
    cache = GpuTensor(backend, nrows, seq)
    LlmContext(backend).matmul_quant_assign(cache.column(pos), m, v)
    got = cache.read_matrix()
    assert rel_err(got[:, pos], w.astype(np.float64) @ x.astype(np.float64)) < 1e-4
    assert np.all(got[:, :pos] == 0) and np.all(got[:, pos + 1:] == 0)
    for o in (m, v, cache):
        o.destroy()


def test_shape_errors_are_reported_not_fatal(backend):
    from slai_amd import _ffi
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext, SlaiError
    with pytest.raises(SlaiError) as e:
        GpuQuantMatrix(backend, 12, 4, 100, np.zeros(1000, np.uint8))     # ncols not a multiple of 256
    assert e.value.code == _ffi.E_SHAPE
    with pytest.raises(SlaiError) as e:
        GpuQuantMatrix(backend, 10, 4, 256, np.zeros(1000, np.uint8))     # Q2_K: no kernel
    assert e.value.code == _ffi.E_TYPE
    m = GpuQuantMatrix(backend, 8, 4, 64, synth.normal_quantized(1, 8, 4, 64))
    v, out = GpuTensor(backend, 32), GpuTensor(backend, 4)
    with pytest.raises(SlaiError) as e:
        LlmContext(backend).matmul_quant_assign(out, m, v)
    assert e.value.code == _ffi.E_SHAPE
    for o in (m, v, out):
        o.destroy()


@pytest.mark.parametrize("t", [8, 12, 14], ids=lambda t: NAMES[t])
def test_fused_op_forms(backend, oracle_lib, t):
    """rms-norm prologue, gate/up + SiLU, and residual-accumulate GEMV against the unfused oracle ops."""
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    dim, hid = 1024, 2816
    ctxt = LlmContext(backend)
    x, w = synth.normal(1, dim, 1.0), (1.0 + synth.normal(2, dim, 0.1)).astype(np.float32)
    xn = np.empty(dim, np.float32)
    oracle_lib.slo_rms_norm(xn.ctypes.data, x.ctypes.data, w.ctypes.data, dim, 1e-5)
    raws = [synth.normal_quantized(10 + i, t, hid, dim, 0.05) for i in range(2)]
    ws = [oracle_deq(oracle_lib, t, r, hid * dim).reshape(hid, dim) for r in raws]
    g = np.empty(hid, np.float32); u = np.empty(hid, np.float32)
    oracle_lib.slo_gemv(g.ctypes.data, ws[0].ctypes.data, xn.ctypes.data, hid, dim)
    oracle_lib.slo_gemv(u.ctypes.data, ws[1].ctypes.data, xn.ctypes.data, hid, dim)
    gate, up = [GpuQuantMatrix(backend, t, hid, dim, r) for r in raws]
    gx, gw, ghb = GpuTensor.vector(backend, x), GpuTensor.vector(backend, w), GpuTensor(backend, hid)
    ctxt.rms_norm_matmul_quant_assign(ghb, gate, gx, gw, 1e-5)
    assert rel_err(ghb.read(), g) < 1e-4
    h = g.copy(); oracle_lib.slo_silu(h.ctypes.data, u.ctypes.data, hid)
    ctxt.ffn_gate_up_silu(ghb, gate, up, gx, gw, 1e-5)
    assert rel_err(ghb.read(), h) < 1e-4
    # residual accumulate: x += Wd . h   (Wd: [dim x hid2])
    hid2 = 2816 if t == 8 else 3072
    rawd = synth.normal_quantized(21, t, dim, hid2, 0.05)
    wd = oracle_deq(oracle_lib, t, rawd, dim * hid2).reshape(dim, hid2)
    hv = synth.normal(22, hid2, 1.0)
    d = np.empty(dim, np.float32)
    oracle_lib.slo_gemv(d.ctypes.data, wd.ctypes.data, hv.ctypes.data, dim, hid2)
    down = GpuQuantMatrix(backend, t, dim, hid2, rawd)
    gh = GpuTensor.vector(backend, hv)
    ctxt.matmul_quant_add_assign(gx, down, gh)
    assert rel_err(gx.read(), x + d) < 1e-4
    for o in (gate, up, down, gx, gw, ghb, gh):
        o.destroy()
