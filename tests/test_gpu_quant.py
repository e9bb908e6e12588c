"""GPU parity: device-layout upload + dequantisation (bit-exact) and dequant-fused GEMV per format."""
import numpy as np
import pytest

from gpu_common import backend, rel_err  # noqa: F401
from helpers import random_blocks, structured_blocks
from slai_amd import synth

pytestmark = pytest.mark.gpu
TYPES = [0, 1, 2, 3, 6, 7, 8, 12, 13, 14, 15]
NAMES = {0: "f32", 1: "f16", 2: "q4_0", 3: "q4_1", 6: "q5_0", 7: "q5_1", 8: "q8_0", 12: "q4_k", 13: "q5_k", 14: "q6_k", 15: "q8_k"}


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


# (the last three are the benchmark's GEMV sweep shapes and the down-projection shape of the 7B layer)
GEMV_SHAPES = [(64, 256), (37, 768), (8, 11008), (1027, 4096), (4096, 4096), (11008, 4096), (4096, 11008)]


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


@pytest.mark.parametrize("t", [2, 8, 12, 13, 14], ids=lambda t: NAMES[t])
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
    hid2 = 2816 if t in (2, 8) else 3072
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


# ---- device layouts: every layout must serve every op with the same results -------------------------------
LAYOUTS = {"rows": 1, "tile16": 2, "tile64": 3}


@pytest.mark.parametrize("layout", list(LAYOUTS), ids=list(LAYOUTS))
@pytest.mark.parametrize("t", [2, 8, 12, 13, 14], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("shape", [(64, 256), (200, 1024), (70, 2816), (1027, 4096)])
def test_layouts_dequantize_and_gemv(backend, oracle_lib, layout, t, shape):
    """Bit-exact dequantisation and GEMV parity in each device layout (row tails, odd super-block counts)."""
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    nrows, ncols = shape
    print("case", layout, NAMES[t], shape, flush=True)
    raw = synth.normal_quantized(500 + t, t, nrows, ncols, 0.02)
    w = oracle_deq(oracle_lib, t, raw, nrows * ncols).reshape(nrows, ncols)
    m = GpuQuantMatrix(backend, t, nrows, ncols, raw, layout=LAYOUTS[layout])
    assert np.array_equal(m.dequantize().view(np.uint32), w.view(np.uint32))
    x = synth.normal(78, ncols, 1.0)
    ref = np.empty(nrows, np.float32)
    oracle_lib.slo_gemv(ref.ctypes.data, w.ctypes.data, x.ctypes.data, nrows, ncols)
    ctxt = LlmContext(backend)
    v, out = GpuTensor.vector(backend, x), GpuTensor(backend, nrows)
    ctxt.matmul_quant_assign(out, m, v)
    got = out.read()
    scale = np.abs(w).astype(np.float64) @ np.abs(x).astype(np.float64)
    assert np.all(np.abs(got - ref) <= 3e-5 * scale + 1e-12), float((np.abs(got - ref) / scale).max())
    for o in (m, v, out):
        o.destroy()


@pytest.mark.parametrize("t", [2, 8, 12, 13, 14], ids=lambda t: NAMES[t])
def test_tile64_fused_forms_and_changing_input(backend, oracle_lib, t):
    """64-row tiles: RMSNorm prologue, gate/up + SiLU and residual accumulate; the input vector changes between
    launches (the kernel reads its activations through the scalar cache, which must never serve stale data)."""
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    dim, hid = 1024, 2880
    ctxt = LlmContext(backend)
    raws = [synth.normal_quantized(30 + i, t, hid, dim, 0.05) for i in range(2)]
    ws = [oracle_deq(oracle_lib, t, r, hid * dim).reshape(hid, dim) for r in raws]
    gate, up = [GpuQuantMatrix(backend, t, hid, dim, r, layout=3) for r in raws]
    gw_np = (1.0 + synth.normal(2, dim, 0.1)).astype(np.float32)
    gx, gw, ghb = GpuTensor(backend, dim), GpuTensor.vector(backend, gw_np), GpuTensor(backend, hid)
    for rep in range(4):
        x = synth.normal(100 + rep, dim, 1.0 + rep)
        gx.write(x)
        xn = np.empty(dim, np.float32)
        oracle_lib.slo_rms_norm(xn.ctypes.data, x.ctypes.data, gw_np.ctypes.data, dim, 1e-5)
        g = np.empty(hid, np.float32); u = np.empty(hid, np.float32)
        oracle_lib.slo_gemv(g.ctypes.data, ws[0].ctypes.data, xn.ctypes.data, hid, dim)
        oracle_lib.slo_gemv(u.ctypes.data, ws[1].ctypes.data, xn.ctypes.data, hid, dim)
        ctxt.rms_norm_matmul_quant_assign(ghb, gate, gx, gw, 1e-5)
        assert rel_err(ghb.read(), g) < 1e-4, rep
        h = g.copy(); oracle_lib.slo_silu(h.ctypes.data, u.ctypes.data, hid)
        ctxt.ffn_gate_up_silu(ghb, gate, up, gx, gw, 1e-5)
        assert rel_err(ghb.read(), h) < 1e-4, rep
        ctxt.matmul_quant_assign(ghb, up, gx)
        plain = np.empty(hid, np.float32)
        oracle_lib.slo_gemv(plain.ctypes.data, ws[1].ctypes.data, x.ctypes.data, hid, dim)
        assert rel_err(ghb.read(), plain) < 1e-4, rep
    # residual accumulate over a wide input (43 super-blocks: waves walk several of them)
    hid2 = 11008
    rawd = synth.normal_quantized(41, t, 192, hid2, 0.05)
    wd = oracle_deq(oracle_lib, t, rawd, 192 * hid2).reshape(192, hid2)
    hv, x0 = synth.normal(42, hid2, 1.0), synth.normal(43, 192, 1.0)
    d = np.empty(192, np.float32)
    oracle_lib.slo_gemv(d.ctypes.data, wd.ctypes.data, hv.ctypes.data, 192, hid2)
    down = GpuQuantMatrix(backend, t, 192, hid2, rawd, layout=3)
    gh, gacc = GpuTensor.vector(backend, hv), GpuTensor.vector(backend, x0)
    ctxt.matmul_quant_add_assign(gacc, down, gh)
    assert rel_err(gacc.read(), x0 + d) < 1e-4
    for o in (gate, up, down, gx, gw, ghb, gh, gacc):
        o.destroy()


@pytest.mark.parametrize("t", [2, 8, 12, 13, 14], ids=lambda t: NAMES[t])
def test_prepared_activations_chain(backend, oracle_lib, t):
    """x += Wd.h leaving the prepared form of the new x, then RMSNorm + gate/up + SiLU (and a plain RMSNorm GEMV) reading
    it: equal to the unfused oracle sequence; also slai_rms_norm_prepare itself."""
    import os
    if os.environ.get("SLAI_ROWTILE") == "0" or os.environ.get("SLAI_TILED") == "0":
        pytest.skip("prepared activations need the tiled layouts, which this environment switches off")
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    dim, hid = 1024, 2816
    ctxt = LlmContext(backend)
    rawd = synth.normal_quantized(61, t, dim, hid, 0.05)
    wd = oracle_deq(oracle_lib, t, rawd, dim * hid).reshape(dim, hid)
    raws = [synth.normal_quantized(62 + i, t, hid, dim, 0.05) for i in range(2)]
    ws = [oracle_deq(oracle_lib, t, r, hid * dim).reshape(hid, dim) for r in raws]
    down = GpuQuantMatrix(backend, t, dim, hid, rawd, layout=2)
    gate, up = [GpuQuantMatrix(backend, t, hid, dim, r, layout=3) for r in raws]
    nw = (1.0 + synth.normal(3, dim, 0.1)).astype(np.float32)
    gnw, gprep, ghb = GpuTensor.vector(backend, nw), GpuTensor(backend, dim + dim // 16), GpuTensor(backend, hid)
    gx, gh = GpuTensor(backend, dim), GpuTensor(backend, hid)
    for rep in range(3):
        x0, hv = synth.normal(200 + rep, dim, 1.0), synth.normal(300 + rep, hid, 1.0 + rep)
        gx.write(x0); gh.write(hv)
        d = np.empty(dim, np.float32)
        oracle_lib.slo_gemv(d.ctypes.data, wd.ctypes.data, hv.ctypes.data, dim, hid)
        x1 = x0 + d
        ctxt.matmul_quant_add_assign_emit(gx, down, gh, gnw, gprep)
        got_x = gx.read()
        assert rel_err(got_x, x1) < 1e-4
        prep = gprep.read()
        assert rel_err(prep[:dim], got_x * nw) < 1e-6
        assert rel_err(prep[dim:], (got_x * nw).reshape(-1, 16).sum(axis=1)) < 1e-5
        xn = np.empty(dim, np.float32)
        oracle_lib.slo_rms_norm(xn.ctypes.data, got_x.ctypes.data, nw.ctypes.data, dim, 1e-5)
        g = np.empty(hid, np.float32); u = np.empty(hid, np.float32)
        oracle_lib.slo_gemv(g.ctypes.data, ws[0].ctypes.data, xn.ctypes.data, hid, dim)
        oracle_lib.slo_gemv(u.ctypes.data, ws[1].ctypes.data, xn.ctypes.data, hid, dim)
        h = g.copy(); oracle_lib.slo_silu(h.ctypes.data, u.ctypes.data, hid)
        if t != 8:                                     # a gated Q8_0 pair takes the general path, which has no prepared form
            ctxt.ffn_gate_up_silu_prepared(ghb, gate, up, gx, gprep, 1e-5)
            assert rel_err(ghb.read(), h) < 1e-4, rep
        ctxt.rms_norm_matmul_quant_assign_prepared(ghb, up, gx, gprep, 1e-5)
        assert rel_err(ghb.read(), u) < 1e-4, rep
        # the stand-alone builder gives the same form
        gprep2 = GpuTensor(backend, dim + dim // 16)
        ctxt.rms_norm_prepare(gprep2, gx, gnw)
        assert rel_err(gprep2.read(), prep) < 1e-6
        gprep2.destroy()
    for o in (down, gate, up, gnw, gprep, ghb, gx, gh):
        o.destroy()


@pytest.mark.parametrize("t", [12, 14, 8], ids=lambda t: NAMES[t])
def test_wide_matrix_in_16_row_tiles_takes_several_launches(backend, oracle_lib, t):
    """More than 16384 columns in 16-row tiles (a feed-forward width like 18944): the GEMV runs as several launches over
    column slices.  Plain product, residual accumulate with the prepared copy emitted by the last slice, and bit-exact
    dequantisation of the layout."""
    import os
    if os.environ.get("SLAI_TILED") == "0":
        pytest.skip("needs the tiled layouts")
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    nrows, ncols = 272, 18944                                  # 74 super-blocks -> 19 column groups -> two launches
    ctxt = LlmContext(backend)
    raw = synth.normal_quantized(900 + t, t, nrows, ncols, 0.02)
    w = oracle_deq(oracle_lib, t, raw, nrows * ncols).reshape(nrows, ncols)
    m = GpuQuantMatrix(backend, t, nrows, ncols, raw, layout=2)
    assert np.array_equal(m.dequantize().view(np.uint32), w.view(np.uint32))
    hv = synth.normal(5, ncols, 1.0)
    ref = np.empty(nrows, np.float32)
    oracle_lib.slo_gemv(ref.ctypes.data, w.ctypes.data, hv.ctypes.data, nrows, ncols)
    gh, out = GpuTensor.vector(backend, hv), GpuTensor(backend, nrows)
    out.write(np.full(nrows, 7.0, np.float32))                 # must be overwritten, not added to
    ctxt.matmul_quant_assign(out, m, gh)
    assert rel_err(out.read(), ref) < 1e-4
    x0 = synth.normal(6, nrows, 1.0)
    nw = (1.0 + synth.normal(7, nrows, 0.1)).astype(np.float32)
    gx, gnw, gprep = GpuTensor.vector(backend, x0), GpuTensor.vector(backend, nw), GpuTensor(backend, nrows + nrows // 16)
    ctxt.matmul_quant_add_assign_emit(gx, m, gh, gnw, gprep)
    got = gx.read()
    assert rel_err(got, x0 + ref) < 1e-4
    prep = gprep.read()
    assert rel_err(prep[:nrows], got * nw) < 1e-6
    assert rel_err(prep[nrows:], (got * nw).reshape(-1, 16).sum(axis=1)) < 1e-5
    for o in (m, gh, out, gx, gnw, gprep):
        o.destroy()


@pytest.mark.parametrize("t", [12, 13, 14, 8, 2], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("shape,layout", [((202, 1024), 3), ((64, 4096), 3), ((102, 1024), 2), ((50, 1536), 2), ((42, 16640), 2)],
                         ids=["64-row-tiles-row-tail", "64-row-tiles-16-super-blocks", "16-row-tiles-row-tail", "32-row-tiles", "16-row-tiles-17-groups"])
def test_matmul_quant_columns_on_the_matrix_cores(backend, oracle_lib, t, shape, layout):
    """slai_matmul_quant_columns (the fp32 MFMA kernels under the chunked prompt pass) against the dequantised matrix
    times the vectors in float64: every format with a tiled layout, the three tile heights, row counts that end inside a
    tile and inside a group of four rows, 1 / 7 / 32 vectors, assign and accumulate."""
    check_matmul_quant_columns(backend, oracle_lib, t, shape, layout)


@pytest.fixture(scope="module")
def backend_split_ops():
    """A context created with SLAI_PROMPT_SPLIT_F16=2: slai_matmul_quant_columns takes the half-precision matrix-core
    kernels (weights and vectors as f16 head + remainder pairs) the models' prompt pass uses."""
    import os
    from slai_amd.runtime import Backend
    old = os.environ.get("SLAI_PROMPT_SPLIT_F16")
    os.environ["SLAI_PROMPT_SPLIT_F16"] = "2"
    try:
        b = Backend(0)
    finally:
        if old is None:
            del os.environ["SLAI_PROMPT_SPLIT_F16"]
        else:
            os.environ["SLAI_PROMPT_SPLIT_F16"] = old
    yield b
    b.close()


@pytest.mark.parametrize("t", [12, 13, 14, 8, 2], ids=lambda t: NAMES[t])
@pytest.mark.parametrize("shape,layout", [((202, 1024), 3), ((64, 4096), 3), ((102, 1024), 2), ((50, 1536), 2), ((42, 16640), 2)],
                         ids=["64-row-tiles-row-tail", "64-row-tiles-16-super-blocks", "16-row-tiles-row-tail", "32-row-tiles", "16-row-tiles-17-groups"])
def test_matmul_quant_columns_split_f16(backend_split_ops, oracle_lib, t, shape, layout):
    """The same bar (1e-5 of the float64 product) for the f16 head + remainder kernels: three half-precision MFMAs per
    step keep about 22 bits of every weight and of every vector element."""
    check_matmul_quant_columns(backend_split_ops, oracle_lib, t, shape, layout)


def check_matmul_quant_columns(backend, oracle_lib, t, shape, layout):
    import os
    if os.environ.get("SLAI_TILED") == "0":
        pytest.skip("needs the tiled layouts")
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    nrows, ncols = shape
    ctxt = LlmContext(backend)
    raw = synth.normal_quantized(1300 + t, t, nrows, ncols, 0.02)
    w = oracle_deq(oracle_lib, t, raw, nrows * ncols).reshape(nrows, ncols).astype(np.float64)
    m = GpuQuantMatrix(backend, t, nrows, ncols, raw, layout=layout)
    for n in (1, 7, 32):
        x = synth.normal(40 + n, ncols * n, 1.0).reshape(ncols, n)
        ref = w @ x.astype(np.float64)
        gx = GpuTensor.matrix(backend, x)
        out = GpuTensor(backend, nrows, n)
        out.write(np.full(nrows * n, 3.0, np.float32))          # must be overwritten, not added to
        ctxt.matmul_quant_columns(out, m, gx)
        got = out.read_matrix()
        assert rel_err(got, ref) < 1e-5, (n, rel_err(got, ref))
        old = synth.normal(90 + n, nrows * n, 1.0).reshape(nrows, n)
        acc = GpuTensor.matrix(backend, old)
        ctxt.matmul_quant_columns(acc, m, gx, accumulate=True)
        assert rel_err(acc.read_matrix(), old + ref) < 1e-5
        for o in (gx, out, acc):
            o.destroy()
    # error paths: too many vectors, wrong shapes
    gx = GpuTensor(backend, ncols, 33); out = GpuTensor(backend, nrows, 33)
    with pytest.raises(Exception):
        ctxt.matmul_quant_columns(out, m, gx)
    bad = GpuTensor(backend, ncols + 4, 2); out2 = GpuTensor(backend, nrows, 2)
    with pytest.raises(Exception):
        ctxt.matmul_quant_columns(out2, m, bad)
    for o in (gx, out, bad, out2):
        o.destroy()
    m.destroy()
