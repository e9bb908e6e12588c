"""GPU parity of the LlmContext ops against the oracle.  LEN 1757 and the tolerances follow the
reference's own op tests (ops/silu.rs:97-131 1e-5, ops/softmax.rs:98-131 1e-7, ops/rope.rs:160-228
1e-5, ops/rms_norm.rs:117-168 1e-4, ops/layernorm.rs:150-190 1e-5, ops/unary.rs:293-408 1e-5)."""
import numpy as np
import pytest

from gpu_common import backend, rel_err  # noqa: F401
from slai_amd import _ffi
from slai_amd._ffi import AttnParams, RmsNormConfig, RopeConfig

pytestmark = pytest.mark.gpu
LEN = 1757


def rnd(seed, n, scale=1.0):
    return np.random.Generator(np.random.PCG64(seed)).normal(0, scale, n).astype(np.float32)


def uni(seed, n):
    return np.random.Generator(np.random.PCG64(seed)).random(n, dtype=np.float32)   # DVector::new_random: U[0,1)


def test_rms_norm(backend, oracle_lib):
    from slai_amd.runtime import GpuTensor, LlmContext
    for n, eps in ((LEN, 1e-5), (4096, 1e-6), (288, 1e-5)):
        v, w = uni(1, n), uni(2, n)
        ref = np.empty(n, np.float32)
        oracle_lib.slo_rms_norm(ref.ctypes.data, v.ctypes.data, w.ctypes.data, n, eps)
        cfg = GpuTensor.scalar(backend, RmsNormConfig(eps, (0, 0, 0)))
        gv, gw, go = GpuTensor.vector(backend, v), GpuTensor.vector(backend, w), GpuTensor(backend, n)
        LlmContext(backend).rms_norm_assign(cfg, go, gv, gw)
        np.testing.assert_allclose(go.read(), ref, rtol=1e-4, atol=1e-6)
        for o in (cfg, gv, gw, go):
            o.destroy()


def test_layernorm_and_gelu_and_silu(backend, oracle_lib):
    from slai_amd.runtime import GpuTensor, LlmContext
    ctxt = LlmContext(backend)
    v = rnd(3, LEN, 2.0)
    ref = np.empty(LEN, np.float32)
    oracle_lib.slo_layernorm(ref.ctypes.data, v.ctypes.data, LEN, 1e-5)
    gv, go = GpuTensor.vector(backend, v), GpuTensor(backend, LEN)
    ctxt.layernorm_assign(go, gv, 1e-5)
    np.testing.assert_allclose(go.read(), ref, rtol=1e-5, atol=1e-6)
    g = v.copy(); oracle_lib.slo_gelu_n(g.ctypes.data, LEN)
    ctxt.gelu_inplace(gv)
    np.testing.assert_allclose(gv.read(), g, rtol=1e-5, atol=1e-6)
    a, b = rnd(4, LEN, 3.0), rnd(5, LEN)
    r = a.copy(); oracle_lib.slo_silu(r.ctypes.data, b.ctypes.data, LEN)
    ga, gb = GpuTensor.vector(backend, a), GpuTensor.vector(backend, b)
    ctxt.silu(ga, gb)
    np.testing.assert_allclose(ga.read(), r, rtol=1e-5, atol=1e-7)
    for o in (gv, go, ga, gb):
        o.destroy()


def test_add_mul_copy(backend):
    from slai_amd.runtime import GpuTensor, LlmContext
    ctxt = LlmContext(backend)
    a, b = rnd(6, LEN), rnd(7, LEN)
    ga, gb, gc = GpuTensor.vector(backend, a), GpuTensor.vector(backend, b), GpuTensor(backend, LEN)
    ctxt.add_assign(ga, gb)
    assert np.array_equal(ga.read(), a + b)
    ctxt.mul_assign(ga, gb)
    assert np.array_equal(ga.read(), (a + b) * b)
    ctxt.copy(gb, gc)
    assert np.array_equal(gc.read(), b)
    # a strided / offset destination: column 2 of a [LEN x 4] matrix
    gm = GpuTensor(backend, LEN, 4)
    ctxt.copy(gb, gm.column(2))
    m = gm.read_matrix()
    assert np.array_equal(m[:, 2], b) and not m[:, [0, 1, 3]].any()
    for o in (ga, gb, gc, gm):
        o.destroy()


@pytest.mark.parametrize("variant", [_ffi.ROPE_ORIGINAL, _ffi.ROPE_NEOX])
def test_rope(backend, oracle_lib, variant):
    from slai_amd.runtime import GpuTensor, LlmContext
    hs, nq, nk, pos = 128, 13, 9, 10                       # ops/rope.rs:160-170
    dim, kv_dim = hs * nq, hs * nk
    q, k = uni(8, dim), uni(9, kv_dim)
    rq, rk = q.copy(), k.copy()
    oracle_lib.slo_rope(rq.ctypes.data, rk.ctypes.data, hs, dim, kv_dim, pos, 10000.0, variant)
    cfg = GpuTensor.scalar(backend, RopeConfig(hs, kv_dim, pos, 10000.0))
    gq, gk = GpuTensor.vector(backend, q), GpuTensor.vector(backend, k)
    LlmContext(backend).rope(variant, cfg, gq, gk)
    np.testing.assert_allclose(gq.read(), rq, rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(gk.read(), rk, rtol=1e-5, atol=2e-6)
    for o in (cfg, gq, gk):
        o.destroy()


def test_softmax_cols(backend, oracle_lib):
    from slai_amd.runtime import GpuTensor, LlmContext
    m = rnd(10, LEN * 5, 3.0).reshape(LEN, 5)
    ref = m.copy()
    for j in range(5):
        col = np.ascontiguousarray(ref[:, j]); oracle_lib.slo_softmax(col.ctypes.data, LEN); ref[:, j] = col
    gm = GpuTensor.matrix(backend, m)
    LlmContext(backend).softmax_cols(gm)
    np.testing.assert_allclose(gm.read_matrix(), ref, rtol=2e-6, atol=1e-7)
    gm.destroy()


def test_argmax_first_maximum(backend):
    from slai_amd.runtime import GpuTensor, LlmContext
    ctxt = LlmContext(backend)
    idx = GpuTensor(backend, 1, 1, _ffi.DT_I32)
    for n, seed in ((32000, 1), (50257, 2), (7, 3)):
        v = rnd(seed, n)
        gv = GpuTensor.vector(backend, v)
        ctxt.argmax(gv, idx)
        assert int(idx.read()[0]) == int(np.argmax(v))
        gv.destroy()
    v = np.zeros(5000, np.float32); v[[4000, 17, 2999]] = 3.0
    gv = GpuTensor.vector(backend, v)
    ctxt.argmax(gv, idx)
    assert int(idx.read()[0]) == 17
    gv.destroy(); idx.destroy()


@pytest.mark.parametrize("cfg", [dict(n_heads=6, kv_mul=1, hs=48, seq=256, pos=37),
                                 dict(n_heads=12, kv_mul=3, hs=64, seq=96, pos=95),
                                 dict(n_heads=32, kv_mul=1, hs=128, seq=512, pos=300),
                                 dict(n_heads=8, kv_mul=2, hs=128, seq=64, pos=0),
                                 # long contexts take the split (flash-decoding) form with a combine pass
                                 dict(n_heads=32, kv_mul=1, hs=128, seq=4096, pos=4000),
                                 dict(n_heads=8, kv_mul=4, hs=64, seq=2048, pos=1029),
                                 # grouped-query shapes whose workgroups are laid out by (kv head, split) over the dies: a
                                 # Qwen2-7B layer (28 / 4) split and unsplit, and a key count that does not fill the dies
                                 dict(n_heads=28, kv_mul=7, hs=128, seq=4096, pos=4047),
                                 dict(n_heads=28, kv_mul=7, hs=128, seq=512, pos=200),
                                 dict(n_heads=24, kv_mul=2, hs=64, seq=3072, pos=2500),
                                 dict(n_heads=6, kv_mul=1, hs=48, seq=1536, pos=700),
                                 dict(n_heads=4, kv_mul=1, hs=128, seq=2048, pos=5)])
@pytest.mark.parametrize("f16", [False, True])
def test_attention_fused_and_reference_sequence(backend, oracle_lib, cfg, f16):
    """`BatchedMultiqueryAttention::launch`: the fused op and the reference's own four-launch
    sequence (ops/batched_multiquery_attention.rs:46-98) both against `run_cpu` (:102-156)."""
    from slai_amd.runtime import GpuTensor, LlmContext
    nh, kv_mul, hs, seq, pos = cfg["n_heads"], cfg["kv_mul"], cfg["hs"], cfg["seq"], cfg["pos"]
    print("case", cfg, f16, flush=True)
    nkv = nh // kv_mul
    kv_dim = nkv * hs
    q = rnd(11, nh * hs)
    kc = rnd(12, seq * kv_dim).reshape(seq, kv_dim); vc = rnd(13, seq * kv_dim).reshape(seq, kv_dim)
    if f16:
        kc = kc.astype(np.float16).astype(np.float32); vc = vc.astype(np.float16).astype(np.float32)
    att = np.zeros(seq * nh, np.float32); ref = np.empty(nh * hs, np.float32)
    oracle_lib.slo_attention(nh, kv_mul, hs, pos, seq, kv_dim, q.ctypes.data, kc.ctypes.data, vc.ctypes.data, att.ctypes.data, ref.ctypes.data)
    ctxt = LlmContext(backend)
    params = AttnParams(seq, kv_dim, kv_mul, nh, hs, pos, (0, 0))
    gparams = GpuTensor.scalar(backend, params)
    gq = GpuTensor.vector(backend, q)
    dt = _ffi.DT_F16 if f16 else _ffi.DT_F32
    npdt = np.float16 if f16 else np.float32
    gk = GpuTensor(backend, kv_dim, seq, dt, data=kc.astype(npdt)); gv = GpuTensor(backend, kv_dim, seq, dt, data=vc.astype(npdt))
    gatt = GpuTensor(backend, seq, nh); gxb = GpuTensor(backend, nh * hs)
    ctxt.attention(params, gparams, gq, gk, gv, gatt, gxb)
    got = gxb.read()
    np.testing.assert_allclose(got, ref, rtol=2e-4, atol=2e-6)
    if not f16:
        # the reference's sequence with its padded views
        rp = (pos + 1 + 3) // 4 * 4
        if rp <= seq:
            gxb2 = GpuTensor(backend, nh * hs)
            k_view = gk.view(0, (hs, rp, nkv, 1), (1, kv_dim, hs, hs * nkv))
            q_view = gq.view(0, (hs, kv_mul, nkv, 1), (1, hs, hs * kv_mul, hs * nh))
            att_view = gatt.view(0, (rp, kv_mul, nkv, 1), (1, rp, rp * kv_mul, rp * nh))
            ctxt.matmul_assign(att_view, k_view, q_view, _ffi.MODE_T, _ffi.MODE_N)
            ctxt.attn_mask(params, gparams, gatt)
            ctxt.softmax_cols(gatt.view(0, (pos + 1, nh, 1, 1), (1, rp, rp * nh, rp * nh)))
            v_view = gv.view(0, (hs, rp, nkv, 1), (1, kv_dim, hs, hs * nkv))
            xb_view = gxb2.view(0, (hs, kv_mul, nkv, 1), (1, hs, hs * kv_mul, hs * nh))
            ctxt.matmul_assign(xb_view, v_view, att_view, _ffi.MODE_N, _ffi.MODE_N)
            np.testing.assert_allclose(gxb2.read(), ref, rtol=2e-4, atol=2e-6)
            probs = gatt.read()[:rp * nh].reshape(nh, rp)
            np.testing.assert_allclose(probs[:, :pos + 1], att.reshape(nh, seq)[:, :pos + 1], rtol=2e-4, atol=1e-7)
            assert not probs[:, pos + 1:].any()
            gxb2.destroy()
    for o in (gparams, gq, gk, gv, gatt, gxb):
        o.destroy()


def test_submission_bracket_and_graph_replay_of_an_op_sequence(backend, oracle_lib):
    """`LlmContext::begin_submission` / `submit` (context.rs:79-95) around op-level launches, eagerly and captured into
    a graph that is replayed several times with eager work and synchronisations in between; every replay must
    reproduce the eager result, which must be the oracle's.  The sequence is a feed-forward block: RMSNorm, gate and up
    projections, SiLU, down projection, residual add (transformer.rs:356-365)."""
    from slai_amd import synth
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext, TensorCache
    dim, hid, t = 512, 1536, 12
    ctxt = LlmContext(backend)
    cache = TensorCache(backend)
    x0 = rnd(1, dim)
    w = (1.0 + 0.1 * rnd(2, dim)).astype(np.float32)
    raws = [synth.normal_quantized(40 + i, t, r, c, 0.05) for i, (r, c) in enumerate(((hid, dim), (hid, dim), (dim, hid)))]
    shapes = ((hid, dim), (hid, dim), (dim, hid))
    deq = []
    for raw, (r, c) in zip(raws, shapes):
        a = np.empty(r * c, np.float32)
        assert oracle_lib.slo_dequantize(t, raw.ctypes.data, r * c, a.ctypes.data) == 0
        deq.append(a.reshape(r, c))
    # oracle: ops of cpu.rs:340-376,555-560 in the same order
    xb = np.empty(dim, np.float32); oracle_lib.slo_rms_norm(xb.ctypes.data, x0.ctypes.data, w.ctypes.data, dim, 1e-5)
    hb = np.empty(hid, np.float32); hb2 = np.empty(hid, np.float32)
    oracle_lib.slo_gemv(hb.ctypes.data, deq[0].ctypes.data, xb.ctypes.data, hid, dim)
    oracle_lib.slo_gemv(hb2.ctypes.data, deq[1].ctypes.data, xb.ctypes.data, hid, dim)
    oracle_lib.slo_silu(hb.ctypes.data, hb2.ctypes.data, hid)
    xb2 = np.empty(dim, np.float32)
    oracle_lib.slo_gemv(xb2.ctypes.data, deq[2].ctypes.data, hb.ctypes.data, dim, hid)
    ref = x0 + xb2

    gate, up, down = [GpuQuantMatrix(backend, t, r, c, raw) for raw, (r, c) in zip(raws, shapes)]
    gx0 = GpuTensor.vector(backend, x0)
    gw = GpuTensor.vector(backend, w)
    cfg = GpuTensor.scalar(backend, _ffi.RmsNormConfig(1e-5, (0, 0, 0)))
    gx = GpuTensor(backend, dim)
    # the temporaries come from the cache, as they do behind the reference's LlmContext
    gxb, gxb2 = cache.get_or_insert(dim), cache.get_or_insert(dim)
    ghb, ghb2 = cache.get_or_insert(hid), cache.get_or_insert(hid)
    assert cache.idle() == 0

    def block():
        ctxt.begin_submission()
        ctxt.copy(gx0, gx)
        ctxt.rms_norm_assign(cfg, gxb, gx, gw)
        ctxt.matmul_quant_assign(ghb, gate, gxb)
        ctxt.matmul_quant_assign(ghb2, up, gxb)
        ctxt.silu(ghb, ghb2)
        ctxt.matmul_quant_assign(gxb2, down, ghb)
        ctxt.add_assign(gx, gxb2)
        ctxt.submit()

    block()
    backend.synchronize()
    eager = gx.read()
    assert rel_err(eager, ref) < 1e-4
    ctxt.begin_submission(); ctxt.begin_submission(); ctxt.submit(); ctxt.submit()     # re-begin submits; a second submit is a no-op
    backend.graph_begin_capture()
    block()
    g = backend.graph_end_capture()
    for rep in range(4):
        gx.write(np.full(dim, float(rep), np.float32))       # eager work between the replays: the graph must overwrite it
        ghb.write(np.zeros(hid, np.float32))
        backend.synchronize()
        backend.graph_launch(g)
        backend.synchronize()
        assert np.array_equal(gx.read().view(np.uint32), eager.view(np.uint32)), rep
    backend.graph_destroy(g)
    # back into the pool, out again: the same buffers, no new allocation; clear frees the idle ones
    for tns in (gxb, gxb2, ghb, ghb2):
        cache.reclaim(tns)
    assert cache.idle() == 4
    again = cache.get_or_insert(hid)
    assert cache.idle() == 3
    assert again.read().shape == (hid,)                                                  # contents are the last holder's
    other = cache.get_or_insert(hid, 2)                                                  # another shape: a miss, a new zeroed buffer
    assert cache.idle() == 3 and not other.read().any()
    handle = again.h
    cache.reclaim(again); cache.reclaim(other)
    assert backend.L.slai_tensor_cache_reclaim(backend.h, cache.h, handle) != 0        # already back: refused, not pooled twice
    assert cache.idle() == 5
    with pytest.raises(Exception):
        cache.get_or_insert(0)                                                           # a dimension of size zero
    cache.clear()
    assert cache.idle() == 0
    cache.destroy()
    for o in (gate, up, down, gx0, gw, cfg, gx):
        o.destroy()


def test_tensor_cache_lifetime_rules(backend):
    """What keeps a pooled tensor's memory valid: an idle tensor cannot be destroyed behind its cache's back; a tensor
    handed out during a graph capture is retired, not freed, by `clear` (the graph that names it replays correctly
    afterwards); `clear` is refused inside a capture; destroying a cache inside a capture leaves the capture running."""
    import ctypes as C
    from slai_amd.runtime import GpuTensor, LlmContext, TensorCache
    ctxt = LlmContext(backend)
    cache = TensorCache(backend)
    n = 4096
    t = cache.get_or_insert(n)
    handle = t.h
    cache.reclaim(t)
    backend.L.slai_buffer_destroy(backend.h, handle)                      # refused: the cache still lists it
    assert b"idle in a tensor cache" in backend.L.slai_last_error(backend.h)
    assert cache.idle() == 1
    src = GpuTensor.vector(backend, rnd(11, n))
    dst = GpuTensor(backend, n)
    backend.graph_begin_capture()
    tmp = cache.get_or_insert(n)                                          # a hit: legal inside a capture
    assert tmp.h.value == handle.value
    ctxt.copy(src, tmp)
    ctxt.copy(tmp, dst)
    assert backend.L.slai_tensor_cache_clear(backend.h, cache.h) == _ffi.E_STATE
    side = TensorCache(backend)
    side.destroy()                                                        # nothing synchronised, the capture goes on
    g = backend.graph_end_capture()
    cache.reclaim(tmp)
    cache.clear()                                                         # the graph still names tmp: retired, not freed
    assert cache.idle() == 0
    junk = [GpuTensor.vector(backend, np.full(n, 7.0, np.float32)) for _ in range(8)]   # would land on freed memory
    for rep in range(3):
        vals = rnd(20 + rep, n)
        src.write(vals)
        dst.write(np.zeros(n, np.float32))
        backend.synchronize()
        backend.graph_launch(g)
        backend.synchronize()
        assert np.array_equal(dst.read(), vals), rep
        assert all(np.all(j.read() == 7.0) for j in junk)
    backend.graph_destroy(g)
    cache.destroy()
    for o in junk + [src, dst]:
        o.destroy()
