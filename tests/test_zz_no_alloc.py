"""slai_attention_static, the entry point that allocates nothing, against slai_attention: same kernels, the split
partials in the library's static device array instead of the context's scratch block.  Two calls in a row, the second
on a smaller input (the array keeps the first call's contents), outputs bit-identical to slai_attention's and within the
attention test's bar of the oracle; a shape whose partials exceed the array is refused."""
import numpy as np
import pytest

from slai_amd import _ffi
from slai_amd._ffi import AttnParams

pytestmark = pytest.mark.gpu


def test_attention_static_matches_attention_on_two_calls_in_a_row():
    import oracle
    from slai_amd.runtime import Backend, GpuTensor, LlmContext, SlaiError
    L = oracle.load()
    b = Backend(0)
    try:
        ctxt = LlmContext(b)
        # first: 32 heads of 128 at position 4000 of 4096 (16 splits); second, smaller: 8 query heads on 2 cache heads of
        # 64 at position 1029 of 2048
        for case, (nh, kv_mul, hs, seq, pos, f16) in enumerate(((32, 1, 128, 4096, 4000, True), (8, 4, 64, 2048, 1029, False))):
            print("case", nh, kv_mul, hs, seq, pos, f16, flush=True)
            kv_dim = nh // kv_mul * hs
            rng = np.random.Generator(np.random.PCG64(100 + case))
            q = rng.standard_normal(nh * hs, dtype=np.float32)
            kc = rng.standard_normal((seq, kv_dim), dtype=np.float32)
            vc = rng.standard_normal((seq, kv_dim), dtype=np.float32)
            if f16:
                kc = kc.astype(np.float16).astype(np.float32); vc = vc.astype(np.float16).astype(np.float32)
            att = np.zeros(seq * nh, np.float32); ref = np.empty(nh * hs, np.float32)
            L.slo_attention(nh, kv_mul, hs, pos, seq, kv_dim, q.ctypes.data, kc.ctypes.data, vc.ctypes.data, att.ctypes.data, ref.ctypes.data)
            params = AttnParams(seq, kv_dim, kv_mul, nh, hs, pos, (0, 0))
            gparams = GpuTensor.scalar(b, params)
            gq = GpuTensor.vector(b, q)
            dt, npdt = (_ffi.DT_F16, np.float16) if f16 else (_ffi.DT_F32, np.float32)
            gk = GpuTensor(b, kv_dim, seq, dt, data=kc.astype(npdt)); gv = GpuTensor(b, kv_dim, seq, dt, data=vc.astype(npdt))
            gatt = GpuTensor(b, seq, nh)
            out_a, out_s = GpuTensor(b, nh * hs), GpuTensor(b, nh * hs)
            ctxt.attention_static(params, gparams, gq, gk, gv, gatt, out_s)
            got_s = out_s.read()
            ctxt.attention(params, gparams, gq, gk, gv, gatt, out_a)
            got_a = out_a.read()
            assert np.array_equal(got_s.view(np.uint32), got_a.view(np.uint32))
            np.testing.assert_allclose(got_s, ref, rtol=2e-4, atol=2e-6)
            for o in (gparams, gq, gk, gv, gatt, out_a, out_s):
                o.destroy()
    finally:
        b.close()
    # Partial results beyond the static array: refused with a shape error, nothing launched.  The automatic choice of
    # splits never gets there (heads * splits stays below 1024); a context created with 64 splits forced does.
    import os
    os.environ["SLAI_ATTN_SPLITS"] = "64"
    try:
        b = Backend(0)
    finally:
        del os.environ["SLAI_ATTN_SPLITS"]
    try:
        ctxt = LlmContext(b)
        nh, hs, seq = 64, 128, 2048
        params = AttnParams(seq, nh * hs, 1, nh, hs, 10, (0, 0))
        gparams = GpuTensor.scalar(b, params)
        gq, gx = GpuTensor(b, nh * hs), GpuTensor(b, nh * hs)
        gk = GpuTensor(b, nh * hs, seq, _ffi.DT_F16); gv = GpuTensor(b, nh * hs, seq, _ffi.DT_F16)
        gatt = GpuTensor(b, 4)
        with pytest.raises(SlaiError) as e:
            ctxt.attention_static(params, gparams, gq, gk, gv, gatt, gx)
        assert e.value.code == _ffi.E_SHAPE and "static scratch" in str(e.value)
        ctxt.attention(params, gparams, gq, gk, gv, gatt, gx)             # the allocating entry point takes the same call
        b.synchronize()
        for o in (gparams, gq, gx, gk, gv, gatt):
            o.destroy()
    finally:
        b.close()
