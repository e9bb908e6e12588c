"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
and fails loudly (no fallback) when no GPU is present.  No compute calls."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from helpers import GOLDEN
from slai_amd import _ffi, build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    if not os.path.exists(build.HIP_LIB):
        build.build_hip()
    return _ffi.lib()


def test_exports_every_declared_symbol(L):
    header = open(os.path.join(ROOT, "include", "slai_hip.h")).read()
    declared = set(re.findall(r"\b(slai_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 60
    assert declared == set(_ffi.SIGNATURES)
    for name in declared:
        assert hasattr(L, name), name


def test_struct_layouts_match_reference_uniforms():
    assert C.sizeof(_ffi.RmsNormConfig) == 16      # ops/rms_norm.rs:15-21
    assert C.sizeof(_ffi.RopeConfig) == 16         # ops/rope.rs:24-33
    assert C.sizeof(_ffi.AttnParams) == 32         # ops/batched_multiquery_attention.rs:17-29
    assert _ffi.AttnParams.pos.offset == 20
    assert C.sizeof(_ffi.View) == 48


def test_gguf_parser_on_reference_fixture(L):
    """Host-side GGUF parser (no GPU needed) against assets/gguf/dummy.gguf of the reference."""
    from slai_amd.runtime import Gguf, SlaiError
    data = np.fromfile(os.path.join(GOLDEN, "dummy.gguf"), dtype=np.uint8)
    g = Gguf(data)
    assert g.version == 3
    assert L.slai_gguf_tensor_count(g.h) == 10 and L.slai_gguf_metadata_count(g.h) == 15
    assert L.slai_gguf_data_start(g.h) == 1216
    t = g.tensors()
    assert t["tensor_0"] == dict(dims=[8, 7, 6, 4], type=0, offset=1216)
    assert t["tensor_4"]["dims"] == [1, 2, 1, 1]
    assert g.meta_u32("some.parameter.uint32") == 0x12345678
    assert abs(g.meta_f32("some.parameter.float32") - 0.123456789) < 1e-8
    assert g.meta_str("some.parameter.string") == "hello world"
    assert g.meta_array_len("some.parameter.arr.str") == 3
    with pytest.raises(SlaiError) as e:
        g.meta_u32("some.parameter.uint8")          # unwrap_u32 on a U8: wrong type (gguf.rs:284-290)
    assert e.value.code == _ffi.E_TYPE
    with pytest.raises(SlaiError) as e:
        g.meta_u32("nope")
    assert e.value.code == _ffi.E_MISSING
    g.close()
    bad = data.copy(); bad[0] = 0
    with pytest.raises(SlaiError) as e:
        Gguf(bad)
    assert e.value.code == _ffi.E_PARSE and "magic number" in str(e.value)
    for cut in (10, 600, 11000):
        with pytest.raises(SlaiError) as e:
            Gguf(data[:cut])
        assert e.value.code == _ffi.E_PARSE


def test_gguf_parser_agrees_with_oracle_on_synthetic_model(L):
    from helpers import OracleGguf
    from slai_amd import gguf_writer as gw
    from slai_amd.runtime import Gguf
    data = gw.llama_gguf(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab=64, seq_len=8, wtype=12, v_type=14, out_type=14)
    g, o = Gguf(data), OracleGguf(data)
    mine = g.tensors()
    assert set(mine) == set(o.tensors)
    for k, v in mine.items():
        assert v["dims"] == o.tensors[k]["dims"] and v["type"] == o.tensors[k]["type"] and v["offset"] == o.tensors[k]["offset"]
    assert g.meta_u32("llama.embedding_length") == 256 and g.meta_array_len("tokenizer.ggml.tokens") == 64
    g.close(); o.close()


def test_no_gpu_is_an_error_not_a_fallback(L):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    assert L.slai_ctx_create(0, C.byref(h)) == _ffi.E_HIP
    assert not h.value
