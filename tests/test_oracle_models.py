"""Whole-forward checks of the C oracle against the independent numpy twin."""
import numpy as np

from helpers import OracleGguf
from oracle import np_oracle
from slai_amd import gguf_writer as gw


def test_llama_forward_c_vs_numpy_twin():
    data = gw.llama_gguf(dim=64, hidden_dim=160, n_layers=3, n_heads=4, n_kv_heads=2, vocab=300, seq_len=24,
                         wtype=8, seed=5, std=0.08, norm_random=True, out_type=14 if False else 8)
    g = OracleGguf(data)
    L = g.L
    m = L.slo_llama2_from_gguf(g.h, b"llama", 0, 0, 0)
    assert m
    cfg = dict(dim=64, hidden_dim=160, n_layers=3, n_heads=4, n_kv_heads=2, vocab=300, seq_len=24)
    twin = np_oracle.NpLlama(cfg, g.np_tensors())
    toks = [5, 17, 200, 3, 3, 250, 9, 0]
    for pos, tok in enumerate(toks):
        L.slo_llama2_forward(m, tok, pos)
        got = np.ctypeslib.as_array(L.slo_llama2_logits(m), (300,)).copy()
        ref = twin.forward(tok, pos)
        scale = np.abs(ref).max()
        assert np.abs(got - ref).max() / scale < 2e-5, (pos, np.abs(got - ref).max() / scale)
        assert int(np.argmax(got)) == int(np.argmax(ref))
    L.slo_llama2_free(m)
    g.close()


def test_llama_kquant_model_and_f16_kv():
    data = gw.llama_gguf(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=4, vocab=128, seq_len=16,
                         wtype=12, v_type=14, out_type=14, embd_type=12, seed=6, std=0.05)
    g = OracleGguf(data)
    L = g.L
    cfg = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=4, vocab=128, seq_len=16)
    twin = np_oracle.NpLlama(cfg, g.np_tensors())
    m32 = L.slo_llama2_from_gguf(g.h, b"llama", 1, 0, 0)
    m16 = L.slo_llama2_from_gguf(g.h, b"llama", 1, 0, 1)
    for pos, tok in enumerate([1, 2, 3, 4, 5]):
        L.slo_llama2_forward(m32, tok, pos); L.slo_llama2_forward(m16, tok, pos)
        a = np.ctypeslib.as_array(L.slo_llama2_logits(m32), (128,)).copy()
        b = np.ctypeslib.as_array(L.slo_llama2_logits(m16), (128,)).copy()
        ref = twin.forward(tok, pos)
        s = np.abs(ref).max()
        assert np.abs(a - ref).max() / s < 2e-5
        assert np.abs(b - ref).max() / s < 5e-3      # fp16 K/V rounding only
        if pos > 0:
            assert not np.array_equal(a, b)
    L.slo_llama2_free(m32); L.slo_llama2_free(m16); g.close()


def test_generate_forced_prompt_then_greedy():
    data = gw.llama_gguf(dim=64, hidden_dim=160, n_layers=2, n_heads=4, n_kv_heads=4, vocab=300, seq_len=32,
                         wtype=8, seed=7, std=0.1)
    g = OracleGguf(data); L = g.L
    m = L.slo_llama2_from_gguf(g.h, b"llama", 0, 0, 0)
    prompt = np.array([4, 8, 15, 16, 23], np.int32)
    out = np.zeros(12, np.int32); logits = np.zeros((12, 300), np.float32)
    n = L.slo_llama2_generate(m, prompt.ctypes.data, 5, 0, 12, -1, out.ctypes.data, logits.ctypes.data)
    assert n == 12
    assert out[:4].tolist() == [8, 15, 16, 23]                     # forced while pos < len-1
    assert out[4:].tolist() == np.argmax(logits[4:], axis=1).tolist()
    L.slo_llama2_free(m); g.close()


def test_gpt2_forward_c_vs_numpy_twin():
    data = gw.gpt2_gguf(n_embd=64, n_layer=2, n_head=4, ff_len=256, vocab=301, n_seq=16, seed=8, std=0.08)
    g = OracleGguf(data); L = g.L
    m = L.slo_gpt2_from_gguf(g.h, 0)
    assert m
    twin = np_oracle.NpGpt2(dict(n_embd=64, n_layer=2, n_head=4, n_seq=16), g.np_tensors())
    for pos, tok in enumerate([3, 300, 7, 7, 100]):
        L.slo_gpt2_forward(m, tok, pos)
        got = np.ctypeslib.as_array(L.slo_gpt2_logits(m), (301,)).copy()
        ref = twin.forward(tok, pos)
        assert np.abs(got - ref).max() / np.abs(ref).max() < 2e-5
    L.slo_gpt2_free(m); g.close()
