"""The benchmark configurations at their stated sizes, through the C ABI.

Configuration 1 (tiny Llama, Q8_0) is test_gpu_models.py::test_tiny_llama_q8_0_config1 and configuration 2 (the GEMV
sweep shapes) is in test_gpu_quant.py::GEMV_SHAPES.  Here: configuration 3 in full against the oracle; configuration 4
and 5 at their full depth as a property check (the fused decode graph against the reference's op-by-op launch sequence of
transformer.rs:316-381 on the same device -- the oracle would need 26 GB of f32 weights), and configuration 5's
attention-heavy case at depth 2 against the oracle with both caches pre-filled with the same seeded rows.
"""
import ctypes as C

import numpy as np
import pytest

from gpu_common import backend, rel_err  # noqa: F401
from helpers import OracleGguf
from slai_amd import _ffi
from slai_amd import gguf_writer as gw

pytestmark = pytest.mark.gpu
LOGIT_TOL = 1e-2          # the task's bar for logits (max-abs error relative to the largest logit)
PROPERTY_TOL = 1e-3       # fused graph vs the op-by-op sequence on the same device: only summation order differs


def test_config3_gpt2_small_full_depth(backend):
    """GPT-2-small shape in full: dim 768, 12 layers, 12 heads, FFN 3072, vocab 50257, context 1024, N(0,0.02) weights
    in Q8_0, 32 seeded prompt ids, 256 greedy tokens -- ids identical to the oracle's, logits within the bar at the
    first, some middle and the last positions."""
    from slai_amd.runtime import Gguf, Gpt2
    data = gw.gpt2_gguf(seed=1234)
    g = OracleGguf(data); L = g.L
    L.slo_set_threads(16)
    om = L.slo_gpt2_from_gguf(g.h, 0)
    assert om
    prompt = np.random.Generator(np.random.PCG64(1234)).integers(0, 50257, 32).astype(np.int32)
    n = 32 + 256 - 1
    ref_tokens = np.zeros(n, np.int32); ref_logits = np.zeros((n, 50257), np.float32)
    print("config 3: oracle run", flush=True)
    assert L.slo_gpt2_generate(om, prompt.ctypes.data, 32, 0, n, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n
    gg = Gguf(data)
    m = Gpt2(backend, gg)
    assert (m.params.n_layer, m.params.n_embd, m.params.n_vocab) == (12, 768, 50257)
    print("config 3: device run", flush=True)
    got, _ = m.generate(prompt, n)
    assert np.array_equal(got, ref_tokens), (got.tolist(), ref_tokens.tolist())
    # the caches now hold the whole run: the logits of any position can be recomputed in place
    for pos in (0, 1, 31, 32, 100, 200, n - 1):
        tok = int(prompt[pos]) if pos < 32 else int(ref_tokens[pos - 1])
        err = rel_err(m.forward_logits(pos, tok), ref_logits[pos])
        assert err < LOGIT_TOL, (pos, err)
    m.destroy(); gg.close(); L.slo_gpt2_free(om); g.close()


def fused_vs_op_sequence(backend, data, prompt, n_steps, kv_fill=None, start_pos=0):
    """One model instance runs the captured decode graph for n_steps greedy tokens; a second one runs the reference's
    launch sequence (`fused=0`: one kernel per op of transformer.rs:316-381) on the tokens the first one chose.  Ids
    must be identical and the logits of every step within PROPERTY_TOL; the fused single-token entry point is checked on
    the way."""
    from slai_amd.runtime import Gguf, Llama2
    gg = Gguf(data)
    a = Llama2(backend, gg, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    b = Llama2(backend, gg, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    if kv_fill is not None:
        for l in range(a.config.n_layers):
            k, v = kv_fill(l)
            a.write_kv(l, k, v); b.write_kv(l, k, v)
    prompt = np.asarray(prompt, np.int32)
    seq = np.zeros(start_pos + prompt.size, np.int32)
    seq[start_pos:] = prompt
    got, ms = a.generate(seq, n_steps, start_pos=start_pos)
    tok = int(prompt[0])
    worst = 0.0
    for i in range(n_steps):
        pos = start_pos + i
        ref = b.forward_logits(pos, tok, fused=False)
        nxt = int(prompt[i + 1]) if i < prompt.size - 1 else int(np.argmax(ref))
        assert nxt == int(got[i]), (i, nxt, int(got[i]))
        if i % 8 == 0:                                     # the fused kernels one token at a time, at this position of a's cache
            err = rel_err(a.forward_logits(pos, tok, fused=True), ref)
            worst = max(worst, err)
            assert err < PROPERTY_TOL, (i, err)
        tok = nxt
    a.destroy(); b.destroy(); gg.close()
    return worst, ms / n_steps


CONFIG4_PROMPT, CONFIG4_TOKENS = 64, 256     # "Prompt is 64 seeded token ids; greedy decode of 256 tokens"


def backend_of_form(resident):
    """A context whose Llama-2 models take the resident launch where their shapes allow it (the default), or never."""
    import os
    from slai_amd.runtime import Backend
    os.environ["SLAI_PERSISTENT"] = "1" if resident else "0"
    try:
        return Backend(0)
    finally:
        del os.environ["SLAI_PERSISTENT"]


def took_the_launches_the_metric_is_quoted_on(m, pos, token, resident):
    """Whether the model's decode sequence is the one the headline figure is quoted on: the whole layer stack in one
    resident launch per token (`llama_decode_persistent_kernel`), or, with that form switched off, q/k/v + attention as one
    launch per layer (`qkv_attention_kernel`).  slai_llama2_time_steps names every launch of a token."""
    names = [s[0] for s in m.time_steps(pos, token, reps=1)]
    if resident:
        return m.decode_form() == 1 and "llama2 resident token" in names and not any("attention" in n or "qkv" in n for n in names)
    return m.decode_form() == 0 and "llama2 qkv + attention" in names and "llama2 attention" not in names and "llama2 qkv" not in names


@pytest.mark.parametrize("resident", [True, False], ids=["one resident launch per token", "one launch per step"])
def test_config4_depth2_vs_oracle_at_the_metric_positions(resident):
    """Configuration 4's layer shapes (dim 4096, 32 heads of 128, FFN 11008, vocab 32000, Q4_K with Q6_K v-proj and output,
    fp16 cache) at depth 2 against the oracle over ALL the positions the metric is quoted on: 64 seeded prompt ids + 256
    greedy tokens = positions 0 .. 319, which takes the attention through its second and third pass over the cache (128
    positions per pass), in both launch forms.  Ids identical (chat_llama2.rs:105-158 loop, cpu.rs:488-539 attention);
    logits within the bar at the pass boundaries and at both ends, through the fused kernels one token at a time."""
    from slai_amd.runtime import Gguf, Llama2
    data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=2, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=512, wtype=12, v_type=14,
                         out_type=14, embd_type=12, seed=4242)
    g = OracleGguf(data); L = g.L
    L.slo_set_threads(16)
    om = L.slo_llama2_from_gguf(g.h, b"llama", 1, 0, 1)
    assert om
    prompt = np.random.Generator(np.random.PCG64(4242)).integers(0, 32000, CONFIG4_PROMPT).astype(np.int32)
    n = CONFIG4_PROMPT + CONFIG4_TOKENS
    ref_tokens = np.zeros(n, np.int32); ref_logits = np.zeros((n, 32000), np.float32)
    print("config 4 depth 2: oracle run", flush=True)
    assert L.slo_llama2_generate(om, prompt.ctypes.data, prompt.size, 0, n, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n
    backend = backend_of_form(resident)
    try:
        gg = Gguf(data)
        m = Llama2(backend, gg, _ffi.MODEL_LLAMA, _ffi.KV_F16)
        assert m.decode_form() == int(resident)
        print("config 4 depth 2: device run", flush=True)
        got, _ = m.generate(prompt, n)
        assert np.array_equal(got, ref_tokens), (np.flatnonzero(got != ref_tokens)[:4].tolist(), got.tolist(), ref_tokens.tolist())
        assert took_the_launches_the_metric_is_quoted_on(m, 5, int(prompt[5]), resident)
        # the caches hold the whole run: the logits of any position can be recomputed in place
        worst = 0.0
        for pos in (0, 1, 63, 64, 126, 127, 128, 129, 191, 192, 255, 256, 257, 318, 319):
            tok = int(prompt[pos]) if pos < CONFIG4_PROMPT else int(ref_tokens[pos - 1])
            for fused in (True, False):
                err = rel_err(m.forward_logits(pos, tok, fused=fused), ref_logits[pos])
                worst = max(worst, err)
                assert err < LOGIT_TOL, (pos, fused, err)
        print("config 4 depth 2, positions 0..319: worst logits rel err %.2e" % worst)
        m.destroy(); gg.close()
    finally:
        backend.close()
    L.slo_llama2_free(om); g.close()


@pytest.mark.parametrize("resident", [True, False], ids=["one resident launch per token", "one launch per step"])
def test_config4_llama7b_q4k_full_depth(resident):
    """Llama-2-7B shape at its full 32 layers (Q4_K, Q6_K v-proj / output, fp16 cache, context 512) over the metric's own
    run: 64 prompt ids + 256 greedy tokens (positions 0 .. 319) from the decode loop equal those of the op-by-op
    sequence, and the loop is made of the launches the headline figure is quoted on, in both launch forms."""
    from slai_amd.runtime import Gguf, Llama2
    data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=32, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=512, wtype=12, v_type=14,
                         out_type=14, embd_type=12, seed=1234, distinct_layers=4)
    prompt = np.random.Generator(np.random.PCG64(1234)).integers(0, 32000, CONFIG4_PROMPT)
    backend = backend_of_form(resident)
    try:
        gg = Gguf(data)
        probe = Llama2(backend, gg, _ffi.MODEL_LLAMA, _ffi.KV_F16)
        assert took_the_launches_the_metric_is_quoted_on(probe, 0, int(prompt[0]), resident)
        probe.destroy(); gg.close()
        worst, ms = fused_vs_op_sequence(backend, data, prompt, CONFIG4_PROMPT + CONFIG4_TOKENS)
        print("config 4 at 32 layers, positions 0..319: worst logits rel err %.2e, %.3f ms/token" % (worst, ms))
    finally:
        backend.close()


def seeded_kv(seed, layer, n_pos, kv_dim):
    rng = np.random.Generator(np.random.PCG64(seed * 1000 + layer))
    k = rng.standard_normal((n_pos, kv_dim), dtype=np.float32)
    v = rng.standard_normal((n_pos, kv_dim), dtype=np.float32)
    return k, v


def test_config5_long_context_depth2_vs_oracle(backend):
    """The attention-heavy configuration at depth 2 against the oracle: 7B layer shapes, Q8_0, fp16 cache pre-filled to
    4000 positions with seeded N(0,1) rows on both sides, 96 tokens decoded up to the 4096th position."""
    from slai_amd.runtime import Gguf, Llama2
    data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=2, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=4096, wtype=8, seed=55)
    g = OracleGguf(data); L = g.L
    L.slo_set_threads(16)
    om = L.slo_llama2_from_gguf(g.h, b"llama", 1, 0, 1)
    assert om
    gg = Gguf(data)
    m = Llama2(backend, gg, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    for l in range(2):
        k, v = seeded_kv(5, l, 4000, 4096)
        L.slo_llama2_fill_kv(om, l, 4000, k.ctypes.data, v.ctypes.data)        # rounds to f16 like the device cache
        m.write_kv(l, k.astype(np.float16), v.astype(np.float16))
    n = 96
    first = 17
    seq = np.zeros(4001, np.int32); seq[4000] = first
    ref_tokens = np.zeros(n, np.int32); ref_logits = np.zeros((n, 32000), np.float32)
    print("config 5 depth 2: oracle run", flush=True)
    assert L.slo_llama2_generate(om, seq.ctypes.data, seq.size, 4000, n, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n
    print("config 5 depth 2: device run", flush=True)
    got, _ = m.generate(seq, n, start_pos=4000)
    assert np.array_equal(got, ref_tokens), (got.tolist(), ref_tokens.tolist())
    for i in (0, 1, 47, 95):
        tok = first if i == 0 else int(ref_tokens[i - 1])
        for fused in (True, False):
            err = rel_err(m.forward_logits(4000 + i, tok, fused=fused), ref_logits[i])
            assert err < LOGIT_TOL, (i, fused, err)
    m.destroy(); gg.close(); L.slo_llama2_free(om); g.close()


def test_config5_long_context_full_depth(backend):
    """Configuration 5 at its full 32 layers (Q8_0, fp16 cache pre-filled to 4000 positions): 32 tokens from position
    4000 on, decode graph against the op-by-op sequence."""
    data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=32, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=4096, wtype=8, seed=56,
                         distinct_layers=2)

    def fill(l):
        k, v = seeded_kv(6, l % 4, 4000, 4096)
        return k.astype(np.float16), v.astype(np.float16)
    worst, ms = fused_vs_op_sequence(backend, data, [23], 32, kv_fill=fill, start_pos=4000)
    print("config 5 at 32 layers: worst logits rel err %.2e, %.3f ms/token" % (worst, ms))
