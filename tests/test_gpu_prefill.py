"""Prompt tokens in chunks (slai_llama2_prefill) against the oracle and against the token-by-token device loop.

Three paths, picked by the model's layouts (Llama2.prefill_path): 2 = fp32 matrix-core GEMM (every format with a tiled
layout), 1 = the GEMV kernels with one workgroup per token and tile (the same layouts with SLAI_PROMPT_GEMM=0; a gated
Q8_0 pair has no such kernel), 0 = the ordinary loop.

The reference has no batched prompt pass: it feeds the prompt one token per forward pass (chat_llama2.rs:105-158).
The chunked pass must leave the caches that loop leaves, so: greedy ids after the prompt identical to the oracle's,
logits at the last prompt position within 1e-2 of the oracle's (the bar of every model test) and within 1e-3 of the
device's own token-by-token result (fp32 sums in another order), cache rows equal to the token-by-token ones within
f16 rounding."""
import ctypes as C

import numpy as np
import pytest

from gpu_common import backend, rel_err  # noqa: F401
from test_gpu_models import oracle_llama
from slai_amd import _ffi
from slai_amd import gguf_writer as gw
from slai_amd.runtime import Gguf, Llama2, SlaiError

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def backend_no_gemm():
    """A context created with SLAI_PROMPT_GEMM=0: chunks never take the matrix-core kernels."""
    import os
    from slai_amd.runtime import Backend
    old = os.environ.get("SLAI_PROMPT_GEMM")
    os.environ["SLAI_PROMPT_GEMM"] = "0"
    try:
        b = Backend(0)
    finally:
        if old is None:
            del os.environ["SLAI_PROMPT_GEMM"]
        else:
            os.environ["SLAI_PROMPT_GEMM"] = old
    yield b
    b.close()


LOGIT_TOL = 1e-2      # against the oracle
SELF_TOL = 1e-3       # against the device's token-by-token pass (fp32 sums in another order; an f16 cache entry may round the other way)
CACHE_TOL = 2e-3      # cache rows, relative to the largest entry (f16 rounding of values that differ in the last bits)


def read_cache(backend, m, layer, nbytes):
    k, v = m.kv_buffers(layer)
    out = []
    for h in (k, v):
        a = np.empty(nbytes, np.uint8)
        backend.check(backend.L.slai_read_buffer(backend.h, h, 0, a.ctypes.data, a.nbytes))
        out.append(a)
    return out


def check_prefill(backend, data, prompt, n_gen, chunks, kv_f16, model_type=_ffi.MODEL_LLAMA, neox=0, name=b"llama", expect_path=2,
                  split_at=None, expect_repeats=None):
    g, om = oracle_llama(data, 1, neox, int(kv_f16), name)
    L = g.L
    prompt = np.asarray(prompt, np.int32)
    n = prompt.size
    n_steps = n - 1 + n_gen
    gg = Gguf(data)
    kv = _ffi.KV_F16 if kv_f16 else _ffi.KV_F32
    m = Llama2(backend, gg, model_type, kv)
    vocab = m.config.vocab_size
    kv_dim = m.config.dim * m.config.n_kv_heads // m.config.n_q_heads
    ref_tokens = np.zeros(n_steps, np.int32)
    ref_logits = np.zeros((n_steps, vocab), np.float32)
    assert L.slo_llama2_generate(om, prompt.ctypes.data, n, 0, n_steps, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n_steps
    assert m.prefill_path() == expect_path
    # the token-by-token device pass: caches and the logits at the last prompt position
    m.generate(prompt, n - 1)
    esz = 2 if kv_f16 else 4
    row_bytes = kv_dim * esz
    base = [read_cache(backend, m, l, (n - 1) * row_bytes) for l in range(m.config.n_layers)]
    base_logits = m.forward_logits(n - 1, int(prompt[-1]), fused=True)
    m.destroy()
    dt = np.float16 if kv_f16 else np.float32
    for chunk in chunks:
        m = Llama2(backend, gg, model_type, kv)
        if split_at is None:
            m.prefill(prompt[:-1], 0, chunk)
        else:                                               # two calls: the second continues at a later position
            m.prefill(prompt[:split_at], 0, chunk)
            m.prefill(prompt[split_at:-1], split_at, chunk)
        for l in range(m.config.n_layers):
            got = read_cache(backend, m, l, (n - 1) * row_bytes)
            for a, b in zip(got, base[l]):
                fa, fb = a.view(dt).astype(np.float32), b.view(dt).astype(np.float32)
                assert np.abs(fa - fb).max() <= CACHE_TOL * np.abs(fb).max(), (chunk, l)
        logits = m.forward_logits(n - 1, int(prompt[-1]), fused=True)
        assert rel_err(logits, ref_logits[n - 1]) < LOGIT_TOL, chunk
        assert rel_err(logits, base_logits) < SELF_TOL, (chunk, rel_err(logits, base_logits))
        got, _ = m.generate(prompt, n_gen, start_pos=n - 1)
        assert np.array_equal(got, ref_tokens[n - 1:]), (chunk, got.tolist(), ref_tokens[n - 1:].tolist())
        if expect_repeats is not None:
            assert m.prefill_fp32_repeats() == expect_repeats, (chunk, m.prefill_fp32_repeats())
        m.destroy()
    gg.close(); L.slo_llama2_free(om); g.close()


@pytest.mark.parametrize("kv_f16", [False, True])
def test_prefill_matrix_cores_kquants_gqa_ragged_chunks(backend, kv_f16):
    """Q4_K with Q6_K v / output, grouped-query attention (4 query heads per kv head), head size 128; a prompt of 45
    tokens in chunks of 1 (the plain loop), 5, 32 (ragged last chunk) and 64 (clamped to 32)."""
    data = gw.llama_gguf(dim=1024, hidden_dim=2048, n_layers=3, n_heads=8, n_kv_heads=2, vocab=1000, seq_len=64,
                         wtype=12, v_type=14, out_type=14, embd_type=12, seed=11, std=0.04, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(8)).integers(0, 1000, 45)
    check_prefill(backend, data, prompt, 16, [1, 5, 32, 64], kv_f16, expect_path=2)


@pytest.mark.parametrize("wtype", [13, 14], ids=["q5_k", "q6_k"])
def test_prefill_matrix_cores_other_kquants(backend, wtype):
    """Every matrix in Q5_K / Q6_K, head size 64, multi-head attention."""
    data = gw.llama_gguf(dim=1024, hidden_dim=1024, n_layers=2, n_heads=16, n_kv_heads=16, vocab=800, seq_len=64, wtype=wtype, seed=5 + wtype,
                         std=0.04, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(wtype)).integers(0, 800, 37)
    check_prefill(backend, data, prompt, 12, [32], True, expect_path=2)


def test_prefill_7b_width_head_128(backend):
    """The shapes of BASELINE configuration 4 at depth 2 (dim 4096, hidden 11008, 32 heads of 128, fp16 cache): here
    the token-by-token pass runs q/k/v and attention as one launch, the chunked pass as three."""
    data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=2, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=128,
                         wtype=12, v_type=14, out_type=14, embd_type=12, seed=41)
    prompt = np.random.Generator(np.random.PCG64(41)).integers(0, 32000, 41)
    check_prefill(backend, data, prompt, 12, [8, 32], True, expect_path=2)


def test_prefill_matrix_cores_qwen2_bias_neox(backend):
    """Qwen2: q/k/v biases and Neox pairs in the chunk's bias + RoPE + cache-write launch."""
    data = gw.llama_gguf(dim=1024, hidden_dim=1024, n_layers=2, n_heads=8, n_kv_heads=2, vocab=400, seq_len=48, wtype=12,
                         seed=31, std=0.05, arch="qwen2", bias=True, norm_random=True, rope_base=1000000.0, rms_eps=1e-6)
    prompt = np.random.Generator(np.random.PCG64(3)).integers(0, 400, 35)
    check_prefill(backend, data, prompt, 12, [32], True, model_type=_ffi.MODEL_QWEN2, neox=1, name=b"qwen2", expect_path=2)


@pytest.mark.parametrize("kv_f16", [False, True])
def test_prefill_matrix_cores_32_row_tiles(backend, kv_f16):
    """A width (512) whose attention output and down matrices get 32-row tiles (two super-blocks per wave), head size 64,
    grouped-query attention.  Chunks of 3, 8 (ragged last chunk) and 32 (one chunk)."""
    data = gw.llama_gguf(dim=512, hidden_dim=2816, n_layers=3, n_heads=8, n_kv_heads=2, vocab=1000, seq_len=64,
                         wtype=12, v_type=14, out_type=14, embd_type=12, seed=11, std=0.06, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(8)).integers(0, 1000, 22)
    check_prefill(backend, data, prompt, 16, [3, 8, 32], kv_f16, expect_path=2)


@pytest.mark.parametrize("wtype", [12, 2], ids=["q4_k", "q4_0"])
def test_prefill_feed_forward_wider_than_16384(backend, backend_no_gemm, wtype):
    """A down projection of 16640 columns (17 column groups of 16-row tiles): more groups than a workgroup has waves,
    so it takes two launches over slices of the groups, the second accumulating; on the matrix cores and through the
    GEMV kernels."""
    data = gw.llama_gguf(dim=512, hidden_dim=16640, n_layers=2, n_heads=8, n_kv_heads=8, vocab=600, seq_len=48, wtype=wtype, seed=19,
                         std=0.03, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(19)).integers(0, 600, 25)
    check_prefill(backend, data, prompt, 10, [16], True, expect_path=2)
    check_prefill(backend_no_gemm, data, prompt, 10, [16], True, expect_path=1)


@pytest.mark.parametrize("wtype", [8, 2], ids=["q8_0", "q4_0"])
def test_prefill_matrix_cores_q8_0_q4_0(backend, wtype):
    """The two 32-element block formats on the matrix cores: 64-row tiles (q/k/v, gate/up), 32-row tiles (attention
    output at this width) and 16-row tiles (down), ragged chunks, f16 cache."""
    data = gw.llama_gguf(dim=512, hidden_dim=1024, n_layers=3, n_heads=8, n_kv_heads=2, vocab=1000, seq_len=64,
                         wtype=wtype, seed=11, std=0.06, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(8)).integers(0, 1000, 40)
    check_prefill(backend, data, prompt, 16, [7, 32], True, expect_path=2)


@pytest.mark.parametrize("kv_f16", [False, True])
def test_prefill_shared_weights_q4_0_gqa_ragged_chunks(backend_no_gemm, kv_f16):
    """Without the matrix-core kernels the chunks go through the GEMV kernels, one workgroup per token and tile.
    Chunks of 3, 8 (ragged last chunk) and 32 (one chunk)."""
    data = gw.llama_gguf(dim=512, hidden_dim=2816, n_layers=3, n_heads=8, n_kv_heads=2, vocab=1000, seq_len=64,
                         wtype=2, seed=11, std=0.06, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(8)).integers(0, 1000, 22)
    check_prefill(backend_no_gemm, data, prompt, 16, [3, 8, 32], kv_f16, expect_path=1)


def test_prefill_shared_weights_kquants_qwen2(backend_no_gemm):
    """The GEMV path with q/k/v biases and Neox pairs, Q4_K with a Q6_K v projection."""
    data = gw.llama_gguf(dim=1024, hidden_dim=1024, n_layers=2, n_heads=8, n_kv_heads=2, vocab=400, seq_len=48, wtype=12, v_type=14,
                         seed=31, std=0.05, arch="qwen2", bias=True, norm_random=True, rope_base=1000000.0, rms_eps=1e-6)
    prompt = np.random.Generator(np.random.PCG64(3)).integers(0, 400, 19)
    check_prefill(backend_no_gemm, data, prompt, 12, [4, 8], True, model_type=_ffi.MODEL_QWEN2, neox=1, name=b"qwen2", expect_path=1)


def test_prefill_continues_at_a_later_position(backend):
    data = gw.llama_gguf(dim=1024, hidden_dim=2048, n_layers=2, n_heads=8, n_kv_heads=8, vocab=2048, seq_len=128, wtype=13, seed=77,
                         std=0.04, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(5)).integers(0, 2048, 80)
    check_prefill(backend, data, prompt, 10, [32], True, split_at=13, expect_path=2)


def test_prefill_long_prompt(backend):
    """1100 prompt tokens in a context of 1280: every chunk's attention runs over the whole cache in one workgroup per
    head and token, while the token-by-token pass it is compared with uses the split kernel at this context length."""
    data = gw.llama_gguf(dim=1024, hidden_dim=1024, n_layers=1, n_heads=8, n_kv_heads=4, vocab=512, seq_len=1280, wtype=12, seed=21,
                         std=0.05, norm_random=True)
    prompt = np.random.Generator(np.random.PCG64(9)).integers(0, 512, 1100)
    check_prefill(backend, data, prompt, 8, [0], True, expect_path=2)


def test_prefill_falls_back_to_the_token_loop_for_other_layouts(backend):
    """Widths that are no multiple of 256 keep the row layout, which has no chunked kernels: the call then runs the
    ordinary loop and still leaves the same caches."""
    data = gw.tiny_llama_gguf(seed=99, std=0.1, norm_random=True, vocab=4096)
    prompt = np.random.Generator(np.random.PCG64(5)).integers(0, 4096, 12)
    check_prefill(backend, data, prompt, 10, [8], False, expect_path=0)


def test_prefill_argument_errors(backend):
    data = gw.llama_gguf(dim=256, hidden_dim=512, n_layers=1, n_heads=4, n_kv_heads=4, vocab=300, seq_len=16, wtype=12, seed=2)
    gg = Gguf(data)
    m = Llama2(backend, gg, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    assert m.prefill(np.zeros(0, np.int32)) == 0.0                       # nothing to do
    with pytest.raises(SlaiError):
        m.prefill(np.arange(17, dtype=np.int32))                         # past the context
    with pytest.raises(SlaiError):
        m.prefill(np.arange(10, dtype=np.int32), start_pos=8)
    with pytest.raises(SlaiError):
        m.prefill(np.array([1, 300], np.int32))                          # token out of range
    with pytest.raises(SlaiError):
        m.prefill(np.array([1, -1], np.int32))
    with pytest.raises(SlaiError):
        m.prefill(np.array([1, 2, 3], np.int32), chunk=65)
    m.prefill(np.arange(16, dtype=np.int32))                             # exactly the context
    m.destroy(); gg.close()


@pytest.mark.parametrize("kv_f16", [False, True])
def test_gpt2_prefill_matrix_cores(backend, kv_f16):
    """GPT-2-small widths (dim 768, 12 heads of 64, ff 3072, Q8_0) at depth 2: LayerNorm, biases, learned positions and
    GELU in the chunked pass.  Greedy ids after a 45-token prompt identical to the oracle's, logits at the last prompt
    position within 1e-2 of the oracle's and within 1e-3 of the device's token-by-token pass; chunks of 7 and 32, and a
    continuation at a later position."""
    from helpers import OracleGguf
    from slai_amd.runtime import Gpt2
    data = gw.gpt2_gguf(n_layer=2, seed=51, std=0.05)
    g = OracleGguf(data); L = g.L
    om = L.slo_gpt2_from_gguf(g.h, int(kv_f16))
    assert om
    prompt = np.random.Generator(np.random.PCG64(52)).integers(0, 50257, 45).astype(np.int32)
    n, n_gen = prompt.size, 10
    n_steps = n - 1 + n_gen
    ref_tokens = np.zeros(n_steps, np.int32); ref_logits = np.zeros((n_steps, 50257), np.float32)
    assert L.slo_gpt2_generate(om, prompt.ctypes.data, n, 0, n_steps, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n_steps
    gg = Gguf(data)
    kv = _ffi.KV_F16 if kv_f16 else _ffi.KV_F32
    m = Gpt2(backend, gg, kv)
    assert m.prefill_path() == 2
    m.generate(prompt, n - 1)
    base_logits = m.forward_logits(n - 1, int(prompt[-1]))
    m.destroy()
    for chunk, split_at in ((7, None), (32, None), (32, 13)):
        m = Gpt2(backend, gg, kv)
        if split_at is None:
            m.prefill(prompt[:-1], 0, chunk)
        else:
            m.prefill(prompt[:split_at], 0, chunk)
            m.prefill(prompt[split_at:-1], split_at, chunk)
        logits = m.forward_logits(n - 1, int(prompt[-1]))
        assert rel_err(logits, ref_logits[n - 1]) < LOGIT_TOL, chunk
        assert rel_err(logits, base_logits) < SELF_TOL, (chunk, rel_err(logits, base_logits))
        got, _ = m.generate(prompt, n_gen, start_pos=n - 1)
        assert np.array_equal(got, ref_tokens[n - 1:]), (chunk, got.tolist(), ref_tokens[n - 1:].tolist())
        m.destroy()
    # the plain loop behind the same call, and argument errors
    m = Gpt2(backend, gg, kv)
    m.prefill(prompt[:-1], 0, 1)
    assert rel_err(m.forward_logits(n - 1, int(prompt[-1])), base_logits) < 1e-6
    with pytest.raises(SlaiError):
        m.prefill(np.array([1, 50257], np.int32))
    with pytest.raises(SlaiError):
        m.prefill(np.arange(10, dtype=np.int32), start_pos=1020)
    m.destroy(); gg.close(); L.slo_gpt2_free(om); g.close()


def test_prefill_split_f16_and_its_fp32_repeat(backend):
    """The matrix-core path runs on the half-precision units with f16 head + remainder pairs; a model whose normalised
    rows exceed the f16 range (ffn_norm weights of 5e4) must notice, repeat the call with fp32 MFMA and still match the
    oracle; an ordinary model must not repeat."""
    import os
    if os.environ.get("SLAI_PROMPT_SPLIT_F16") == "0" or os.environ.get("SLAI_PROMPT_GEMM") == "0":
        pytest.skip("needs the split path")
    for scale, repeats in ((1.0, 0), (5.0e4, 1)):
        data = gw.llama_gguf(dim=1024, hidden_dim=2816, n_layers=2, n_heads=8, n_kv_heads=8, vocab=500, seq_len=64, wtype=12, v_type=14, seed=77,
                             std=0.05, ffn_norm_scale=scale)
        prompt = np.random.Generator(np.random.PCG64(78)).integers(0, 500, 40).astype(np.int32)
        check_prefill(backend, data, prompt, 6, (32,), True, expect_repeats=repeats)


def test_prefill_large_weights_take_fp32_from_the_start(backend):
    """The f16 head + remainder form needs 256 * |w| within f16; the block scales of every matrix bound |w| at load time,
    and a model beyond the bound (weights of std 40) takes the fp32 kernels at once: same parity, no repeated call."""
    data = gw.llama_gguf(dim=1024, hidden_dim=2816, n_layers=2, n_heads=8, n_kv_heads=8, vocab=500, seq_len=64, wtype=12, v_type=14, seed=79,
                         std=40.0)
    prompt = np.random.Generator(np.random.PCG64(80)).integers(0, 500, 40).astype(np.int32)
    check_prefill(backend, data, prompt, 6, (32,), True, expect_repeats=0)


def test_gpt2_prefill_fp32_repeat(backend):
    """GPT-2 with ffn_norm gains of 5e4: the normalised rows do not fit the f16 heads, the call is repeated with the
    fp32 kernels and the continuation still matches the oracle's greedy ids."""
    import os
    if os.environ.get("SLAI_PROMPT_SPLIT_F16") == "0" or os.environ.get("SLAI_PROMPT_GEMM") == "0":
        pytest.skip("needs the split path")
    from helpers import OracleGguf
    from slai_amd.runtime import Gpt2
    for scale, repeats in ((1.0, 0), (5.0e4, 1)):
        data = gw.gpt2_gguf(n_layer=2, seed=53, std=0.05, ffn_norm_scale=scale)
        g = OracleGguf(data); L = g.L
        om = L.slo_gpt2_from_gguf(g.h, 0)
        assert om
        prompt = np.random.Generator(np.random.PCG64(54)).integers(0, 50257, 40).astype(np.int32)
        n, n_gen = prompt.size, 6
        n_steps = n - 1 + n_gen
        ref_tokens = np.zeros(n_steps, np.int32); ref_logits = np.zeros((n_steps, 50257), np.float32)
        assert L.slo_gpt2_generate(om, prompt.ctypes.data, n, 0, n_steps, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n_steps
        gg = Gguf(data)
        m = Gpt2(backend, gg, _ffi.KV_F32)
        m.prefill(prompt[:-1], 0, 32)
        assert m.prefill_fp32_repeats() == repeats, (scale, m.prefill_fp32_repeats())
        logits = m.forward_logits(n - 1, int(prompt[-1]))
        assert rel_err(logits, ref_logits[n - 1]) < LOGIT_TOL, scale
        got, _ = m.generate(prompt, n_gen, start_pos=n - 1)
        assert np.array_equal(got, ref_tokens[n - 1:]), (scale, got.tolist(), ref_tokens[n - 1:].tolist())
        m.destroy(); gg.close(); L.slo_gpt2_free(om); g.close()
