"""End-to-end GPU parity: Llama-2 / Qwen2 / GPT-2 decode against the oracle on identical seeded
GGUF bytes.  Bars (from the task statement): logits max-abs-rel <= 1e-2, greedy ids identical."""
import ctypes as C

import numpy as np
import pytest

from gpu_common import backend, rel_err  # noqa: F401
from helpers import OracleGguf
from slai_amd import _ffi
from slai_amd import gguf_writer as gw

pytestmark = pytest.mark.gpu
LOGIT_TOL = 1e-2


def oracle_llama(data, gpu_semantics=1, neox=0, kv_f16=0, name=b"llama"):
    g = OracleGguf(data)
    m = g.L.slo_llama2_from_gguf(g.h, name, gpu_semantics, neox, kv_f16)
    assert m
    return g, m


def check_llama(backend, data, prompt, n_steps, kv_f16=False, model_type=_ffi.MODEL_LLAMA, neox=0, name=b"llama",
                check_logit_steps=8, tol=LOGIT_TOL, decode_form=None):
    from slai_amd.runtime import Gguf, Llama2
    g, om = oracle_llama(data, 1, neox, int(kv_f16), name)
    L = g.L
    vocab = int(np.prod(g.tensors["token_embd.weight"]["dims"][:1]))
    prompt = np.asarray(prompt, np.int32)
    ref_tokens = np.zeros(n_steps, np.int32)
    ref_logits = np.zeros((n_steps, vocab), np.float32)
    assert L.slo_llama2_generate(om, prompt.ctypes.data, prompt.size, 0, n_steps, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n_steps
    gg = Gguf(data)
    kv = _ffi.KV_F16 if kv_f16 else _ffi.KV_F32
    worst = 0.0
    # step-by-step logits, reference op order (fused=0) and fused kernels (fused=1), fed the oracle's tokens
    for fused in (False, True):
        m = Llama2(backend, gg, model_type, kv)
        if decode_form is not None:
            assert m.decode_form() == decode_form      # the form under test is the one the model took
        tok = int(prompt[0])
        for pos in range(min(check_logit_steps, n_steps)):
            logits = m.forward_logits(pos, tok, fused=fused)
            err = rel_err(logits, ref_logits[pos])
            worst = max(worst, err)
            assert err < tol, (fused, pos, err)
            tok = int(ref_tokens[pos])
        m.destroy()
    # the device-resident greedy loop
    m = Llama2(backend, gg, model_type, kv)
    got, ms = m.generate(prompt, n_steps)
    assert np.array_equal(got, ref_tokens), (got.tolist(), ref_tokens.tolist())
    # a second call resumes from the kept KV cache (chat "resume" semantics: start_pos > 0)
    if n_steps > prompt.size + 4:
        cut = prompt.size + 2
        seq = np.concatenate([prompt[:1], ref_tokens[:cut]]).astype(np.int32)   # tokens fed at positions 0..cut
        again, _ = m.generate(seq, n_steps - cut, start_pos=cut)
        assert np.array_equal(again, ref_tokens[cut:])
    m.destroy()
    gg.close(); L.slo_llama2_free(om); g.close()
    return worst


def test_tiny_llama_q8_0_config1(backend):
    """BASELINE configuration 1: dim 288, 6 layers, 6 heads, hidden 768, vocab 32000, seq 256, Q8_0;
    16 seeded prompt ids, 128 greedy tokens."""
    data = gw.tiny_llama_gguf(seed=1234)
    prompt = np.random.Generator(np.random.PCG64(1234)).integers(0, 32000, 16)
    worst = check_llama(backend, data, prompt, 16 + 128 - 1, check_logit_steps=20)
    print("worst logits rel err", worst)


def test_tiny_llama_wider_weights_nontrivial_sequence(backend):
    """Same shape with std 0.1 weights and random norm gains, so greedy decoding does not collapse
    onto one token and the id comparison is a real test."""
    data = gw.tiny_llama_gguf(seed=99, std=0.1, norm_random=True, vocab=4096)
    prompt = np.random.Generator(np.random.PCG64(5)).integers(0, 4096, 16)
    check_llama(backend, data, prompt, 16 + 64, check_logit_steps=24)


@pytest.mark.parametrize("kv_f16", [False, True])
def test_llama_kquants_gqa(backend, kv_f16):
    """Q4_K weights with Q6_K v-proj / output (Q4_K_M-style), grouped-query attention, f32 and f16 KV."""
    data = gw.llama_gguf(dim=512, hidden_dim=1280, n_layers=3, n_heads=8, n_kv_heads=2, vocab=1000, seq_len=64,
                         wtype=12, v_type=14, out_type=14, embd_type=12, seed=11, std=0.06, norm_random=True)
    prompt = [3, 500, 999, 7, 42, 42, 1]
    check_llama(backend, data, prompt, 40, kv_f16=kv_f16, check_logit_steps=12)


@pytest.mark.parametrize("wtype", [2, 3, 6, 7, 13, 1, 0], ids=["q4_0", "q4_1", "q5_0", "q5_1", "q5_k", "f16", "f32"])
def test_llama_other_formats(backend, wtype):
    data = gw.llama_gguf(dim=256, hidden_dim=768, n_layers=2, n_heads=4, n_kv_heads=4, vocab=512, seq_len=32,
                         wtype=wtype, seed=21 + wtype, std=0.08, norm_random=True, with_output=(wtype != 1))
    check_llama(backend, data, [1, 2, 3, 4], 24, check_logit_steps=8)


def test_qwen2_bias_and_neox_rope(backend):
    """The Qwen2 variant of the loop: q/k/v biases (transformer.rs:336-344) + Neox RoPE (llama2/mod.rs:27-32)."""
    data = gw.llama_gguf(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab=400, seq_len=32, wtype=8,
                         seed=31, std=0.08, arch="qwen2", bias=True, norm_random=True, rope_base=1000000.0, rms_eps=1e-6)
    check_llama(backend, data, [9, 8, 7], 20, model_type=_ffi.MODEL_QWEN2, neox=1, name=b"qwen2", kv_f16=True)


def test_llama_7b_width_two_layers(backend):
    """Real 7B matrix shapes (dim 4096, hidden 11008, 32 heads of 128, vocab 32000) at depth 2,
    Q4_K / Q6_K, fp16 KV: the kernels at the shapes of BASELINE configuration 4."""
    data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=2, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=128,
                         wtype=12, v_type=14, out_type=14, embd_type=12, seed=41)
    prompt = np.random.Generator(np.random.PCG64(41)).integers(0, 32000, 8)
    check_llama(backend, data, prompt, 40, kv_f16=True, check_logit_steps=10)


def test_gpt2_config3_shape_small_depth(backend):
    """GPT-2-small widths (dim 768, 12 heads, ff 3072, vocab 50257 with its row tail, ctx 1024), 2 layers."""
    from slai_amd.runtime import Gguf, Gpt2
    data = gw.gpt2_gguf(n_layer=2, seed=51, std=0.05)
    g = OracleGguf(data); L = g.L
    om = L.slo_gpt2_from_gguf(g.h, 0)
    assert om
    prompt = np.random.Generator(np.random.PCG64(51)).integers(0, 50257, 8).astype(np.int32)
    n = 32
    ref_tokens = np.zeros(n, np.int32); ref_logits = np.zeros((n, 50257), np.float32)
    assert L.slo_gpt2_generate(om, prompt.ctypes.data, 8, 0, n, -1, ref_tokens.ctypes.data, ref_logits.ctypes.data) == n
    gg = Gguf(data)
    m = Gpt2(backend, gg)
    assert m.params.attn_b == 2304
    tok = int(prompt[0])
    for pos in range(10):
        err = rel_err(m.forward_logits(pos, tok), ref_logits[pos])
        assert err < LOGIT_TOL, (pos, err)
        tok = int(ref_tokens[pos])
    m.destroy()
    m = Gpt2(backend, gg)
    got, _ = m.generate(prompt, n)
    assert np.array_equal(got, ref_tokens)
    m.destroy(); gg.close(); L.slo_gpt2_free(om); g.close()


def test_model_load_errors(backend):
    from slai_amd.runtime import Gguf, Llama2, SlaiError
    data = gw.llama_gguf(dim=64, hidden_dim=128, n_layers=1, n_heads=2, n_kv_heads=2, vocab=32, seq_len=8, wtype=8)
    g = Gguf(data)
    with pytest.raises(SlaiError) as e:
        Llama2(backend, g, _ffi.MODEL_QWEN2)          # keys are "llama.*": missing "qwen2.embedding_length"
    assert e.value.code == _ffi.E_MISSING
    m = Llama2(backend, g)
    with pytest.raises(SlaiError):
        m.forward_logits(8, 0)                         # position past the context
    with pytest.raises(SlaiError):
        m.generate([1, 2, 40], 2)                      # token id out of range
    m.destroy(); g.close()


def test_generate_works_as_the_first_call_on_a_fresh_context():
    """The captured decode graph must not need any allocation: everything the kernels use is sized at load time, so
    `generate` may be the very first thing a context does (no eager forward before it)."""
    from slai_amd import _ffi, gguf_writer as gw
    from slai_amd.runtime import Backend, Gguf, Gpt2, Llama2
    b = Backend(0)
    try:
        g = Gguf(gw.gpt2_gguf(n_embd=768, n_layer=2, n_head=12, ff_len=3072, vocab=1000, n_seq=64, wtype=8, seed=5))
        m = Gpt2(b, g, _ffi.KV_F32)
        toks, _ = m.generate(np.array([1, 2, 3], np.int32), 8)
        assert toks.shape == (8,)
        m.destroy(); g.close()
        g = Gguf(gw.llama_gguf(dim=512, hidden_dim=1536, n_layers=2, n_heads=8, n_kv_heads=8, vocab=1024, seq_len=64, wtype=12, seed=6))
        m = Llama2(b, g, _ffi.MODEL_LLAMA, _ffi.KV_F16)
        toks, _ = m.generate(np.array([1, 2, 3], np.int32), 8)
        assert toks.shape == (8,)
        m.destroy(); g.close()
    finally:
        b.close()


@pytest.mark.parametrize("wtype", [8, 2, 13, 14], ids=["q8_0", "q4_0", "q5_k", "q6_k"])
def test_llama_tiled_layouts_every_format(backend, wtype):
    """Widths that take the tiled layouts (multiples of 256) in every format that has them, MHA, fp16 cache: logits and
    greedy ids against the oracle."""
    data = gw.llama_gguf(dim=512, hidden_dim=1536, n_layers=3, n_heads=8, n_kv_heads=8, vocab=2048, seq_len=128, wtype=wtype, seed=77,
                         std=0.05, norm_random=True)
    check_llama(backend, data, [5, 1000, 2047, 9, 77, 3], 40, kv_f16=True, check_logit_steps=12)


@pytest.mark.parametrize("kv_f16", [False, True])
def test_llama_context_beyond_1024_uses_split_attention(backend, kv_f16):
    """A model whose context (1280) is past the single-workgroup attention limit: the decode graph then runs the split
    (flash-decoding) kernel with its combine pass from position 0 on; ids must match the oracle through position 1100."""
    data = gw.llama_gguf(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab=512, seq_len=1280, wtype=12, seed=21,
                         std=0.08, norm_random=True)
    check_llama(backend, data, [5, 100, 511, 9, 77, 3, 8, 1], 1100, kv_f16=kv_f16, check_logit_steps=6)


def test_model_load_refuses_vectors_of_the_wrong_length(backend):
    """A file whose norm vector or bias is shorter than the model's width is refused by the load itself (E_SHAPE), with
    nothing uploaded or launched: the fused kernels would otherwise read past the allocation."""
    from slai_amd.runtime import Gguf, Gpt2, Llama2, SlaiError

    def short(target, n):
        return lambda name, d, t, x: ([n], t, x[:4 * n]) if name == target else (d, t, x)
    for target, n in (("blk.1.attn_norm.weight", 100), ("blk.0.attn_k.bias", 64), ("output_norm.weight", 8)):
        g = Gguf(gw.llama_gguf(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab=64, seq_len=16, wtype=8, seed=5,
                               bias=True, tensor_hook=short(target, n)))
        with pytest.raises(SlaiError) as e:
            Llama2(backend, g)
        assert e.value.code == _ffi.E_SHAPE and target in str(e.value)
        g.close()
    g = Gguf(gw.gpt2_gguf(n_embd=64, n_layer=2, n_head=2, ff_len=128, vocab=50, n_seq=16, tensor_hook=short("blk.1.ffn_up.bias", 64)))
    with pytest.raises(SlaiError) as e:
        Gpt2(backend, g)
    assert e.value.code == _ffi.E_SHAPE
    g.close()


def test_small_model_keeps_working_after_the_context_scratch_grew():
    """The decode graph of a model holds the addresses of the context's scratch blocks.  A second, larger model, a long
    slai_attention call, a wide slai_matmul_quant_columns and a sampler over a larger vocabulary all make those blocks
    grow; the first model's graph must go on reading and writing valid memory and produce the oracle's tokens."""
    from slai_amd.runtime import Backend, Gguf, GpuQuantMatrix, GpuTensor, Llama2, LlmContext
    from slai_amd import synth
    b = Backend(0)
    try:
        # a context of 1280 positions: the small model's graph uses the split attention kernel and its scratch
        small = gw.llama_gguf(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab=512, seq_len=1280, wtype=12, seed=21,
                              std=0.08, norm_random=True)
        prompt = np.array([5, 100, 511, 9], np.int32)
        n = 24
        og, om = oracle_llama(small, 1, 0, 1)
        ref = np.zeros(n, np.int32)
        assert og.L.slo_llama2_generate(om, prompt.ctypes.data, prompt.size, 0, n, -1, ref.ctypes.data, None) == n
        g1 = Gguf(small)
        m1 = Llama2(b, g1, _ffi.MODEL_LLAMA, _ffi.KV_F16)
        got, _ = m1.generate(prompt, n)                                   # captures the graph
        assert np.array_equal(got, ref)
        # now everything that grows the context's scratch blocks
        big = gw.llama_gguf(dim=1024, hidden_dim=2816, n_layers=1, n_heads=8, n_kv_heads=8, vocab=40000, seq_len=4096, wtype=12, seed=22)
        g2 = Gguf(big)
        m2 = Llama2(b, g2, _ffi.MODEL_LLAMA, _ffi.KV_F16)
        m2.generate(np.array([1, 2, 3], np.int32), 4)
        m2.generate_sampled(np.array([1, 2, 3], np.int32), 4, 0.7, 0.95, 1)
        ctxt = LlmContext(b)
        w = GpuQuantMatrix(b, 12, 64, 8192, synth.normal_quantized(3, 12, 64, 8192, 0.02), layout=_ffi.LAYOUT_TILE16)
        x = GpuTensor.matrix(b, np.ones((8192, 32), np.float32))
        out = GpuTensor(b, 64, 32)
        ctxt.matmul_quant_columns(out, w, x)
        b.synchronize()
        got, _ = m1.generate(prompt, n)                                   # replays the graph captured before
        assert np.array_equal(got, ref)
        got, _ = m1.generate_sampled(prompt, n, 0.0, 1.0, 7)              # and a graph captured afterwards
        assert np.array_equal(got, ref)
        for t in (w, x, out):
            t.destroy()
        m2.destroy(); g2.close(); m1.destroy(); g1.close()
        og.L.slo_llama2_free(om); og.close()
    finally:
        b.close()


def test_device_against_the_transformers_library_directly(backend):
    """The device path against an implementation that shares nothing with this repository: tiny seeded
    LlamaForCausalLM (grouped-query attention, rows permuted to adjacent-pair order), Qwen2ForCausalLM (biases, NeoX
    pairs) and GPT2LMHeadModel from the `transformers` library in fp32 on the CPU, exported as F32 GGUF tensors.  Logits
    within 1e-4 of the library's at every step, greedy ids identical."""
    hf = pytest.importorskip("test_oracle_models_hf")
    from slai_amd.runtime import Gguf, Gpt2, Llama2
    prompt = hf.PROMPT
    n = len(prompt) - 1 + 24

    def run(model, tok0):
        got_logits, got_ids = [], []
        tok = tok0
        for pos in range(n):
            lg = model.forward_logits(pos, tok)
            got_logits.append(lg)
            tok = int(prompt[pos + 1]) if pos < len(prompt) - 1 else int(np.argmax(lg))
            got_ids.append(tok)
        return np.stack(got_logits), np.array(got_ids, np.int32)

    cases = []
    m = hf.llama_model(202, 2, 500000.0, 1e-6)
    cases.append(("llama gqa", m, hf.llama_family_gguf(m, "llama", permute=True), _ffi.MODEL_LLAMA))
    cfg = hf.transformers.Qwen2Config(hidden_size=64, intermediate_size=176, num_hidden_layers=3, num_attention_heads=4, num_key_value_heads=2,
                                      vocab_size=160, max_position_embeddings=64, rms_norm_eps=1e-6,
                                      rope_parameters={"rope_type": "default", "rope_theta": 1000000.0}, tie_word_embeddings=False,
                                      use_sliding_window=False, attn_implementation="eager")
    q = hf.transformers.Qwen2ForCausalLM(cfg).eval()
    hf.seeded_weights(q, 204)
    cases.append(("qwen2", q, hf.llama_family_gguf(q, "qwen2", permute=False), _ffi.MODEL_QWEN2))
    for what, model, data, mtype in cases:
        lib_logits, lib_ids = hf.library_run(model, prompt, n)
        gg = Gguf(data)
        for kv in (_ffi.KV_F32,):
            dm = Llama2(backend, gg, mtype, kv)
            got_logits, got_ids = run(dm, int(prompt[0]))
            hf.compare(lib_logits, lib_ids, got_logits, got_ids, what + " on the device")
            ids, _ = dm.generate(np.array(prompt, np.int32), n)
            assert np.array_equal(ids, lib_ids), what
            dm.destroy()
        gg.close()


def test_time_steps_names_every_launch_of_a_token(backend):
    """slai_llama2_time_steps: the launch-per-step form of a 3-layer model reports each of its steps with the number of
    launches per token and a positive time; the logits afterwards are those of an ordinary forward at that position."""
    from slai_amd.runtime import Gguf, Llama2
    data = gw.llama_gguf(dim=512, hidden_dim=1536, n_layers=3, n_heads=4, n_kv_heads=4, vocab=1024, seq_len=64, wtype=12, seed=9, std=0.05)
    g = Gguf(data)
    m = Llama2(backend, g, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    toks, _ = m.generate(np.array([1, 2, 3], np.int32), 8)
    ref = m.forward_logits(8, int(toks[7]))
    steps = m.time_steps(8, int(toks[7]), reps=4)
    names = [s[0] for s in steps]
    assert names[0] == "embedding row" and names[-1] == "llama2 output", names
    per = {s[0]: s[2] for s in steps}
    assert per["llama2 attn_output"] == 3 and per["llama2 ffn gate/up"] == 3 and per["llama2 ffn_down"] == 3 and per["llama2 output"] == 1, per
    assert all(s[1] > 0.0 and s[3] > 0.0 for s in steps), steps
    assert np.array_equal(m.forward_logits(8, int(toks[7])), ref)
    m.destroy(); g.close()
