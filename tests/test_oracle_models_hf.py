"""Pins the oracle's whole-model functions against an independent implementation: the `transformers` library's
LlamaForCausalLM, Qwen2ForCausalLM and GPT2LMHeadModel on the CPU in fp32.

Tiny models are built from a config with seeded weights (nothing is downloaded), exported through the GGUF writer as
F32 tensors under the names the loader reads, and run through `slo_llama2_forward` / `slo_gpt2_forward`.  What this
fixes, and what only the builder's own numpy twin checked before: the order of the residual additions, the mapping of
query heads onto cache heads under grouped-query attention, biases added before the rotation, the pairing of the
rotated dimensions in both RoPE variants, epsilon and frequency base taken from the file, LayerNorm / GELU placement and
the tied output matrix of GPT-2.  The functions restate crates/slai/src/models/llama2/cpu.rs:379-446,
models/llama2/transformer.rs:316-381 (bias, rope variant, eps / base from the config), shaders/slai/rope.slang:56-84
and models/gpt2/cpu.rs:225-383.

`transformers` rotates (i, i + head/2) pairs ("NeoX" order).  The reference's Llama path rotates adjacent pairs, which
is why GGUF converters permute the rows of the q / k matrices; `permute_qk` below is that permutation, so the permuted
file under the adjacent-pair oracle and the unpermuted file under the NeoX oracle must both reproduce the library.
"""
import ctypes as C

import numpy as np
import pytest

from helpers import OracleGguf
from slai_amd import gguf_writer as gw

torch = pytest.importorskip("torch")
transformers = pytest.importorskip("transformers")

LOGIT_TOL = 1e-4      # max-abs error relative to the largest logit; both sides are fp32, only summation order differs
N_GREEDY = 32


def seeded_weights(model, seed, std=0.15, std_of=None):
    """Every parameter from one seeded generator: matrices N(0, std) (`std_of`: name fragment -> another std), norm
    gains N(1, 0.1), biases N(0, 0.1)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    with torch.no_grad():
        for name, p in model.named_parameters():
            shape = tuple(p.shape)
            if p.dim() == 1 and ("norm" in name or "ln_" in name) and name.endswith("weight"):
                a = rng.normal(1.0, 0.1, shape)
            elif p.dim() == 1:
                a = rng.normal(0.0, 0.1, shape)
            else:
                sd = std
                for frag, v in (std_of or {}).items():
                    if frag in name:
                        sd = v
                a = rng.normal(0.0, sd, shape)
            p.copy_(torch.from_numpy(a.astype(np.float32)))


def permute_qk(w, n_head):
    """Rows of a q / k matrix (or entries of its bias) from (i, i + hs/2) pairing to adjacent (2i, 2i+1) pairing."""
    w = np.asarray(w)
    return w.reshape(n_head, 2, w.shape[0] // n_head // 2, *w.shape[1:]).swapaxes(1, 2).reshape(w.shape)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint8).reshape(-1)


def llama_family_gguf(model, arch, permute):
    cfg = model.config
    sd = {k: v.detach().numpy() for k, v in model.state_dict().items()}
    w = gw.GgufWriter()
    w.add_meta("general.architecture", gw.T_STR, arch)
    w.add_meta(arch + ".embedding_length", gw.T_U32, cfg.hidden_size)
    w.add_meta(arch + ".feed_forward_length", gw.T_U32, cfg.intermediate_size)
    w.add_meta(arch + ".block_count", gw.T_U32, cfg.num_hidden_layers)
    w.add_meta(arch + ".attention.head_count", gw.T_U32, cfg.num_attention_heads)
    w.add_meta(arch + ".attention.head_count_kv", gw.T_U32, cfg.num_key_value_heads)
    w.add_meta(arch + ".context_length", gw.T_U32, cfg.max_position_embeddings)
    w.add_meta(arch + ".rope.freq_base", gw.T_F32, float(cfg.rope_parameters["rope_theta"]))
    w.add_meta(arch + ".attention.layer_norm_rms_epsilon", gw.T_F32, float(cfg.rms_norm_eps))
    w.add_meta("tokenizer.ggml.tokens", gw.T_ARR, [""] * cfg.vocab_size, elem_type=gw.T_STR)

    def mat(name, a):
        w.add_tensor(name, [a.shape[1], a.shape[0]], 0, f32(a))

    def vec(name, a):
        w.add_tensor(name, [a.shape[0]], 0, f32(a))

    mat("token_embd.weight", sd["model.embed_tokens.weight"])
    for l in range(cfg.num_hidden_layers):
        hp, p = "model.layers.%d." % l, "blk.%d." % l
        vec(p + "attn_norm.weight", sd[hp + "input_layernorm.weight"])
        for nm, hf, heads in (("attn_q", "q_proj", cfg.num_attention_heads), ("attn_k", "k_proj", cfg.num_key_value_heads), ("attn_v", "v_proj", 0)):
            a = sd[hp + "self_attn." + hf + ".weight"]
            b = sd.get(hp + "self_attn." + hf + ".bias")
            if permute and heads:
                a = permute_qk(a, heads)
                b = None if b is None else permute_qk(b, heads)
            mat(p + nm + ".weight", a)
            if b is not None:
                vec(p + nm + ".bias", b)
        mat(p + "attn_output.weight", sd[hp + "self_attn.o_proj.weight"])
        vec(p + "ffn_norm.weight", sd[hp + "post_attention_layernorm.weight"])
        mat(p + "ffn_gate.weight", sd[hp + "mlp.gate_proj.weight"])
        mat(p + "ffn_up.weight", sd[hp + "mlp.up_proj.weight"])
        mat(p + "ffn_down.weight", sd[hp + "mlp.down_proj.weight"])
    vec("output_norm.weight", sd["model.norm.weight"])
    mat("output.weight", sd["lm_head.weight"])
    return w.to_bytes()


def library_run(model, prompt, n_steps):
    """Teacher-forced logits at every position of the greedy continuation, and the greedy ids (forced-token rule of
    slai-chat/src/sampler.rs:91-111: inside the prompt the next token is the prompt's)."""
    seq = [int(prompt[0])]
    logits, picks = [], []
    with torch.no_grad():
        for pos in range(n_steps):
            out = model(torch.tensor([seq])).logits[0, -1].numpy().astype(np.float32)    # full recompute: no cache involved
            logits.append(out)
            nxt = int(prompt[pos + 1]) if pos < len(prompt) - 1 else int(np.argmax(out))
            picks.append(nxt)
            seq.append(nxt)
    return np.stack(logits), np.array(picks, np.int32)


def compare(lib_logits, lib_ids, got_logits, got_ids, what):
    for pos in range(lib_logits.shape[0]):
        err = np.abs(got_logits[pos].astype(np.float64) - lib_logits[pos]).max() / np.abs(lib_logits[pos]).max()
        assert err < LOGIT_TOL, (what, pos, err)
    assert np.array_equal(got_ids, lib_ids), (what, got_ids.tolist(), lib_ids.tolist())
    # the comparison means something only if the continuation is not one repeated token
    assert len(set(lib_ids[-16:].tolist())) > 2, (what, lib_ids.tolist())


def oracle_llama_run(data, name, gpu_semantics, neox, prompt, n_steps):
    g = OracleGguf(data)
    L = g.L
    m = L.slo_llama2_from_gguf(g.h, name, gpu_semantics, neox, 0)
    assert m
    vocab = g.tensors["token_embd.weight"]["dims"][0]
    ids = np.zeros(n_steps, np.int32)
    logits = np.zeros((n_steps, vocab), np.float32)
    p = np.ascontiguousarray(prompt, np.int32)
    assert L.slo_llama2_generate(m, p.ctypes.data, p.size, 0, n_steps, -1, ids.ctypes.data, logits.ctypes.data) == n_steps
    L.slo_llama2_free(m)
    g.close()
    return logits, ids


def llama_model(seed, n_kv_heads, theta, eps):
    cfg = transformers.LlamaConfig(hidden_size=64, intermediate_size=176, num_hidden_layers=3, num_attention_heads=4,
                                   num_key_value_heads=n_kv_heads, vocab_size=160, max_position_embeddings=64, rms_norm_eps=eps,
                                   rope_parameters={"rope_type": "default", "rope_theta": theta}, tie_word_embeddings=False,
                                   attention_bias=False, mlp_bias=False, attn_implementation="eager")
    m = transformers.LlamaForCausalLM(cfg).eval()
    seeded_weights(m, seed)
    return m


PROMPT = [3, 77, 150, 9, 21, 0, 64]


def test_llama_cpu_path_adjacent_pairs_mha():
    """cpu.rs:379-446 as it is (eps 1e-5 and base 10000 hard-coded, adjacent-pair RoPE), multi-head attention."""
    m = llama_model(101, 4, 10000.0, 1e-5)
    lib_logits, lib_ids = library_run(m, PROMPT, len(PROMPT) - 1 + N_GREEDY)
    got = oracle_llama_run(llama_family_gguf(m, "llama", permute=True), b"llama", 0, 0, PROMPT, lib_ids.size)
    compare(lib_logits, lib_ids, *got, "llama cpu semantics, MHA")


def test_llama_gpu_semantics_gqa_eps_and_base_from_the_file():
    """transformer.rs:316-381: grouped-query attention (4 query heads on 2 cache heads), eps 1e-6 and base 5e5 read
    from the metadata; adjacent pairs on the permuted file."""
    m = llama_model(102, 2, 500000.0, 1e-6)
    lib_logits, lib_ids = library_run(m, PROMPT, len(PROMPT) - 1 + N_GREEDY)
    got = oracle_llama_run(llama_family_gguf(m, "llama", permute=True), b"llama", 1, 0, PROMPT, lib_ids.size)
    compare(lib_logits, lib_ids, *got, "llama gpu semantics, GQA, adjacent pairs")
    # the CPU semantics ignore both metadata values (cpu.rs:345,468): with this file they must NOT match
    other_logits, _ = oracle_llama_run(llama_family_gguf(m, "llama", permute=True), b"llama", 0, 0, PROMPT, 8)
    assert np.abs(other_logits[7] - lib_logits[7]).max() / np.abs(lib_logits[7]).max() > 10 * LOGIT_TOL


def test_llama_neox_pairing_on_the_unpermuted_file():
    """rope.slang:56-84: the (i, i + head/2) pairing, on the weights exactly as the library holds them; and the two
    pairings are really different (the adjacent-pair oracle on the same file is far off)."""
    m = llama_model(103, 1, 10000.0, 1e-5)
    lib_logits, lib_ids = library_run(m, PROMPT, len(PROMPT) - 1 + N_GREEDY)
    data = llama_family_gguf(m, "llama", permute=False)
    compare(lib_logits, lib_ids, *oracle_llama_run(data, b"llama", 1, 1, PROMPT, lib_ids.size), "llama, NeoX pairs, MQA")
    wrong_logits, _ = oracle_llama_run(data, b"llama", 1, 0, PROMPT, 8)
    assert np.abs(wrong_logits[7] - lib_logits[7]).max() / np.abs(lib_logits[7]).max() > 100 * LOGIT_TOL


def test_qwen2_biases_before_the_rotation():
    """The Qwen2 variant (llama2/mod.rs:19-32, transformer.rs:336-347): q / k / v biases added before RoPE, NeoX pairs,
    base 1e6, eps 1e-6, 4 query heads on 2 cache heads."""
    cfg = transformers.Qwen2Config(hidden_size=64, intermediate_size=176, num_hidden_layers=3, num_attention_heads=4, num_key_value_heads=2,
                                   vocab_size=160, max_position_embeddings=64, rms_norm_eps=1e-6,
                                   rope_parameters={"rope_type": "default", "rope_theta": 1000000.0}, tie_word_embeddings=False,
                                   use_sliding_window=False, attn_implementation="eager")
    m = transformers.Qwen2ForCausalLM(cfg).eval()
    seeded_weights(m, 104)
    assert m.model.layers[0].self_attn.q_proj.bias is not None
    lib_logits, lib_ids = library_run(m, PROMPT, len(PROMPT) - 1 + N_GREEDY)
    data = llama_family_gguf(m, "qwen2", permute=False)
    compare(lib_logits, lib_ids, *oracle_llama_run(data, b"qwen2", 1, 1, PROMPT, lib_ids.size), "qwen2")
    # permuted file + permuted biases under the adjacent-pair rotation: the same function again, so bias placement is
    # checked under both pairings
    data = llama_family_gguf(m, "qwen2", permute=True)
    compare(lib_logits, lib_ids, *oracle_llama_run(data, b"qwen2", 1, 0, PROMPT, lib_ids.size), "qwen2, permuted")


def test_gpt2_forward():
    """gpt2/cpu.rs:225-383: token + learned position rows, LayerNorm (eps 1e-5) with gain and bias, fused qkv with bias,
    attention, projections with bias into the residual, tanh-GELU, final LayerNorm, output matrix tied to wte; the
    vocabulary is not a multiple of four."""
    cfg = transformers.GPT2Config(n_embd=64, n_layer=3, n_head=4, n_positions=64, vocab_size=131, n_inner=None, activation_function="gelu_new",
                                  layer_norm_epsilon=1e-5, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0, bos_token_id=0, eos_token_id=0,
                                  attn_implementation="eager")
    m = transformers.GPT2LMHeadModel(cfg).eval()
    # (the output matrix is the embedding matrix: with small layer weights every token predicts itself for ever, so
    # the layers and the position rows get more weight than the embeddings)
    seeded_weights(m, 105, std=0.35, std_of={"wte": 0.1, "wpe": 0.3})
    assert m.lm_head.weight.data_ptr() == m.transformer.wte.weight.data_ptr()
    prompt = [3, 77, 130, 9, 21, 0, 64]
    lib_logits, lib_ids = library_run(m, prompt, len(prompt) - 1 + N_GREEDY)
    sd = {k: v.detach().numpy() for k, v in m.state_dict().items()}
    w = gw.GgufWriter()
    w.add_meta("general.architecture", gw.T_STR, "gpt2")
    w.add_meta("general.file_type", gw.T_U32, 0)
    w.add_meta("gpt2.context_length", gw.T_U32, 64)
    w.add_meta("gpt2.embedding_length", gw.T_U32, 64)
    w.add_meta("gpt2.attention.head_count", gw.T_U32, 4)
    w.add_meta("gpt2.block_count", gw.T_U32, 3)
    w.add_meta("gpt2.feed_forward_length", gw.T_U32, 256)
    w.add_meta("tokenizer.ggml.tokens", gw.T_ARR, [""] * 131, elem_type=gw.T_STR)

    def mat(name, a):                        # [nrows, ncols]
        w.add_tensor(name, [a.shape[1], a.shape[0]], 0, f32(a))

    def vec(name, a):
        w.add_tensor(name, [a.shape[0]], 0, f32(a))

    mat("token_embd.weight", sd["transformer.wte.weight"])
    mat("position_embd.weight", sd["transformer.wpe.weight"])
    for l in range(3):
        hp, p = "transformer.h.%d." % l, "blk.%d." % l
        vec(p + "attn_norm.weight", sd[hp + "ln_1.weight"]); vec(p + "attn_norm.bias", sd[hp + "ln_1.bias"])
        # the library's Conv1D keeps [in, out]; the loader reads [out rows, in columns]
        mat(p + "attn_qkv.weight", sd[hp + "attn.c_attn.weight"].T); vec(p + "attn_qkv.bias", sd[hp + "attn.c_attn.bias"])
        mat(p + "attn_output.weight", sd[hp + "attn.c_proj.weight"].T); vec(p + "attn_output.bias", sd[hp + "attn.c_proj.bias"])
        vec(p + "ffn_norm.weight", sd[hp + "ln_2.weight"]); vec(p + "ffn_norm.bias", sd[hp + "ln_2.bias"])
        mat(p + "ffn_up.weight", sd[hp + "mlp.c_fc.weight"].T); vec(p + "ffn_up.bias", sd[hp + "mlp.c_fc.bias"])
        mat(p + "ffn_down.weight", sd[hp + "mlp.c_proj.weight"].T); vec(p + "ffn_down.bias", sd[hp + "mlp.c_proj.bias"])
    vec("output_norm.weight", sd["transformer.ln_f.weight"]); vec("output_norm.bias", sd["transformer.ln_f.bias"])
    g = OracleGguf(w.to_bytes())
    L = g.L
    om = L.slo_gpt2_from_gguf(g.h, 0)
    assert om
    n = lib_ids.size
    ids = np.zeros(n, np.int32)
    logits = np.zeros((n, 131), np.float32)
    p = np.array(prompt, np.int32)
    assert L.slo_gpt2_generate(om, p.ctypes.data, p.size, 0, n, -1, ids.ctypes.data, logits.ctypes.data) == n
    L.slo_gpt2_free(om); g.close()
    compare(lib_logits, lib_ids, logits, ids, "gpt2")
