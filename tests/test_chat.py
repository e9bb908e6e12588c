"""The headless chat loop (crates/slai-chat/src/{cli,chat_llama2,chat_template,prompt}.rs) over the C ABI."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
from oracle import text_oracle as to  # noqa: E402
from slai_amd import _ffi, gguf_writer as gw  # noqa: E402
from slai_amd.chat import DEFAULT_CHAT_TEMPLATE, ChatLlm, ChatTemplate, Prompt  # noqa: E402
from test_tokenizers import llama_vocab  # noqa: E402


def test_default_template_is_the_llama2_layout():
    t = ChatTemplate(DEFAULT_CHAT_TEMPLATE)
    p = Prompt()
    p.append_user(" hi there ")
    assert t.apply(p, "<s>", "</s>") == "<s>[INST] hi there [/INST]"
    p.append_assistant("hello! ")
    p.append_user("again")
    assert t.apply(p, "<s>", "</s>") == "<s>[INST] hi there [/INST] hello! </s><s>[INST] again [/INST]"
    q = Prompt()
    q.append_system("be brief")
    q.append_user("hi")
    assert t.apply(q, "<s>", "</s>") == "<s>[INST] <<SYS>>\nbe brief\n<</SYS>>\n\nhi [/INST]"


def test_template_from_metadata_sees_the_reference_globals():
    src = "{% for m in messages %}{{ m['role'] }}:{{ m['content'] }}|{% endfor %}{{ bos_token }}{{ eos_token }}{% if add_generation_prompt %}>{% endif %}"
    p = Prompt()
    p.append_user("a")
    p.append_assistant("b")
    assert ChatTemplate(src).apply(p, "B", "E") == "user:a|assistant:b|BE>"
    # templates written for Python's jinja use method calls and indexing, which the reference rewrites into filters
    assert ChatTemplate("{{ messages[0]['content'].split('x')[-1] }}").apply(p, "", "") == "a"


def chat_gguf(eos=2, template=None):
    vocab, scores = llama_vocab()
    tok = dict(model="llama", tokens=vocab, scores=scores, bos=1, eos=eos, unk=0, chat_template=template)
    data = gw.llama_gguf(dim=64, hidden_dim=128, n_layers=2, n_heads=2, n_kv_heads=2, vocab=len(vocab), seq_len=128, wtype=8, seed=9,
                         std=0.4, norm_random=True, tokenizer=tok)
    return data, vocab, scores


@pytest.mark.gpu
def test_chat_turns_follow_the_decode_loop():
    from slai_amd.runtime import Backend, Gguf, Llama2
    data, vocab, scores = chat_gguf()
    b = Backend(0)
    g = Gguf(data)
    ref_tok = to.LlamaTokenizer(vocab, scores, 1, 2, 0)
    seed = 31337
    llm = ChatLlm(b, g, _ffi.KV_F32, 0.7, 0.95, seed, chunk=5)
    prompt = Prompt()
    prompt.append_user("hello world")
    pieces = []
    text, next_pos, n_new, _ = llm.forward(prompt, 0, pieces.append, max_new_tokens=12)
    templated = "<s>[INST] hello world [/INST]"
    toks = ref_tok.encode(templated, False, False)
    assert toks[0] == 1                                            # "<s>" typed in the template becomes the bos id
    # the same tokens come out of one uninterrupted run of the loop on a fresh model
    m = Llama2(b, g, _ffi.MODEL_LLAMA, _ffi.KV_F32)
    ids, _ = m.generate_sampled(np.asarray(toks, np.int32), len(toks) - 1 + 12, 0.7, 0.95, seed)
    m.destroy()
    gen = ids[len(toks) - 1:].tolist()
    if 2 in gen:
        gen = gen[:gen.index(2)]
    assert n_new == len(gen) and n_new > 0
    prev, want = toks[-1], ""
    for t in gen:
        want += ref_tok.decode(prev, t)
        prev = t
    assert text == want == "".join(pieces)
    assert next_pos == len(toks) - 1 + n_new - 1                    # position of the last reported token
    # a second turn resumes there and runs
    prompt.append_assistant(text)
    prompt.append_user("and then")
    text2, next_pos2, n2, _ = llm.forward(prompt, next_pos, max_new_tokens=6)
    assert next_pos2 > next_pos and n2 >= 0
    llm.close(); g.close(); b.close()


@pytest.mark.gpu
def test_chat_stops_at_the_end_token():
    from slai_amd.runtime import Backend, Gguf
    b = Backend(0)
    data, vocab, scores = chat_gguf()
    g = Gguf(data)
    llm = ChatLlm(b, g, _ffi.KV_F32, 0.0, 0.95, 0, chunk=4)          # greedy: the continuation is a fixed sequence
    prompt = Prompt()
    prompt.append_user("the thing")
    text, _, n_new, _ = llm.forward(prompt, 0, max_new_tokens=10)
    toks = llm.tokenizer.encode("<s>[INST] the thing [/INST]")
    ids, _ = llm.model.generate(np.asarray(toks, np.int32), len(toks) - 1 + 10)
    gen = ids[len(toks) - 1:].tolist()
    llm.close(); g.close()
    # make the token that first shows up at step 4 or later the end token of an otherwise identical file
    stop_at = next(k for k in range(3, 10) if gen[k] not in gen[:k])
    data2, _, _ = chat_gguf(eos=gen[stop_at])
    g2 = Gguf(data2)
    llm2 = ChatLlm(b, g2, _ffi.KV_F32, 0.0, 0.95, 0, chunk=4)
    text2, next_pos, n2, _ = llm2.forward(prompt, 0, max_new_tokens=10)
    assert n2 == stop_at and text.startswith(text2) and len(text2) < len(text)
    llm2.close(); g2.close(); b.close()


@pytest.mark.gpu
def test_cli_runs_a_turn_from_a_file(tmp_path, monkeypatch, capsys):
    import io
    from slai_amd import chat
    data, _, _ = chat_gguf()
    path = tmp_path / "tiny.gguf"
    path.write_bytes(data.tobytes())
    monkeypatch.setattr(sys, "stdin", io.StringIO("hello world\n"))
    chat.main([str(path), "--inspect", "--seed", "5", "--kv", "f32"])
    out = capsys.readouterr().out
    assert "GGUF model loaded" in out and "token_embd.weight" in out and "[Assistant]" in out and "tok/s" in out
