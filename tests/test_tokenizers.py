"""Tokenizers behind the C ABI against the CPU restatement, hand-derived cases and an unrelated BPE implementation.

Reference: crates/slai/src/models/llama2/tokenizer.rs, crates/slai/src/models/gpt2/tokenizer.rs,
crates/slai-chat/src/llm.rs:100-164.  Host-only code: no GPU is needed.
"""
import collections
import os
import random
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
from oracle import text_oracle as to  # noqa: E402
from slai_amd import _ffi, gguf_writer as gw  # noqa: E402
from slai_amd.runtime import Gguf, SlaiError, Tokenizer  # noqa: E402


# ------------------------------------------------------------------------------------------------- fixtures
def llama_vocab():
    vocab = ["<unk>", "<s>", "</s>"] + ["<0x%02X>" % b for b in range(256)]
    scores = [0.0] * len(vocab)
    singles = list("abcdefghijklmnopqrstuvwxyz") + ["▁", "<", ">", "/", ".", ",", "!", "A", "B", "é", "\n"]
    for c in singles:
        vocab.append(c)
        scores.append(-100.0)
    merged = [("he", -1.0), ("ll", -2.0), ("hell", -3.0), ("hello", -4.0), ("lo", -5.0), ("▁hello", -6.0), ("▁w", -7.0),
              ("or", -8.0), ("ld", -9.0), ("▁wor", -10.0), ("▁world", -11.0), ("th", -1.5), ("▁th", -2.5), ("▁the", -3.5),
              ("in", -4.5), ("ing", -5.5), ("▁a", -6.5), ("an", -6.5), ("▁▁", -12.0), ("ab", -0.5), ("ba", -0.5)]
    for s, sc in merged:
        vocab.append(s)
        scores.append(sc)
    vocab.append("ab")          # a duplicate string: the later id must win
    scores.append(-0.25)
    return vocab, scores


def llama_gguf_bytes():
    vocab, scores = llama_vocab()
    w = gw.GgufWriter()
    w.add_meta("general.architecture", gw.T_STR, "llama")
    w.add_meta("tokenizer.ggml.model", gw.T_STR, "llama")
    w.add_meta("tokenizer.ggml.tokens", gw.T_ARR, vocab, elem_type=gw.T_STR)
    w.add_meta("tokenizer.ggml.scores", gw.T_ARR, scores, elem_type=gw.T_F32)
    w.add_meta("tokenizer.ggml.bos_token_id", gw.T_U32, 1)
    w.add_meta("tokenizer.ggml.eos_token_id", gw.T_U32, 2)
    w.add_meta("tokenizer.ggml.unknown_token_id", gw.T_U32, 0)
    return w.to_bytes(), vocab, scores


def train_bpe(corpus, n_merges):
    """A plain byte-level BPE trainer (most frequent pair first) to obtain a consistent vocabulary + merge list."""
    b2u = to.bytes_to_unicode()
    import regex
    words = collections.Counter()
    for m in regex.finditer(to.GPT2_PATTERN, corpus):
        words[tuple(b2u[b] for b in m.group(0).encode("utf-8"))] += 1
    merges = []
    for _ in range(n_merges):
        pairs = collections.Counter()
        for w, c in words.items():
            for p in zip(w, w[1:]):
                pairs[p] += c
        if not pairs:
            break
        best = max(sorted(pairs), key=lambda p: pairs[p])
        merges.append(best)
        new = collections.Counter()
        for w, c in words.items():
            out, i = [], 0
            while i < len(w):
                if i + 1 < len(w) and (w[i], w[i + 1]) == best:
                    out.append(w[i] + w[i + 1]); i += 2
                else:
                    out.append(w[i]); i += 1
            new[tuple(out)] += c
        words = new
    vocab = [b2u[b] for b in range(256)] + [a + b for a, b in merges] + ["<|endoftext|>", "<|im_start|>"]
    return vocab, ["%s %s" % m for m in merges]


CORPUS = ("the quick brown fox jumps over the lazy dog. the dog's bark isn't worse than its bite! "
          "hello world, hello there; numbers 123 and 4567 are here. we'll see what they've done, I'm sure. "
          "naïve café über straße 東京 Привет мир. tabs\tand\nnewlines\n\nhappen too. ") * 3


def gpt2_gguf_bytes():
    vocab, merges = train_bpe(CORPUS, 120)
    w = gw.GgufWriter()
    w.add_meta("general.architecture", gw.T_STR, "gpt2")
    w.add_meta("tokenizer.ggml.model", gw.T_STR, "gpt2")
    w.add_meta("tokenizer.ggml.tokens", gw.T_ARR, vocab, elem_type=gw.T_STR)
    w.add_meta("tokenizer.ggml.merges", gw.T_ARR, merges, elem_type=gw.T_STR)
    w.add_meta("tokenizer.ggml.bos_token_id", gw.T_U32, len(vocab) - 2)
    w.add_meta("tokenizer.ggml.eos_token_id", gw.T_U32, len(vocab) - 2)
    return w.to_bytes(), vocab, merges


@pytest.fixture(scope="module")
def llama_tok():
    data, vocab, scores = llama_gguf_bytes()
    g = Gguf(data)
    t = Tokenizer(g)
    yield t, to.LlamaTokenizer(vocab, scores, 1, 2, 0), vocab
    t.close(); g.close()


@pytest.fixture(scope="module")
def gpt2_tok():
    data, vocab, merges = gpt2_gguf_bytes()
    g = Gguf(data)
    t = Tokenizer(g)
    yield t, to.Gpt2Tokenizer(vocab, merges, len(vocab) - 2, len(vocab) - 2), vocab, merges
    t.close(); g.close()


# ------------------------------------------------------------------------------------------------- GGUF arrays / file
def test_gguf_arrays_and_file_mapping(tmp_path):
    data, vocab, scores = llama_gguf_bytes()
    g = Gguf(data)
    assert [b.decode() for b in g.meta_array_str("tokenizer.ggml.tokens")] == vocab
    assert np.array_equal(g.meta_array_f32("tokenizer.ggml.scores"), np.asarray(scores, dtype=np.float32))
    with pytest.raises(SlaiError):
        g.meta_array_f32("tokenizer.ggml.tokens")           # wrong element type
    with pytest.raises(SlaiError):
        g.meta_array_str("no.such.key")
    path = tmp_path / "tok.gguf"
    path.write_bytes(data.tobytes())
    f = Gguf.open(path)
    assert f.version == g.version
    assert f.meta_array_str("tokenizer.ggml.tokens") == g.meta_array_str("tokenizer.ggml.tokens")
    assert f.meta_u32("tokenizer.ggml.eos_token_id") == 2
    f.close(); g.close()
    with pytest.raises(SlaiError) as e:
        Gguf.open(tmp_path / "missing.gguf")
    assert e.value.code == _ffi.E_IO
    (tmp_path / "junk.gguf").write_bytes(b"not a gguf file at all")
    with pytest.raises(SlaiError) as e:
        Gguf.open(tmp_path / "junk.gguf")
    assert e.value.code == _ffi.E_PARSE


def test_dummy_gguf_string_array():
    """The reference's own fixture holds `arr.str = ["hello", "world", "!"]`."""
    path = os.path.join(os.path.dirname(__file__), "golden", "dummy.gguf")
    g = Gguf.open(path)
    keys = [k for k in ("some.parameter.arr.str", "arr.str") if _has(g, k)]
    assert keys, "the fixture's string array was not found"
    assert g.meta_array_str(keys[0]) == [b"hello", b"world", b"!"]
    lines = g.metadata_debug_strings()
    assert len(lines) == 15 and lines == sorted(lines)
    assert any(l.endswith("= array[3]") for l in lines) and any('String("hello world")' in l for l in lines)
    assert any(l.endswith("U8(18)") for l in lines)                 # some.parameter.uint8 = 0x12
    g.close()


def _has(g, key):
    try:
        g.meta_array_len(key)
        return True
    except SlaiError:
        return False


# ------------------------------------------------------------------------------------------------- Llama
def test_llama_hand_derived(llama_tok):
    t, _, vocab = llama_tok
    ix = {s: i for i, s in enumerate(vocab)}               # last duplicate wins, like the reference's map
    assert (t.bos, t.eos, t.unk, t.kind) == (1, 2, 0, _ffi.TOKENIZER_LLAMA)
    assert t.bos_str() == "<s>" and t.eos_str() == "</s>"
    # h e l l o: he(-1) first, then ll(-2), then hell(-3), then hello(-4)
    assert t.encode("hello") == [ix["hello"]]
    # with the flags
    assert t.encode("hello", bos=True, eos=True) == [1, ix["hello"], 2]
    # a space becomes the boundary mark; "▁hello"(-6) only forms once "hello" exists
    assert t.encode(" hello") == [ix["▁hello"]]
    # a character outside the vocabulary falls back to its UTF-8 bytes + 3
    assert t.encode("ü") == [0xC3 + 3, 0xBC + 3]
    # "<s>" and "</s>" typed as text collapse into the special ids
    assert t.encode("<s>hello</s>") == [1, ix["hello"], 2]
    # equal strings: the later id is the one found
    assert t.encode("ab") == [len(vocab) - 1]
    # equal scores: the leftmost pair merges first ("ab" has the best score here, so a|b|a -> ab|a)
    assert t.encode("aba") == [len(vocab) - 1, ix["a"]]
    # decode: boundary mark back to a space; byte tokens to their byte; leading white space dropped after token 1 only
    assert t.decode([ix["▁hello"]]) == " hello"
    assert t.decode([3 + 0x0A]) == "\n"
    assert t.decode([ix["\n"]], prev_token=1) == ""
    assert t.decode([ix["\n"]], prev_token=0) == "\n"
    assert t.decode_bytes([3 + 0xE9]) == "é".encode()      # `byte as char`: U+00E9, not the raw byte
    assert t.encode("") == []


def test_llama_matches_restatement(llama_tok):
    t, ref, vocab = llama_tok
    rng = random.Random(5)
    alphabet = list("abehlorwdthinag ") * 3 + ["<s>", "</s>", "é", "ü", "\n", " ", "  ", "世", ".", "!", "A", "Z", "<", ">", "/"]
    for case in range(300):
        text = "".join(rng.choice(alphabet) for _ in range(rng.randrange(1, 40)))
        for bos, eos in ((False, False), (True, True)):
            got = t.encode(text, bos=bos, eos=eos)
            assert got == ref.encode(text, bos, eos), (case, text)
        ids = t.encode(text)
        prev, want = 0, ""
        for tok in ids:
            want += ref.decode(prev, tok)
            prev = tok
        assert t.decode(ids, prev_token=0) == want
        want1 = "".join(ref.decode(1 if i == 0 else ids[i - 1], tok) for i, tok in enumerate(ids))
        assert t.decode(ids, prev_token=1) == want1


def test_llama_round_trip_ascii(llama_tok):
    t, _, _ = llama_tok
    for text in ("hello world", "the thing in a land", " a  b   c", "what, then!"):
        assert t.decode(t.encode(text)) == text


def test_llama_errors():
    # a vocabulary too small for the byte fallback: the reference would index out of bounds
    w = gw.GgufWriter()
    w.add_meta("tokenizer.ggml.model", gw.T_STR, "llama")
    w.add_meta("tokenizer.ggml.tokens", gw.T_ARR, ["<unk>", "<s>", "</s>", "a"], elem_type=gw.T_STR)
    w.add_meta("tokenizer.ggml.scores", gw.T_ARR, [0.0] * 4, elem_type=gw.T_F32)
    for k, v in (("bos", 1), ("eos", 2), ("unknown", 0)):
        w.add_meta("tokenizer.ggml.%s_token_id" % k, gw.T_U32, v)
    g = Gguf(w.to_bytes())
    t = Tokenizer(g)
    assert t.encode("aa") == [3, 3]
    with pytest.raises(SlaiError):
        t.encode("b")
    with pytest.raises(SlaiError):
        t.encode(b"\xff\xfe")                               # not UTF-8
    with pytest.raises(SlaiError):
        t.decode([99])
    t.close(); g.close()
    # missing metadata
    w = gw.GgufWriter()
    w.add_meta("tokenizer.ggml.model", gw.T_STR, "llama")
    w.add_meta("tokenizer.ggml.tokens", gw.T_ARR, ["a"], elem_type=gw.T_STR)
    g = Gguf(w.to_bytes())
    with pytest.raises(SlaiError):
        Tokenizer(g)
    g.close()
    w = gw.GgufWriter()
    w.add_meta("tokenizer.ggml.model", gw.T_STR, "bert")
    g = Gguf(w.to_bytes())
    with pytest.raises(SlaiError) as e:
        Tokenizer(g)
    assert "Unrecognized tokenizer type" in str(e.value)
    g.close()


# ------------------------------------------------------------------------------------------------- GPT-2
def test_gpt2_byte_table_known_values():
    tab = to.bytes_to_unicode()
    assert tab[ord(" ")] == "Ġ" and tab[ord("\n")] == "Ċ" and tab[0xAD] == "Ń" and tab[0] == "Ā"
    assert tab[ord("A")] == "A" and tab[0xFF] == "ÿ"
    assert len(set(tab.values())) == 256


def test_gpt2_pretokenizer_cases(gpt2_tok):
    """The pattern's alternatives, observed through single-byte tokens (no merges apply to these strings)."""
    t, ref, vocab, _ = gpt2_tok
    for text in ("I'm we'll they've isn't 'd 're", "a  b", "x \n y", "12ab 34 !?", " !!", "it's'", "'", " ", "\t\t x", "東京 и мир", "a b",
                 "tab\there", "end ", "end  ", "  lead", "९९ bottles"):
        assert t.encode(text) == ref.encode(text), text


def test_gpt2_matches_restatement_and_round_trips(gpt2_tok):
    t, ref, vocab, _ = gpt2_tok
    assert t.kind == _ffi.TOKENIZER_GPT2 and t.bos == len(vocab) - 2 and t.bos_str() == "<|endoftext|>"
    rng = random.Random(11)
    words = CORPUS.split() + ["<|endoftext|>", "<|im_start|>", "'s", "'ll", "42", "...", "\n", "\t", "  ", "é", "東", "'"]
    for case in range(300):
        text = "".join(rng.choice(words) + rng.choice(["", " ", " ", "  ", "\n"]) for _ in range(rng.randrange(1, 12)))
        ids = t.encode(text)
        assert ids == ref.encode(text), (case, text)
        assert t.decode(ids) == ref.decode(ids)
        if text.isascii() and "<|" not in text:
            assert t.decode(ids) == text
    # bytes above 0x7F decode to U+0080..U+00FF one by one (`b as char` in the reference)
    ids = t.encode("é")
    assert t.decode(ids) == "Ã©"
    # ids outside the vocabulary are skipped
    assert t.decode([10 ** 6] + ids) == "Ã©"


def test_gpt2_against_tokenizers_library(gpt2_tok):
    """An unrelated implementation of byte-level BPE on the same vocabulary and merges."""
    tk = pytest.importorskip("tokenizers")
    t, ref, vocab, merges = gpt2_tok
    model = tk.models.BPE(vocab={s: i for i, s in enumerate(vocab)}, merges=[tuple(m.split(" ")) for m in merges])
    hf = tk.Tokenizer(model)
    hf.pre_tokenizer = tk.pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=True)
    rng = random.Random(3)
    words = [w for w in CORPUS.split()] + ["'s", "'ll", "42", "...", "é", "東"]
    for case in range(200):
        # single spaces only: the library's pattern treats runs of white space differently (a look-ahead)
        text = " ".join(rng.choice(words) for _ in range(rng.randrange(1, 12)))
        assert t.encode(text) == hf.encode(text).ids, (case, text)
        assert ref.encode(text) == hf.encode(text).ids, (case, text)


def test_gpt2_special_tokens_and_errors(gpt2_tok):
    t, ref, vocab, _ = gpt2_tok
    eot = len(vocab) - 2
    assert t.encode("<|endoftext|>") == [eot]
    assert t.encode("a<|endoftext|>b<|im_start|>") == ref.encode("a<|endoftext|>b<|im_start|>")
    with pytest.raises(SlaiError):
        t.encode("x <nope> y")                              # a <...> span that is not a token: the reference panics
    with pytest.raises(KeyError):
        ref.encode("x <nope> y")
    assert t.encode("1 << 2") == ref.encode("1 << 2")       # no closing bracket: plain text
    assert t.encode("") == []
