"""Damaged GGUF files: the parser and the tokenizer constructors must answer with an error (or a valid handle), never
crash or read outside the buffer.  The reference panics on truncation (gguf.rs:722); here that is SLAI_E_PARSE."""
import os
import random
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(__file__), ".."))
from slai_amd.runtime import Gguf, SlaiError, Tokenizer  # noqa: E402
from test_tokenizers import gpt2_gguf_bytes, llama_gguf_bytes  # noqa: E402


def test_mutated_files_are_rejected_or_read_safely():
    rng = random.Random(7)
    here = os.path.dirname(__file__)
    seeds = [np.fromfile(os.path.join(here, "golden", "dummy.gguf"), dtype=np.uint8), llama_gguf_bytes()[0], gpt2_gguf_bytes()[0]]
    parsed = rejected = 0
    for it in range(600):
        data = seeds[it % 3].copy()
        mode = rng.randrange(4)
        if mode == 0:                                              # a few random bytes in the header region
            for _ in range(rng.randrange(1, 8)):
                data[rng.randrange(min(data.size, 4096))] = rng.randrange(256)
        elif mode == 1:                                            # truncation
            data = data[:rng.randrange(1, data.size)]
        elif mode == 2:                                            # a length / count / offset field replaced by an extreme value
            i = rng.randrange(min(data.size, 4096) - 8)
            v = rng.choice([0, 1, 2 ** 32, 2 ** 63, 2 ** 64 - 1, data.size, data.size * 2])
            data[i:i + 8] = np.frombuffer(np.uint64(v).tobytes(), dtype=np.uint8)
        else:                                                      # one flipped bit anywhere
            data[rng.randrange(data.size)] ^= 1 << rng.randrange(8)
        try:
            g = Gguf(data)
        except SlaiError:
            rejected += 1
            continue
        parsed += 1
        try:
            g.metadata_debug_strings()
            g.tensors()
            try:
                t = Tokenizer(g)
            except SlaiError:
                continue
            try:
                t.encode("hello <s> world's 123 \n é")
                t.decode([1, 5, 300])
            except SlaiError:
                pass
            t.close()
        finally:
            g.close()
    assert parsed > 50 and rejected > 50


# ---- model files whose tensors do not fit their hyper-parameters -------------------------------------------------
# The kernels index norm vectors, biases and weight rows by the model's widths; a file with a shorter tensor must be
# refused on the host, before anything is uploaded or launched (the reference unwraps / asserts:
# transformer.rs:202-297, gpt2/cpu.rs:118-190).
import pytest  # noqa: E402

from slai_amd import _ffi  # noqa: E402
from slai_amd import gguf_writer as gw  # noqa: E402


def _llama(hook=None, **kw):
    args = dict(dim=256, hidden_dim=512, n_layers=2, n_heads=4, n_kv_heads=2, vocab=64, seq_len=16, wtype=8, seed=5, bias=True, arch="qwen2")
    args.update(kw)
    return gw.llama_gguf(tensor_hook=hook, **args)


def _short(target, new_len=None):
    def hook(name, dims, t, data):
        if name != target:
            return dims, t, data
        if new_len is None:
            return None                                            # tensor left out
        return [new_len], t, data[:4 * new_len]
    return hook


def test_good_model_files_pass_the_host_check():
    g = Gguf(_llama())
    g.check_llama2(_ffi.MODEL_QWEN2)
    g.close()
    g = Gguf(gw.gpt2_gguf(n_embd=64, n_layer=2, n_head=2, ff_len=128, vocab=50, n_seq=16))
    g.check_gpt2()
    g.close()


@pytest.mark.parametrize("name,new_len", [
    ("blk.0.attn_norm.weight", 255), ("blk.1.ffn_norm.weight", 0), ("output_norm.weight", 128), ("blk.0.attn_q.bias", 128),
    ("blk.1.attn_k.bias", 256), ("blk.0.attn_v.bias", 1), ("blk.1.attn_norm.weight", 512)])
def test_llama_vector_of_the_wrong_length_is_refused(name, new_len):
    g = Gguf(_llama(_short(name, new_len)))
    with pytest.raises(SlaiError) as e:
        g.check_llama2(_ffi.MODEL_QWEN2)
    assert e.value.code == _ffi.E_SHAPE and name in str(e.value)
    g.close()


def test_llama_missing_and_mistyped_tensors_are_refused():
    g = Gguf(_llama(_short("blk.1.ffn_norm.weight")))
    with pytest.raises(SlaiError) as e:
        g.check_llama2(_ffi.MODEL_QWEN2)
    assert e.value.code == _ffi.E_MISSING
    g.close()
    g = Gguf(_llama(lambda n, d, t, x: (d, 1, x[:x.size // 2]) if n == "output_norm.weight" else (d, t, x)))   # f16 norm vector
    with pytest.raises(SlaiError) as e:
        g.check_llama2(_ffi.MODEL_QWEN2)
    assert e.value.code == _ffi.E_TYPE
    g.close()
    # a weight matrix with the model's row count but another width
    g = Gguf(_llama(lambda n, d, t, x: ([d[0] // 2, d[1]], t, x[:x.size // 2]) if n == "blk.0.ffn_gate.weight" else (d, t, x)))
    with pytest.raises(SlaiError) as e:
        g.check_llama2(_ffi.MODEL_QWEN2)
    assert e.value.code == _ffi.E_SHAPE and "ffn_gate" in str(e.value)
    g.close()
    # the architecture's keys missing altogether
    g = Gguf(_llama())
    with pytest.raises(SlaiError) as e:
        g.check_llama2(_ffi.MODEL_LLAMA)
    assert e.value.code == _ffi.E_MISSING
    g.close()


@pytest.mark.parametrize("name,new_len", [
    ("blk.0.attn_norm.weight", 63), ("blk.1.attn_norm.bias", 0), ("blk.0.attn_qkv.bias", 64), ("blk.1.ffn_up.bias", 64),
    ("blk.0.ffn_down.bias", 8), ("output_norm.bias", 32), ("blk.1.attn_output.bias", 65)])
def test_gpt2_vector_of_the_wrong_length_is_refused(name, new_len):
    data = gw.gpt2_gguf(n_embd=64, n_layer=2, n_head=2, ff_len=128, vocab=50, n_seq=16, tensor_hook=_short(name, new_len))
    g = Gguf(data)
    with pytest.raises(SlaiError) as e:
        g.check_gpt2()
    assert e.value.code == _ffi.E_SHAPE and name in str(e.value)
    g.close()
