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
