"""CPU restatement of the reference's tokenizers and sampler -- TEST INFRASTRUCTURE ONLY.

Nothing outside ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg may import this.

Restated from the reference text:
  * ``LlamaTokenizer``   crates/slai/src/models/llama2/tokenizer.rs:23-179
  * ``Gpt2Tokenizer``    crates/slai/src/models/gpt2/tokenizer.rs:22-216
  * ``Sampler``          crates/slai/src/models/sampler.rs:33-131 (the random draw `coin` is an argument here)

Pinned by tests/test_tokenizers.py and tests/test_oracle_sampler.py:
  * GPT-2 byte table: the published values (space -> U+0120, newline -> U+010A, 0xAD -> U+0143), bijectivity;
  * GPT-2 encode: agreement with the `tokenizers` library's byte-level BPE (an unrelated implementation) on a
    constructed vocabulary, for texts without runs of spaces (its pattern has a look-ahead the reference lacks);
    decode(encode(x)) == x for ASCII text;
  * Llama encode/decode: hand-derived cases (byte fallback, "<s>" collapsing, score order), decode(encode(x)) == x;
  * sampler: closed forms (uniform distribution: index = floor(coin * n); one dominant logit; top-p keeps exactly
    the k largest when probabilities are 2^-i), agreement of `sample_mult` with numpy's cumulative sum + searchsorted.
Parity unpinned: Unicode categories of code points assigned after Unicode 13 (the tables are this interpreter's),
and the exact version of the `regex` crate's tables the reference was built with.
"""
import math

import numpy as np

try:                                    # third-party `regex` knows \\p{L}; the standard `re` does not
    import regex as _regex
except ImportError:                     # pragma: no cover
    _regex = None


# ---------------------------------------------------------------------------------------------- Llama
class LlamaTokenizer:
    def __init__(self, vocab, scores, bos, eos, unk):
        self.vocab = list(vocab)                    # str per id
        self.scores = [np.float32(s) for s in scores]
        self.bos, self.eos, self.unk = bos, eos, unk
        self.index = {}
        for i, s in enumerate(self.vocab):          # tokenizer.rs:37-40: later duplicates replace earlier ones
            self.index[s] = i

    def encode(self, text, bos, eos):               # tokenizer.rs:72-166
        text = text.replace(" ", "▁")
        toks = [self.bos] if bos else []
        for ch in text:
            if ch in self.index:
                toks.append(self.index[ch])
            else:
                toks.extend(b + 3 for b in ch.encode("utf-8"))
        for width, spelled, tid in ((3, "<s>", self.bos), (4, "</s>", self.eos)):
            i = 0
            while i < max(len(toks) - (width - 1), 0):
                if "".join(self.vocab[t] for t in toks[i:i + width]) == spelled:
                    toks[i:i + width] = [tid]
                i += 1
        while len(toks) >= 2:
            best, best_id, best_i = -math.inf, None, None
            for i in range(len(toks) - 1):
                tid = self.index.get(self.vocab[toks[i]] + self.vocab[toks[i + 1]])
                if tid is not None and self.scores[tid] > best:
                    best, best_id, best_i = self.scores[tid], tid, i
            if best_i is None:
                break
            toks[best_i:best_i + 2] = [best_id]
        if eos:
            toks.append(self.eos)
        return toks

    def decode(self, prev, token):                  # tokenizer.rs:168-179
        piece = self.vocab[token]
        if prev == 1:
            piece = piece.lstrip()                  # Python's str.lstrip and Rust's trim_start both use White_Space (+ a few separators below U+20 in Python)
        if piece.startswith("<0x") and len(piece) >= 5:
            try:
                hx = piece[3:5]
                if all(c in "0123456789abcdefABCDEF+" for c in hx) and "+" not in hx[1:]:
                    return chr(int(hx, 16))
            except ValueError:
                pass
        return piece.replace("▁", " ")


# ---------------------------------------------------------------------------------------------- GPT-2
def bytes_to_unicode():                             # gpt2/tokenizer.rs:22-36
    keep = list(range(33, 127)) + list(range(161, 173)) + list(range(174, 256))
    table, extra = {}, 0
    for b in range(256):
        if b in keep:
            table[b] = chr(b)
        else:
            table[b] = chr(256 + extra)
            extra += 1
    return table


GPT2_PATTERN = r"'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+"       # gpt2/tokenizer.rs:73


class Gpt2Tokenizer:
    def __init__(self, vocab, merges, bos, eos):
        self.vocab = list(vocab)
        self.bos, self.eos = bos, eos
        self.encoder = {}
        for i, s in enumerate(self.vocab):
            self.encoder[s] = i
        self.ranks = {}
        for i, line in enumerate(merges):           # :60-70
            a, b = line.split()[:2]
            self.ranks[(a, b)] = i
        self.byte_encoder = bytes_to_unicode()
        self.byte_decoder = {c: b for b, c in self.byte_encoder.items()}
        self.pat = _regex.compile(GPT2_PATTERN)
        self.special = _regex.compile("<[^<>]*>")

    def bpe(self, token):                           # :171-216
        word = list(token)
        while len(word) > 1:
            ranked = [(self.ranks[p], p) for p in set(zip(word, word[1:])) if p in self.ranks]
            if not ranked:
                break
            first, second = min(ranked)[1]
            out, i = [], 0
            while i < len(word):
                if i + 1 < len(word) and word[i] == first and word[i + 1] == second:
                    out.append(first + second)
                    i += 2
                else:
                    out.append(word[i])
                    i += 1
            word = out
        return word

    def _plain(self, text, out):                    # :107-121
        for m in self.pat.finditer(text):
            mapped = "".join(self.byte_encoder[b] for b in m.group(0).encode("utf-8"))
            for piece in self.bpe(mapped):
                if piece in self.encoder:
                    out.append(self.encoder[piece])

    def encode(self, text):                         # :104-144
        out, cursor = [], 0
        for m in self.special.finditer(text):
            if cursor != m.start():
                self._plain(text[cursor:m.start()], out)
            out.append(self.encoder[m.group(0)])    # KeyError where the reference panics
            cursor = m.end()
        if cursor < len(text):
            self._plain(text[cursor:], out)
        return out

    def decode(self, tokens):                       # :154-168
        joined = "".join(self.vocab[t] for t in tokens if 0 <= t < len(self.vocab))
        return "".join(chr(self.byte_decoder[c]) for c in joined if c in self.byte_decoder)


# ---------------------------------------------------------------------------------------------- sampler
def softmax_f32(x):
    """crates/slai/src/ops/softmax.rs:46-59 `run_cpu`: subtract the max, exp, divide by the sum (sequential f32)."""
    x = np.asarray(x, dtype=np.float32)
    m = x.max()
    e = np.exp((x - m).astype(np.float32)).astype(np.float32)
    s = np.float32(0.0)
    for v in e:
        s = np.float32(s + v)
    return (e / s).astype(np.float32)


def sample_mult(prob, coin):                        # sampler.rs:63-78
    cdf = np.float32(0.0)
    for i, p in enumerate(prob):
        cdf = np.float32(cdf + p)
        if np.float32(coin) < cdf:
            return i
    return len(prob) - 1


def sample_topp(prob, topp, coin):                  # sampler.rs:85-131
    n = len(prob)
    cutoff = np.float32((np.float32(1.0) - np.float32(topp)) / np.float32(np.float32(n) - np.float32(1.0)))
    cand = [(np.float32(p), i) for i, p in enumerate(prob) if p >= cutoff]
    cand.sort(key=lambda pi: -pi[0])                # stable: equal probabilities keep index order
    cum, last = np.float32(0.0), len(cand) - 1
    for i, (p, _) in enumerate(cand):
        cum = np.float32(cum + p)
        if cum > np.float32(topp):
            last = i
            break
    r = np.float32(np.float32(coin) * cum)
    cdf = np.float32(0.0)
    for i in range(last + 1):
        cdf = np.float32(cdf + cand[i][0])
        if r < cdf:
            return cand[i][1]
    return cand[last][1]


def sample(logits, temperature, topp, coin):        # sampler.rs:33-53
    logits = np.asarray(logits, dtype=np.float32)
    if temperature == 0.0:
        return int(np.argmax(logits))
    prob = softmax_f32((logits / np.float32(temperature)).astype(np.float32))
    if topp <= 0.0 or topp >= 1.0:
        return sample_mult(prob, coin)
    return sample_topp(prob, topp, coin)


# ---- the same three functions on numpy scans, for vocabularies where the loops above take too long.  `np.cumsum`
# on float32 adds left to right in float32, like the loops; tests/test_oracle_sampler.py checks that they agree.
def _softmax_fast(x):
    x = np.asarray(x, dtype=np.float32)
    e = np.exp((x - x.max()).astype(np.float32)).astype(np.float32)
    return (e / np.cumsum(e, dtype=np.float32)[-1]).astype(np.float32)


def sample_mult_fast(prob, coin):
    cdf = np.cumsum(np.asarray(prob, dtype=np.float32), dtype=np.float32)
    hit = np.nonzero(np.float32(coin) < cdf)[0]
    return int(hit[0]) if hit.size else len(prob) - 1


def sample_topp_fast(prob, topp, coin):
    prob = np.asarray(prob, dtype=np.float32)
    n = prob.size
    cutoff = np.float32((np.float32(1.0) - np.float32(topp)) / np.float32(np.float32(n) - np.float32(1.0)))
    idx = np.nonzero(prob >= cutoff)[0]
    order = idx[np.argsort(-prob[idx], kind="stable")]
    ps = prob[order]
    cum = np.cumsum(ps, dtype=np.float32)
    over = np.nonzero(cum > np.float32(topp))[0]
    last = int(over[0]) if over.size else ps.size - 1
    r = np.float32(np.float32(coin) * cum[last])
    hit = np.nonzero(r < cum[:last + 1])[0]
    return int(order[hit[0]]) if hit.size else int(order[last])


def sample_fast(logits, temperature, topp, coin):
    logits = np.asarray(logits, dtype=np.float32)
    if temperature == 0.0:
        return int(np.argmax(logits))
    prob = _softmax_fast((logits / np.float32(temperature)).astype(np.float32))
    if topp <= 0.0 or topp >= 1.0:
        return sample_mult_fast(prob, coin)
    return sample_topp_fast(prob, topp, coin)
