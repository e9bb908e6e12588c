// Tokenizers read from GGUF metadata: the host-side mirror of
// crates/slai/src/models/llama2/tokenizer.rs (score-driven pair merging with byte fallback) and
// crates/slai/src/models/gpt2/tokenizer.rs (byte-level BPE behind a pre-tokenizing pattern), behind one handle
// like `AnyTokenizer` (crates/slai-chat/src/llm.rs:100-164).
#include "common.h"
#include "host_gguf.h"
#include "unicode_tables.h"

#include <algorithm>
#include <climits>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

using namespace slai;

namespace {

// ---- UTF-8 ----------------------------------------------------------------------------------------------------
// Decodes one scalar value at s[i]; returns its length, or 0 when the bytes are not well-formed UTF-8 (the
// reference takes `&str`, which cannot hold such bytes).
size_t utf8_next(const std::string &s, size_t i, uint32_t &cp) {
    const size_t n = s.size();
    const uint8_t b0 = (uint8_t)s[i];
    if (b0 < 0x80) { cp = b0; return 1; }
    size_t len; uint32_t minv;
    if ((b0 & 0xE0) == 0xC0) { len = 2; cp = b0 & 0x1F; minv = 0x80; }
    else if ((b0 & 0xF0) == 0xE0) { len = 3; cp = b0 & 0x0F; minv = 0x800; }
    else if ((b0 & 0xF8) == 0xF0) { len = 4; cp = b0 & 0x07; minv = 0x10000; }
    else return 0;
    if (i + len > n) return 0;
    for (size_t k = 1; k < len; ++k) {
        const uint8_t b = (uint8_t)s[i + k];
        if ((b & 0xC0) != 0x80) return 0;
        cp = (cp << 6) | (b & 0x3F);
    }
    if (cp < minv || cp > 0x10FFFF || (cp >= 0xD800 && cp <= 0xDFFF)) return 0;
    return len;
}
void utf8_append(std::string &out, uint32_t cp) {
    if (cp < 0x80) out += (char)cp;
    else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
    else if (cp < 0x10000) { out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
    else { out += (char)(0xF0 | (cp >> 18)); out += (char)(0x80 | ((cp >> 12) & 0x3F)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
}
bool utf8_valid(const std::string &s) {
    uint32_t cp;
    for (size_t i = 0; i < s.size();) { const size_t l = utf8_next(s, i, cp); if (!l) return false; i += l; }
    return true;
}

template <size_t N> bool in_ranges(const uint32_t (&r)[N][2], uint32_t cp) {
    size_t lo = 0, hi = N;
    while (lo < hi) {
        const size_t mid = (lo + hi) / 2;
        if (cp < r[mid][0]) hi = mid; else if (cp > r[mid][1]) lo = mid + 1; else return true;
    }
    return false;
}
bool is_letter(uint32_t cp) { return in_ranges(kUnicodeLetterRanges, cp); }
bool is_number(uint32_t cp) { return in_ranges(kUnicodeNumberRanges, cp); }
// the White_Space property: what `\s` (in a Unicode-aware pattern) and `str::trim_start` mean in the reference
bool is_space(uint32_t cp) {
    return (cp >= 0x9 && cp <= 0xD) || cp == 0x20 || cp == 0x85 || cp == 0xA0 || cp == 0x1680 || (cp >= 0x2000 && cp <= 0x200A) ||
           cp == 0x2028 || cp == 0x2029 || cp == 0x202F || cp == 0x205F || cp == 0x3000;
}

const char kLowerOneEighthBlock[] = "\xE2\x96\x81";   // U+2581, the word-boundary mark of the Llama vocabulary

void replace_all(std::string &s, const std::string &from, const std::string &to) {
    std::string out;
    size_t i = 0;
    for (;;) {
        const size_t j = s.find(from, i);
        if (j == std::string::npos) break;
        out.append(s, i, j - i); out += to; i = j + from.size();
    }
    out.append(s, i, std::string::npos);
    s.swap(out);
}

bool gguf_strings(const Gguf &g, const char *key, std::vector<std::string> &out, std::string &err) {
    const GgufMetaValue *v = g.meta(key);
    if (!v || v->type != 9 || v->arr_type != 8) { err = std::string("missing string array '") + key + "'"; return false; }
    out.clear(); out.reserve((size_t)v->arr_len);
    size_t off = (size_t)v->arr_offset;
    for (uint64_t i = 0; i < v->arr_len; ++i) {
        uint64_t n;
        memcpy(&n, g.bytes + off, 8); off += 8;
        out.emplace_back((const char *)g.bytes + off, (size_t)n); off += (size_t)n;
    }
    return true;
}
bool gguf_u32(const Gguf &g, const char *key, uint32_t &out, std::string &err) {
    const GgufMetaValue *v = g.meta(key);
    if (!v || v->type != 4) { err = std::string("missing u32 '") + key + "'"; return false; }
    out = (uint32_t)v->u;
    return true;
}

}  // namespace

struct slai_tokenizer {
    int kind = SLAI_TOKENIZER_LLAMA;
    uint32_t bos = 0, eos = 0, unk = UINT32_MAX;
    std::vector<std::string> vocab;
    std::unordered_map<std::string, uint32_t> index;      // string -> id; of equal strings the last id wins, as HashMap::insert does
    // llama
    std::vector<float> scores;
    // gpt2
    std::string byte_to_str[256];                          // the printable stand-in of each byte, UTF-8 encoded
    std::unordered_map<uint32_t, uint8_t> char_to_byte;
    std::unordered_map<std::string, uint32_t> merge_rank;  // "first second" -> rank
    std::string error;

    int fail(int rc, const std::string &m) { error = m; return rc; }

    // ---- Llama (tokenizer.rs:72-160) -----------------------------------------------------------------------------
    int encode_llama(std::string text, bool add_bos, bool add_eos, std::vector<uint32_t> &tokens) {
        replace_all(text, " ", kLowerOneEighthBlock);                                   // :73
        if (add_bos) tokens.push_back(bos);
        for (size_t i = 0; i < text.size();) {                                          // :80-94
            uint32_t cp;
            const size_t l = utf8_next(text, i, cp);
            auto it = index.find(text.substr(i, l));
            if (it != index.end()) tokens.push_back(it->second);
            else for (size_t k = 0; k < l; ++k) tokens.push_back((uint8_t)text[i + k] + 3u);   // bytes sit after <unk>, <s>, </s>
            i += l;
        }
        for (uint32_t t : tokens)
            if (t >= vocab.size()) return fail(SLAI_E_ARG, "tokenizer: byte fallback outside the vocabulary (the reference indexes out of bounds here)");
        // :96-135: runs of single-character tokens spelling "<s>" / "</s>" collapse into the special ids.  Each scan
        // moves on by one token whether or not it collapsed, and its bound follows the shrinking list.
        collapse(tokens, 3, "<s>", bos);
        collapse(tokens, 4, "</s>", eos);
        // :137-160: merge the adjacent pair whose concatenation has the highest score; of equal scores the leftmost
        while (tokens.size() >= 2) {
            float best = -INFINITY; uint32_t best_id = 0; size_t best_at = SIZE_MAX;
            for (size_t i = 0; i + 1 < tokens.size(); ++i) {
                auto it = index.find(vocab[tokens[i]] + vocab[tokens[i + 1]]);
                if (it != index.end() && scores[it->second] > best) { best = scores[it->second]; best_id = it->second; best_at = i; }
            }
            if (best_at == SIZE_MAX) break;
            tokens[best_at] = best_id;
            tokens.erase(tokens.begin() + best_at + 1);
        }
        if (add_eos) tokens.push_back(eos);
        return SLAI_OK;
    }
    void collapse(std::vector<uint32_t> &tokens, size_t width, const char *spelled, uint32_t id) {
        for (size_t i = 0; i + (width - 1) < tokens.size(); ++i) {
            std::string cat;
            for (size_t k = 0; k < width; ++k) cat += vocab[tokens[i + k]];
            if (cat == spelled) {
                tokens[i] = id;
                tokens.erase(tokens.begin() + i + 1, tokens.begin() + i + width);
            }
        }
    }
    // tokenizer.rs:168-179 `decode(prev_token, token)`
    int decode_llama(uint32_t prev, uint32_t token, std::string &out) {
        if (token >= vocab.size()) return fail(SLAI_E_ARG, "tokenizer: token id outside the vocabulary");
        std::string piece = vocab[token];
        if (prev == 1) {                                                                // literally 1, not `bos` (:170)
            size_t i = 0;
            while (i < piece.size()) {
                uint32_t cp;
                const size_t l = utf8_next(piece, i, cp);
                if (!l || !is_space(cp)) break;
                i += l;
            }
            piece.erase(0, i);
        }
        if (piece.compare(0, 3, "<0x") == 0 && piece.size() >= 5) {                     // :173-177 (shorter pieces panic there)
            // usize::from_str_radix on two characters: hex digits, or '+' and one hex digit
            auto hexv = [](char c) -> int { return c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : -1; };
            const int h = hexv(piece[3]), l = hexv(piece[4]);
            int byte = -1;
            if (h >= 0 && l >= 0) byte = h * 16 + l;
            else if (piece[3] == '+' && l >= 0) byte = l;
            if (byte >= 0) { utf8_append(out, (uint32_t)byte); return SLAI_OK; }        // `byte as u8 as char`
        }
        replace_all(piece, kLowerOneEighthBlock, " ");
        out += piece;
        return SLAI_OK;
    }

    // ---- GPT-2 (gpt2/tokenizer.rs) -----------------------------------------------------------------------------------
    void build_byte_table() {                                                           // :22-36 bytes_to_unicode
        uint32_t next = 256;
        for (uint32_t b = 0; b < 256; ++b) {
            const bool printable = (b >= 33 && b <= 126) || (b >= 161 && b <= 172) || (b >= 174);
            const uint32_t cp = printable ? b : next++;
            utf8_append(byte_to_str[b], cp);
            char_to_byte[cp] = (uint8_t)b;
        }
    }
    // :73 the pattern `'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+`, leftmost-first: returns the end
    // of the match that starts at byte i
    static size_t pretoken_end(const std::string &s, size_t i) {
        static const char *const contractions[] = {"'s", "'t", "'re", "'ve", "'m", "'ll", "'d"};
        for (const char *c : contractions) { const size_t n = strlen(c); if (s.compare(i, n, c) == 0) return i + n; }
        enum Class { LETTER, NUMBER, SPACE, OTHER };
        auto cls = [&](size_t at, size_t &len) {
            uint32_t cp;
            len = utf8_next(s, at, cp);
            return is_letter(cp) ? LETTER : is_number(cp) ? NUMBER : is_space(cp) ? SPACE : OTHER;
        };
        auto run = [&](size_t at, Class want) {                                         // end of the run of `want` at `at`
            while (at < s.size()) { size_t l; if (cls(at, l) != want) break; at += l; }
            return at;
        };
        size_t l0;
        const Class c0 = cls(i, l0);
        // the three " ?X+" alternatives: an optional single space, then a run of one class
        if (s[i] == ' ' && i + 1 < s.size()) {
            size_t l1;
            const Class c1 = cls(i + 1, l1);
            if (c1 != SPACE) return run(i + 1, c1);
        }
        if (c0 != SPACE) return run(i, c0);
        return run(i, SPACE);
    }
    // :171-216 `bpe`: repeatedly merge every occurrence of the lowest-ranked adjacent pair
    void bpe(std::vector<std::string> &word) const {
        while (word.size() > 1) {
            uint32_t best = UINT32_MAX; size_t at = 0;
            for (size_t i = 0; i + 1 < word.size(); ++i) {
                auto it = merge_rank.find(word[i] + " " + word[i + 1]);
                if (it != merge_rank.end() && it->second < best) { best = it->second; at = i; }
            }
            if (best == UINT32_MAX) break;
            const std::string first = word[at], second = word[at + 1];
            std::vector<std::string> merged;
            for (size_t i = 0; i < word.size();) {
                if (i + 1 < word.size() && word[i] == first && word[i + 1] == second) { merged.push_back(first + second); i += 2; }
                else merged.push_back(word[i++]);
            }
            word.swap(merged);
        }
    }
    void encode_gpt2_piece(const std::string &text, size_t b, size_t e, std::vector<uint32_t> &tokens) const {   // :107-121
        const std::string piece = text.substr(b, e - b);       // the pattern sees nothing outside the piece
        for (size_t i = 0; i < piece.size();) {
            const size_t j = pretoken_end(piece, i);
            std::vector<std::string> word;
            for (size_t k = i; k < j; ++k) word.push_back(byte_to_str[(uint8_t)piece[k]]);
            bpe(word);
            for (const std::string &w : word) {
                auto it = index.find(w);
                if (it != index.end()) tokens.push_back(it->second);                    // pieces outside the vocabulary are dropped (:116)
            }
            i = j;
        }
    }
    int encode_gpt2(const std::string &text, std::vector<uint32_t> &tokens) {           // :104-144
        size_t cursor = 0, i = 0;
        while (i < text.size()) {
            // the special-token pattern `<[^<>]*>`
            if (text[i] == '<') {
                size_t j = i + 1;
                while (j < text.size() && text[j] != '<' && text[j] != '>') ++j;
                if (j < text.size() && text[j] == '>') {
                    if (cursor != i) encode_gpt2_piece(text, cursor, i, tokens);
                    auto it = index.find(text.substr(i, j + 1 - i));
                    if (it == index.end()) return fail(SLAI_E_MISSING, "tokenizer: '" + text.substr(i, j + 1 - i) + "' is not in the vocabulary (the reference panics here)");
                    tokens.push_back(it->second);
                    cursor = i = j + 1;
                    continue;
                }
            }
            ++i;
        }
        if (cursor < text.size()) encode_gpt2_piece(text, cursor, text.size(), tokens);
        return SLAI_OK;
    }
    // :154-168 `decode`: stand-in characters back to bytes, each byte then taken as a character of its own
    // (`b as char`), so bytes above 0x7F come out as the two-byte encoding of U+0080..U+00FF
    int decode_gpt2(const int32_t *ids, size_t n, std::string &out) const {
        std::string joined;
        for (size_t k = 0; k < n; ++k)
            if (ids[k] >= 0 && (size_t)ids[k] < vocab.size()) joined += vocab[(size_t)ids[k]];
        for (size_t i = 0; i < joined.size();) {
            uint32_t cp;
            const size_t l = utf8_next(joined, i, cp);
            if (!l) { ++i; continue; }
            auto it = char_to_byte.find(cp);
            if (it != char_to_byte.end()) utf8_append(out, it->second);
            i += l;
        }
        return SLAI_OK;
    }
};

// `AnyTokenizer::from_gguf` (crates/slai-chat/src/llm.rs:106-118) when kind is SLAI_TOKENIZER_AUTO
SLAI_EXPORT int slai_tokenizer_from_gguf(const slai_gguf *g, int kind, slai_tokenizer **out, char *err, size_t err_len) {
    if (!g || !out) return SLAI_E_ARG;
    *out = nullptr;
    auto fail = [&](int rc, const std::string &m) { if (err && err_len) snprintf(err, err_len, "%s", m.c_str()); return rc; };
    if (kind == SLAI_TOKENIZER_AUTO) {
        const GgufMetaValue *v = g->g.meta("tokenizer.ggml.model");
        if (!v || v->type != 8) return fail(SLAI_E_MISSING, "Missing tokenizer.ggml.model");
        if (v->s == "gpt2") kind = SLAI_TOKENIZER_GPT2;
        else if (v->s == "llama") kind = SLAI_TOKENIZER_LLAMA;
        else return fail(SLAI_E_TYPE, "Unrecognized tokenizer type: " + v->s);
    }
    if (kind != SLAI_TOKENIZER_LLAMA && kind != SLAI_TOKENIZER_GPT2) return fail(SLAI_E_ARG, "unknown tokenizer kind");
    slai_tokenizer *t = new slai_tokenizer();
    t->kind = kind;
    std::string e;
    bool ok = gguf_strings(g->g, "tokenizer.ggml.tokens", t->vocab, e) && gguf_u32(g->g, "tokenizer.ggml.bos_token_id", t->bos, e) &&
              gguf_u32(g->g, "tokenizer.ggml.eos_token_id", t->eos, e);
    if (ok && kind == SLAI_TOKENIZER_LLAMA) {                                           // llama2/tokenizer.rs:23-52
        ok = gguf_u32(g->g, "tokenizer.ggml.unknown_token_id", t->unk, e);
        const GgufMetaValue *v = g->g.meta("tokenizer.ggml.scores");
        if (ok && (!v || v->type != 9 || v->arr_type != 6)) { ok = false; e = "missing f32 array 'tokenizer.ggml.scores'"; }
        if (ok) {
            t->scores.resize((size_t)v->arr_len);
            if (v->arr_len) memcpy(t->scores.data(), g->g.bytes + v->arr_offset, (size_t)v->arr_len * sizeof(float));
            if (t->scores.size() < t->vocab.size()) { ok = false; e = "tokenizer.ggml.scores is shorter than tokenizer.ggml.tokens"; }
        }
    }
    if (ok && kind == SLAI_TOKENIZER_GPT2) {                                            // gpt2/tokenizer.rs:55-100
        std::vector<std::string> merges;
        ok = gguf_strings(g->g, "tokenizer.ggml.merges", merges, e);
        for (size_t i = 0; ok && i < merges.size(); ++i) {
            // `split_whitespace`: the first two fields of the line
            std::vector<std::string> fields;
            const std::string &line = merges[i];
            for (size_t p = 0; p < line.size() && fields.size() < 2;) {
                uint32_t cp; size_t l = utf8_next(line, p, cp);
                if (!l) { l = 1; cp = 0xFFFD; }
                if (is_space(cp)) { p += l; continue; }
                size_t q = p;
                while (q < line.size()) { uint32_t c2; size_t l2 = utf8_next(line, q, c2); if (!l2) { l2 = 1; c2 = 0xFFFD; } if (is_space(c2)) break; q += l2; }
                fields.push_back(line.substr(p, q - p));
                p = q;
            }
            if (fields.size() < 2) { ok = false; e = "tokenizer.ggml.merges: line " + std::to_string(i) + " has fewer than two fields"; break; }
            t->merge_rank[fields[0] + " " + fields[1]] = (uint32_t)i;
        }
        t->build_byte_table();
    }
    if (ok && (t->bos >= t->vocab.size() || t->eos >= t->vocab.size())) { ok = false; e = "bos / eos token id outside the vocabulary"; }
    if (!ok) { delete t; return fail(SLAI_E_MISSING, e); }
    for (size_t i = 0; i < t->vocab.size(); ++i) t->index[t->vocab[i]] = (uint32_t)i;
    *out = t;
    return SLAI_OK;
}
SLAI_EXPORT void slai_tokenizer_free(slai_tokenizer *t) { delete t; }
SLAI_EXPORT int slai_tokenizer_kind(const slai_tokenizer *t) { return t ? t->kind : SLAI_E_ARG; }
SLAI_EXPORT uint32_t slai_tokenizer_bos(const slai_tokenizer *t) { return t ? t->bos : UINT32_MAX; }
SLAI_EXPORT uint32_t slai_tokenizer_eos(const slai_tokenizer *t) { return t ? t->eos : UINT32_MAX; }
SLAI_EXPORT uint32_t slai_tokenizer_unk(const slai_tokenizer *t) { return t ? t->unk : UINT32_MAX; }
SLAI_EXPORT uint32_t slai_tokenizer_vocab_size(const slai_tokenizer *t) { return t ? (uint32_t)t->vocab.size() : 0; }
SLAI_EXPORT const char *slai_tokenizer_last_error(const slai_tokenizer *t) { return t ? t->error.c_str() : ""; }
// `bos_str` / `eos_str` and the vocabulary in general: bytes (not NUL-terminated) and length of token `id`
SLAI_EXPORT int slai_tokenizer_token_str(const slai_tokenizer *t, uint32_t id, const char **ptr, size_t *len) {
    if (!t || id >= t->vocab.size()) return SLAI_E_ARG;
    if (ptr) *ptr = t->vocab[id].data();
    if (len) *len = t->vocab[id].size();
    return SLAI_OK;
}
// `AnyTokenizer::encode(text, bos, eos)` (llm.rs:156-162): the GPT-2 tokenizer ignores the two flags
SLAI_EXPORT int slai_tokenizer_encode(slai_tokenizer *t, const char *text, size_t text_len, int bos, int eos, int32_t *out,
                                      size_t capacity, size_t *count) {
    if (!t || (!text && text_len) || !count) return SLAI_E_ARG;
    const std::string s(text ? text : "", text_len);
    if (!utf8_valid(s)) return t->fail(SLAI_E_ARG, "tokenizer: the text is not valid UTF-8");
    std::vector<uint32_t> tokens;
    const int rc = t->kind == SLAI_TOKENIZER_LLAMA ? t->encode_llama(s, bos != 0, eos != 0, tokens) : t->encode_gpt2(s, tokens);
    if (rc) return rc;
    *count = tokens.size();
    if (tokens.size() > capacity) return t->fail(SLAI_E_SHAPE, "tokenizer: the output holds fewer ids than the text produces");
    for (size_t i = 0; i < tokens.size(); ++i) out[i] = (int32_t)tokens[i];
    return SLAI_OK;
}
// `AnyTokenizer::decode(prev_token, token)` (llm.rs:149-154) over a run of tokens: the Llama tokenizer decodes token i
// with token i-1 (`prev_token` for the first) as its predecessor, the GPT-2 tokenizer decodes the run as a whole.
// The text is not NUL-terminated; `len` receives its length even when it does not fit.
SLAI_EXPORT int slai_tokenizer_decode(slai_tokenizer *t, const int32_t *tokens, size_t n, int32_t prev_token, char *out, size_t capacity,
                                      size_t *len) {
    if (!t || (!tokens && n) || !len) return SLAI_E_ARG;
    std::string s;
    if (t->kind == SLAI_TOKENIZER_LLAMA) {
        uint32_t prev = (uint32_t)prev_token;
        for (size_t i = 0; i < n; ++i) {
            if (tokens[i] < 0) return t->fail(SLAI_E_ARG, "tokenizer: negative token id");
            const int rc = t->decode_llama(prev, (uint32_t)tokens[i], s);
            if (rc) return rc;
            prev = (uint32_t)tokens[i];
        }
    } else {
        t->decode_gpt2(tokens, n, s);
    }
    *len = s.size();
    if (s.size() > capacity) return t->fail(SLAI_E_SHAPE, "tokenizer: the output buffer is shorter than the text");
    if (s.size()) memcpy(out, s.data(), s.size());
    return SLAI_OK;
}
