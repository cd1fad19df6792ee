// Tokenizers of the two model families (host code, no GPU involved):
//   LlamaTokenizer  models/llama2/tokenizer.rs:8-180 of the reference: characters
//                   looked up in the vocabulary (bytes + 3 as fallback), "<s>" /
//                   "</s>" spotted, then the best-scoring adjacent pair merged until
//                   none is left;
//   Gpt2Tokenizer   models/gpt2/tokenizer.rs:13-217: special "<...>" strings, the
//                   pre-tokenizer pattern, byte-to-unicode mapping, ranked BPE merges.
// Both keep the reference's behaviour where it is peculiar (noted at each place).
#include <algorithm>
#include <cmath>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "common.h"
#include "unicode_tables.h"

using namespace wgml;

struct wgml_tokenizer {
    int kind = 0;  // 0 Llama, 1 GPT-2
    uint32_t bos = 0, eos = 0, unk = 0;
    std::vector<std::string> vocab;
    std::vector<float> scores;
    std::unordered_map<std::string, uint32_t> index;  // later duplicates win, as HashMap::insert
    // GPT-2
    std::unordered_map<std::string, uint32_t> merges;  // "first second" -> rank
    uint32_t byte_to_cp[256];
    std::unordered_map<uint32_t, uint8_t> cp_to_byte;
};

namespace {

// ---- UTF-8 ------------------------------------------------------------------
// Decodes one scalar at s[i]; malformed bytes come out one at a time as U+FFFD
// (what String::from_utf8_lossy would have made of them before the reference saw them).
uint32_t utf8_next(const char *s, size_t n, size_t &i) {
    const uint8_t c = (uint8_t)s[i];
    auto cont = [&](size_t k) { return i + k < n && ((uint8_t)s[i + k] & 0xC0) == 0x80; };
    if (c < 0x80) {
        i += 1;
        return c;
    }
    if ((c & 0xE0) == 0xC0 && c >= 0xC2 && cont(1)) {
        const uint32_t cp = ((c & 0x1Fu) << 6) | ((uint8_t)s[i + 1] & 0x3Fu);
        i += 2;
        return cp;
    }
    if ((c & 0xF0) == 0xE0 && cont(1) && cont(2)) {
        const uint32_t cp = ((c & 0x0Fu) << 12) | (((uint8_t)s[i + 1] & 0x3Fu) << 6) |
                            ((uint8_t)s[i + 2] & 0x3Fu);
        if (cp >= 0x800 && !(cp >= 0xD800 && cp <= 0xDFFF)) {
            i += 3;
            return cp;
        }
    }
    if ((c & 0xF8) == 0xF0 && cont(1) && cont(2) && cont(3)) {
        const uint32_t cp = ((c & 0x07u) << 18) | (((uint8_t)s[i + 1] & 0x3Fu) << 12) |
                            (((uint8_t)s[i + 2] & 0x3Fu) << 6) | ((uint8_t)s[i + 3] & 0x3Fu);
        if (cp >= 0x10000 && cp <= 0x10FFFF) {
            i += 4;
            return cp;
        }
    }
    i += 1;
    return 0xFFFD;
}

void utf8_append(std::string &out, uint32_t cp) {
    if (cp < 0x80) {
        out.push_back((char)cp);
    } else if (cp < 0x800) {
        out.push_back((char)(0xC0 | (cp >> 6)));
        out.push_back((char)(0x80 | (cp & 0x3F)));
    } else if (cp < 0x10000) {
        out.push_back((char)(0xE0 | (cp >> 12)));
        out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
        out.push_back((char)(0x80 | (cp & 0x3F)));
    } else {
        out.push_back((char)(0xF0 | (cp >> 18)));
        out.push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
        out.push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
        out.push_back((char)(0x80 | (cp & 0x3F)));
    }
}

bool in_ranges(const uint32_t (*r)[2], uint32_t count, uint32_t cp) {
    uint32_t lo = 0, hi = count;
    while (lo < hi) {
        const uint32_t mid = (lo + hi) / 2;
        if (cp < r[mid][0])
            hi = mid;
        else if (cp > r[mid][1])
            lo = mid + 1;
        else
            return true;
    }
    return false;
}
bool is_letter(uint32_t cp) { return in_ranges(kUnicodeLetters, kUnicodeLetters_count, cp); }
bool is_number(uint32_t cp) { return in_ranges(kUnicodeNumbers, kUnicodeNumbers_count, cp); }
// White_Space: \s of the pattern and what str::trim_start removes
bool is_space(uint32_t cp) {
    return (cp >= 0x09 && cp <= 0x0D) || cp == 0x20 || cp == 0x85 || cp == 0xA0 || cp == 0x1680 ||
           (cp >= 0x2000 && cp <= 0x200A) || cp == 0x2028 || cp == 0x2029 || cp == 0x202F ||
           cp == 0x205F || cp == 0x3000;
}

int copy_out(const std::string &s, char *buf, uint64_t cap, uint64_t *n_out) {
    if (n_out) *n_out = s.size();
    if (buf && cap) memcpy(buf, s.data(), std::min<uint64_t>(cap, s.size()));
    return WGML_OK;
}
int copy_ids(const std::vector<uint32_t> &ids, uint32_t *out, uint64_t cap, uint64_t *n_out) {
    if (n_out) *n_out = ids.size();
    if (out && cap) memcpy(out, ids.data(), std::min<uint64_t>(cap, ids.size()) * sizeof(uint32_t));
    return WGML_OK;
}

int fill_vocab(wgml_tokenizer *t, const char *tokens, const uint64_t *offsets, uint32_t n) {
    t->vocab.resize(n);
    for (uint32_t i = 0; i < n; ++i) {
        if (offsets[i + 1] < offsets[i])
            return set_error(WGML_E_INVALID, "tokenizer: token offsets must not decrease (at %u)", i);
        t->vocab[i].assign(tokens + offsets[i], (size_t)(offsets[i + 1] - offsets[i]));
        t->index[t->vocab[i]] = i;
    }
    return WGML_OK;
}

// ---- GPT-2 ------------------------------------------------------------------
// bytes_to_unicode (tokenizer.rs:21-36): printable bytes map to themselves, the
// other 68 to U+0100 onwards in byte order.
void build_byte_map(wgml_tokenizer *t) {
    bool keep[256] = {false};
    for (int b = 33; b <= 126; ++b) keep[b] = true;
    for (int b = 161; b <= 172; ++b) keep[b] = true;
    for (int b = 174; b <= 255; ++b) keep[b] = true;
    uint32_t n = 0;
    for (int b = 0; b < 256; ++b) {
        t->byte_to_cp[b] = keep[b] ? (uint32_t)b : 256 + n++;
        t->cp_to_byte[t->byte_to_cp[b]] = (uint8_t)b;
    }
}

// One match of 's|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+
// (tokenizer.rs:75) starting at scalar index p of cps; returns the index after it.
// Alternatives are tried in the order written, each one greedy: the semantics of
// the regex crate's leftmost-first matching.
size_t pretoken_end(const std::vector<uint32_t> &cps, size_t p) {
    const size_t n = cps.size();
    auto at = [&](size_t i) { return i < n ? cps[i] : 0u; };
    if (cps[p] == '\'') {
        const uint32_t a = at(p + 1), b = at(p + 2);
        if (a == 's' || a == 't') return p + 2;
        if ((a == 'r' && b == 'e') || (a == 'v' && b == 'e')) return p + 3;
        if (a == 'm') return p + 2;
        if (a == 'l' && b == 'l') return p + 3;
        if (a == 'd') return p + 2;
    }
    auto is_other = [&](uint32_t c) { return !is_space(c) && !is_letter(c) && !is_number(c); };
    auto run = [&](size_t i, auto pred) {
        while (i < n && pred(cps[i])) ++i;
        return i;
    };
    // " ?X+": with the optional space when a member of X follows it, else without
    const size_t q = (cps[p] == ' ' && p + 1 < n) ? p + 1 : p;
    if (q > p && is_letter(cps[q])) return run(q, is_letter);
    if (is_letter(cps[p])) return run(p, is_letter);
    if (q > p && is_number(cps[q])) return run(q, is_number);
    if (is_number(cps[p])) return run(p, is_number);
    if (q > p && is_other(cps[q])) return run(q, is_other);
    if (is_other(cps[p])) return run(p, is_other);
    return run(p, is_space);  // every scalar is a letter, a number, white space or "other"
}

// bpe (tokenizer.rs:168-216): the adjacent pair with the lowest merge rank is merged
// at all its occurrences, left to right, until no pair has a rank.
std::vector<std::string> bpe(const wgml_tokenizer *t, const std::vector<std::string> &symbols) {
    std::vector<std::string> word = symbols;
    while (word.size() > 1) {
        uint32_t best = UINT32_MAX;
        size_t best_i = 0;
        for (size_t i = 0; i + 1 < word.size(); ++i) {
            auto it = t->merges.find(word[i] + " " + word[i + 1]);
            if (it != t->merges.end() && it->second < best) {
                best = it->second;
                best_i = i;
            }
        }
        if (best == UINT32_MAX) break;
        const std::string first = word[best_i], second = word[best_i + 1];
        std::vector<std::string> next;
        for (size_t i = 0; i < word.size();) {
            if (word[i] == first && i + 1 < word.size() && word[i + 1] == second) {
                next.push_back(first + second);
                i += 2;
            } else {
                next.push_back(word[i]);
                i += 1;
            }
        }
        word.swap(next);
    }
    return word;
}

int gpt2_tokenize_piece(const wgml_tokenizer *t, const char *s, size_t n, std::vector<uint32_t> &out) {
    std::vector<uint32_t> cps;
    std::vector<size_t> starts;  // byte offset of every scalar, plus the end
    for (size_t i = 0; i < n;) {
        starts.push_back(i);
        cps.push_back(utf8_next(s, n, i));
    }
    starts.push_back(n);
    for (size_t p = 0; p < cps.size();) {
        const size_t e = pretoken_end(cps, p);
        // the match's bytes, each as its stand-in character
        std::vector<std::string> symbols;
        for (size_t b = starts[p]; b < starts[e]; ++b) {
            std::string sym;
            utf8_append(sym, t->byte_to_cp[(uint8_t)s[b]]);
            symbols.push_back(sym);
        }
        for (const std::string &piece : bpe(t, symbols)) {
            auto it = t->index.find(piece);
            if (it != t->index.end()) out.push_back(it->second);  // unknown pieces are dropped
        }
        p = e;
    }
    return WGML_OK;
}

}  // namespace

extern "C" {

int wgml_llama_tokenizer_create(const char *tokens, const uint64_t *offsets, uint32_t n_tokens,
                                const float *scores, uint32_t bos, uint32_t eos, uint32_t unk,
                                wgml_tokenizer **out) {
    WGML_REQUIRE(tokens && offsets && scores && out, "wgml_llama_tokenizer_create: null argument");
    WGML_REQUIRE(n_tokens > 0 && bos < n_tokens && eos < n_tokens && unk < n_tokens,
                 "wgml_llama_tokenizer_create: bos/eos/unk outside the %u tokens", n_tokens);
    wgml_tokenizer *t = new wgml_tokenizer();
    t->kind = 0;
    t->bos = bos;
    t->eos = eos;
    t->unk = unk;
    if (int rc = fill_vocab(t, tokens, offsets, n_tokens)) {
        delete t;
        return rc;
    }
    t->scores.assign(scores, scores + n_tokens);
    *out = t;
    return WGML_OK;
}

int wgml_gpt2_tokenizer_create(const char *tokens, const uint64_t *token_offsets, uint32_t n_tokens,
                               const char *merges, const uint64_t *merge_offsets, uint32_t n_merges,
                               uint32_t bos, uint32_t eos, wgml_tokenizer **out) {
    WGML_REQUIRE(tokens && token_offsets && out && (n_merges == 0 || (merges && merge_offsets)),
                 "wgml_gpt2_tokenizer_create: null argument");
    WGML_REQUIRE(n_tokens > 0 && bos < n_tokens && eos < n_tokens,
                 "wgml_gpt2_tokenizer_create: bos/eos outside the %u tokens", n_tokens);
    wgml_tokenizer *t = new wgml_tokenizer();
    t->kind = 1;
    t->bos = bos;
    t->eos = eos;
    if (int rc = fill_vocab(t, tokens, token_offsets, n_tokens)) {
        delete t;
        return rc;
    }
    build_byte_map(t);
    for (uint32_t i = 0; i < n_merges; ++i) {
        // "first second": split at white space (tokenizer.rs:61-68)
        const std::string line(merges + merge_offsets[i],
                               (size_t)(merge_offsets[i + 1] - merge_offsets[i]));
        std::vector<std::string> parts;
        for (size_t a = 0; a < line.size();) {
            size_t k = a;
            const uint32_t cp = utf8_next(line.data(), line.size(), k);
            if (is_space(cp)) {
                a = k;
                continue;
            }
            size_t b = a;
            while (b < line.size()) {
                size_t k2 = b;
                if (is_space(utf8_next(line.data(), line.size(), k2))) break;
                b = k2;
            }
            parts.push_back(line.substr(a, b - a));
            a = b;
        }
        if (parts.size() < 2) {
            delete t;
            return set_error(WGML_E_INVALID, "wgml_gpt2_tokenizer_create: merge %u is not a pair", i);
        }
        t->merges[parts[0] + " " + parts[1]] = i;  // a repeated pair keeps its last rank
    }
    *out = t;
    return WGML_OK;
}

int wgml_tokenizer_destroy(wgml_tokenizer *t) {
    delete t;
    return WGML_OK;
}

uint32_t wgml_tokenizer_vocab_size(const wgml_tokenizer *t) { return t ? (uint32_t)t->vocab.size() : 0; }
uint32_t wgml_tokenizer_bos(const wgml_tokenizer *t) { return t ? t->bos : 0; }
uint32_t wgml_tokenizer_eos(const wgml_tokenizer *t) { return t ? t->eos : 0; }
uint32_t wgml_tokenizer_unk(const wgml_tokenizer *t) { return t ? t->unk : 0; }

int wgml_tokenizer_token(const wgml_tokenizer *t, uint32_t id, const char **str, uint64_t *len) {
    WGML_REQUIRE(t && str && len, "wgml_tokenizer_token: null argument");
    WGML_REQUIRE(id < t->vocab.size(), "wgml_tokenizer_token: id %u outside the %zu tokens", id,
                 t->vocab.size());
    *str = t->vocab[id].data();
    *len = t->vocab[id].size();
    return WGML_OK;
}

int wgml_llama_tokenizer_encode(const wgml_tokenizer *t, const char *text, uint64_t text_len,
                                int bos, int eos, uint32_t *out, uint64_t cap, uint64_t *n_out) {
    WGML_REQUIRE(t && (text || text_len == 0) && n_out, "wgml_llama_tokenizer_encode: null argument");
    WGML_REQUIRE(t->kind == 0, "wgml_llama_tokenizer_encode: not a Llama tokenizer");
    const size_t nv = t->vocab.size();
    std::vector<uint32_t> tokens;
    if (bos) tokens.push_back(t->bos);
    // every space becomes U+2581; every character its own token, or its bytes + 3
    for (size_t i = 0; i < text_len;) {
        uint32_t cp = utf8_next(text, (size_t)text_len, i);
        if (cp == ' ') cp = 0x2581;
        std::string ch;
        utf8_append(ch, cp);
        auto it = t->index.find(ch);
        if (it != t->index.end()) {
            tokens.push_back(it->second);
        } else {
            for (unsigned char b : ch) {
                WGML_REQUIRE((size_t)b + 3 < nv,
                             "LlamaTokenizer::encode: byte fallback %u outside the %zu tokens", b + 3, nv);
                tokens.push_back((uint32_t)b + 3);
            }
        }
    }
    // "<s>" / "</s>" written out in the text: three (four) consecutive tokens whose
    // strings concatenate to it become the special token.  The scan moves on by one
    // position after every test, replaced or not (tokenizer.rs:95-133).
    for (size_t i = 0; i + 2 < tokens.size(); ++i) {
        if (t->vocab[tokens[i]] + t->vocab[tokens[i + 1]] + t->vocab[tokens[i + 2]] == "<s>") {
            tokens[i] = t->bos;
            tokens.erase(tokens.begin() + i + 1, tokens.begin() + i + 3);
        }
    }
    for (size_t i = 0; i + 3 < tokens.size(); ++i) {
        if (t->vocab[tokens[i]] + t->vocab[tokens[i + 1]] + t->vocab[tokens[i + 2]] +
                t->vocab[tokens[i + 3]] == "</s>") {
            tokens[i] = t->eos;
            tokens.erase(tokens.begin() + i + 1, tokens.begin() + i + 4);
        }
    }
    // The reference's merge loop indexes tokens.len() - 1 and panics on an empty list.
    WGML_REQUIRE(!tokens.empty(), "LlamaTokenizer::encode: nothing to encode (empty text, no bos)");
    // merge the best-scoring adjacent pair until no pair is in the vocabulary; of equal
    // scores the leftmost pair wins (strict comparison, tokenizer.rs:136-160)
    for (;;) {
        float best_score = -INFINITY;
        uint32_t best_id = 0;
        size_t best_idx = SIZE_MAX;
        for (size_t i = 0; i + 1 < tokens.size(); ++i) {
            auto it = t->index.find(t->vocab[tokens[i]] + t->vocab[tokens[i + 1]]);
            if (it != t->index.end() && t->scores[it->second] > best_score) {
                best_score = t->scores[it->second];
                best_id = it->second;
                best_idx = i;
            }
        }
        if (best_idx == SIZE_MAX) break;
        tokens[best_idx] = best_id;
        tokens.erase(tokens.begin() + best_idx + 1);
    }
    if (eos) tokens.push_back(t->eos);
    return copy_ids(tokens, out, cap, n_out);
}

int wgml_llama_tokenizer_decode(const wgml_tokenizer *t, uint32_t prev_token, uint32_t token,
                                char *buf, uint64_t cap, uint64_t *n_out) {
    WGML_REQUIRE(t && n_out, "wgml_llama_tokenizer_decode: null argument");
    WGML_REQUIRE(t->kind == 0, "wgml_llama_tokenizer_decode: not a Llama tokenizer");
    WGML_REQUIRE(token < t->vocab.size(), "LlamaTokenizer::decode: token %u outside the %zu tokens",
                 token, t->vocab.size());
    std::string piece = t->vocab[token];
    if (prev_token == 1) {  // after <s> (id 1 is hard-coded, tokenizer.rs:170): drop leading white space
        size_t i = 0;
        while (i < piece.size()) {
            size_t k = i;
            if (!is_space(utf8_next(piece.data(), piece.size(), k))) break;
            i = k;
        }
        piece.erase(0, i);
    }
    if (piece.compare(0, 3, "<0x") == 0 && piece.size() >= 5) {
        auto hexval = [](char c) {
            if (c >= '0' && c <= '9') return c - '0';
            if (c >= 'a' && c <= 'f') return c - 'a' + 10;
            if (c >= 'A' && c <= 'F') return c - 'A' + 10;
            return -1;
        };
        const int h = hexval(piece[3]), l = hexval(piece[4]);
        if (h >= 0 && l >= 0) {
            // byte_pieces[b] is the *character* U+00b (tokenizer.rs:36,175): bytes from
            // 0x80 up come out as two-byte UTF-8, not as the raw byte
            std::string s;
            utf8_append(s, (uint32_t)(h * 16 + l));
            return copy_out(s, buf, cap, n_out);
        }
    }
    std::string s;
    for (size_t i = 0; i < piece.size();) {
        if (piece.compare(i, 3, "\xE2\x96\x81") == 0) {
            s.push_back(' ');
            i += 3;
        } else {
            s.push_back(piece[i++]);
        }
    }
    return copy_out(s, buf, cap, n_out);
}

int wgml_gpt2_tokenizer_encode(const wgml_tokenizer *t, const char *text, uint64_t text_len,
                               uint32_t *out, uint64_t cap, uint64_t *n_out) {
    WGML_REQUIRE(t && (text || text_len == 0) && n_out, "wgml_gpt2_tokenizer_encode: null argument");
    WGML_REQUIRE(t->kind == 1, "wgml_gpt2_tokenizer_encode: not a GPT-2 tokenizer");
    std::vector<uint32_t> ids;
    // "<[^<>]*>" marks a special token, which must be in the vocabulary as it is
    // written (the reference indexes its map and panics otherwise, tokenizer.rs:128-134)
    size_t cursor = 0, i = 0;
    const size_t n = (size_t)text_len;
    while (i < n) {
        if (text[i] != '<') {
            ++i;
            continue;
        }
        size_t j = i + 1;
        while (j < n && text[j] != '<' && text[j] != '>') ++j;
        if (j < n && text[j] == '>') {
            if (cursor != i) WGML_TRY(gpt2_tokenize_piece(t, text + cursor, i - cursor, ids));
            const std::string special(text + i, j + 1 - i);
            auto it = t->index.find(special);
            WGML_REQUIRE(it != t->index.end(), "Gpt2Tokenizer::encode: '%s' is not in the vocabulary",
                         special.c_str());
            ids.push_back(it->second);
            cursor = i = j + 1;
        } else {
            i = j;  // another '<' (a new candidate starts there) or the end
        }
    }
    if (cursor < n) WGML_TRY(gpt2_tokenize_piece(t, text + cursor, n - cursor, ids));
    return copy_ids(ids, out, cap, n_out);
}

int wgml_gpt2_tokenizer_decode(const wgml_tokenizer *t, const uint32_t *tokens, uint64_t n_tokens,
                               int raw_bytes, char *buf, uint64_t cap, uint64_t *n_out) {
    WGML_REQUIRE(t && (tokens || n_tokens == 0) && n_out, "wgml_gpt2_tokenizer_decode: null argument");
    WGML_REQUIRE(t->kind == 1, "wgml_gpt2_tokenizer_decode: not a GPT-2 tokenizer");
    std::string s;
    for (uint64_t k = 0; k < n_tokens; ++k) {
        if (tokens[k] >= t->vocab.size()) continue;  // unknown ids are skipped (filter_map)
        const std::string &piece = t->vocab[tokens[k]];
        for (size_t i = 0; i < piece.size();) {
            const uint32_t cp = utf8_next(piece.data(), piece.size(), i);
            auto it = t->cp_to_byte.find(cp);
            if (it == t->cp_to_byte.end()) continue;  // characters outside the byte alphabet are dropped
            // the reference turns every byte into the character of that value
            // (`b as char`, tokenizer.rs:163): text beyond ASCII comes out as Latin-1
            // read as code points; raw_bytes gives the bytes themselves instead
            if (raw_bytes)
                s.push_back((char)it->second);
            else
                utf8_append(s, it->second);
        }
    }
    return copy_out(s, buf, cap, n_out);
}

}  // extern "C"
