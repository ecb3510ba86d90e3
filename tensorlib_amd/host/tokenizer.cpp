// llama2.c-format BPE tokenizer: host-side text <-> token ids for the Llama2 driver.
//
// Behaviour follows the reference's Tokenizer (model/llama2_7b/src/Tokenizer.cpp:7-169, a C++ rendering of
// llama2.c's): a dummy-prefix space, one token per UTF-8 character with byte fallback (byte + 3), then
// repeatedly merge the adjacent pair whose concatenation is the vocabulary entry with the highest score
// (first such pair wins ties).  Deliberate differences, all in error handling: an empty token list is not
// walked (the reference's `tokens.size() - 1` underflows), a vocabulary without " " skips the dummy prefix
// instead of pushing -1, decode leaves the stored vocabulary untouched, and of several entries with the same
// string the lowest id is the one looked up (the reference's unstable sort leaves that unspecified).
#include "tensorlib_tokenizer.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <string>
#include <unordered_map>
#include <vector>

struct tlt_tokenizer {
    std::vector<std::string> vocab;
    std::vector<float> scores;
    std::unordered_map<std::string, int> index;  // piece -> lowest id
    unsigned max_token_length = 0;
};

namespace {

thread_local std::string g_error;

int fail(const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return -1;
}

int lookup(const tlt_tokenizer& t, const std::string& s) {
    auto it = t.index.find(s);
    return it == t.index.end() ? -1 : it->second;
}

int hex_digit(char c) {
    if (c >= '0' && c <= '9') return c - '0';
    if (c >= 'A' && c <= 'F') return c - 'A' + 10;
    if (c >= 'a' && c <= 'f') return c - 'a' + 10;
    return -1;
}

}  // namespace

extern "C" {

const char* tlt_last_error(void) { return g_error.c_str(); }

int tlt_load(const char* path, int vocab_size, tlt_tokenizer** out) {
    if (!path || !out) return fail("tlt_load: null argument");
    if (vocab_size <= 0) return fail("tlt_load: vocab_size %d", vocab_size);
    std::ifstream f(path, std::ios::binary);
    if (!f) return fail("tlt_load: cannot open %s", path);
    auto t = new tlt_tokenizer;
    t->vocab.resize(vocab_size);
    t->scores.resize(vocab_size);
    int max_len = 0;
    f.read(reinterpret_cast<char*>(&max_len), sizeof(int));
    if (!f || max_len < 0) {
        delete t;
        return fail("tlt_load: %s: cannot read max_token_length", path);
    }
    t->max_token_length = (unsigned)max_len;
    for (int i = 0; i < vocab_size; ++i) {
        int len = 0;
        f.read(reinterpret_cast<char*>(&t->scores[i]), sizeof(float));
        f.read(reinterpret_cast<char*>(&len), sizeof(int));
        if (!f || len < 0 || len > (1 << 20)) {
            delete t;
            return fail("tlt_load: %s: truncated or corrupt at token %d of %d", path, i, vocab_size);
        }
        t->vocab[i].resize((size_t)len);
        f.read(&t->vocab[i][0], len);
        if (!f) {
            delete t;
            return fail("tlt_load: %s: truncated inside token %d of %d", path, i, vocab_size);
        }
        t->index.emplace(t->vocab[i], i);  // keeps the first (lowest) id of a repeated piece
    }
    *out = t;
    return 0;
}

int tlt_destroy(tlt_tokenizer* t) {
    delete t;
    return 0;
}

int tlt_vocab_size(const tlt_tokenizer* t) { return t ? (int)t->vocab.size() : fail("tlt_vocab_size: null tokenizer"); }

int tlt_encode(const tlt_tokenizer* t, const char* text, size_t text_len, int bos, int eos, int* out_tokens,
               size_t capacity, size_t* n_tokens) {
    if (!t || (!text && text_len) || !n_tokens || (!out_tokens && capacity)) return fail("tlt_encode: null argument");
    std::vector<int> tokens;
    tokens.reserve(text_len + 3);
    if (bos) tokens.push_back(1);
    if (text_len) {
        const int dummy_prefix = lookup(*t, " ");
        if (dummy_prefix >= 0) tokens.push_back(dummy_prefix);
    }
    // one token per UTF-8 character (a lead byte and up to three continuation bytes 10xxxxxx); a character the
    // vocabulary lacks becomes its bytes, as byte tokens
    std::string ch;
    for (size_t i = 0; i < text_len; ++i) {
        const unsigned char c = (unsigned char)text[i];
        if ((c & 0xC0) != 0x80) ch.clear();
        ch.push_back((char)c);
        const unsigned char next = i + 1 < text_len ? (unsigned char)text[i + 1] : 0;
        if ((next & 0xC0) == 0x80 && ch.size() < 4) continue;
        const int id = lookup(*t, ch);
        if (id >= 0) {
            tokens.push_back(id);
        } else {
            for (unsigned char b : ch) tokens.push_back((int)b + 3);
        }
        ch.clear();
    }
    for (int id : tokens)
        if (id < 0 || id >= (int)t->vocab.size()) return fail("tlt_encode: vocabulary of %zu entries has no byte tokens", t->vocab.size());
    // merge the best adjacent pair until none is in the vocabulary
    std::string pair;
    for (;;) {
        float best_score = -1e10f;
        int best_id = -1;
        size_t best_idx = 0;
        for (size_t i = 0; i + 1 < tokens.size(); ++i) {
            pair.assign(t->vocab[tokens[i]]);
            pair.append(t->vocab[tokens[i + 1]]);
            const int id = lookup(*t, pair);
            if (id >= 0 && t->scores[id] > best_score) {
                best_score = t->scores[id];
                best_id = id;
                best_idx = i;
            }
        }
        if (best_id < 0) break;
        tokens[best_idx] = best_id;
        tokens.erase(tokens.begin() + (long)best_idx + 1);
    }
    if (eos) tokens.push_back(2);
    *n_tokens = tokens.size();
    if (tokens.size() > capacity) return fail("tlt_encode: %zu tokens do not fit a buffer of %zu", tokens.size(), capacity);
    if (!tokens.empty()) memcpy(out_tokens, tokens.data(), tokens.size() * sizeof(int));
    return 0;
}

int tlt_decode(const tlt_tokenizer* t, int prev_token, int token, char* out, size_t capacity, size_t* n_bytes) {
    if (!t || !n_bytes || (!out && capacity)) return fail("tlt_decode: null argument");
    if (token < 0 || token >= (int)t->vocab.size()) return fail("tlt_decode: token %d outside [0, %zu)", token, t->vocab.size());
    const std::string& stored = t->vocab[token];
    const char* p = stored.data();
    size_t n = stored.size();
    if (prev_token == 1 && n > 0 && p[0] == ' ') {
        ++p;
        --n;
    }
    char byte;
    if (n == 6 && p[0] == '<' && p[1] == '0' && p[2] == 'x' && hex_digit(p[3]) >= 0 && hex_digit(p[4]) >= 0 && p[5] == '>') {
        byte = (char)(hex_digit(p[3]) * 16 + hex_digit(p[4]));
        p = &byte;
        n = 1;
    }
    *n_bytes = n;
    if (n > capacity) return fail("tlt_decode: piece of %zu bytes does not fit a buffer of %zu", n, capacity);
    if (n) memcpy(out, p, n);
    return 0;
}

}  // extern "C"
