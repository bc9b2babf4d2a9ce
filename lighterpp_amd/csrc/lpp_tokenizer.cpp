// lpp_tokenizer.cpp -- section D of lpp.h, text half: the tokenizer of the
// reference (src/tokenizer.cpp, src/loader.cpp:643-699).  Host code only.
//
// A vocabulary is a list of byte strings with one score each.  Encoding turns the
// text, with a blank put in front, into one id per byte (a blank becomes the
// vocabulary's space marker; a byte without an entry of its own becomes its
// "<0xXX>" entry) and then keeps merging the adjacent pair whose concatenation is
// the vocabulary entry with the highest score, leftmost first among equals, until
// no pair is an entry.  Decoding maps an id back to its string with the space (and,
// for the byte-pair kind, newline) markers replaced.
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "lpp_internal.hpp"

namespace lpp {
// defined in lpp_gguf.cpp
lpp_status gguf_vocabulary(const lpp_gguf* g, int* kind, std::vector<std::string>* tokens, std::vector<float>* scores);
}  // namespace lpp

struct lpp_tokenizer {
    int kind = LPP_TOKENIZER_SENTENCEPIECE;
    std::vector<std::string> vocab;
    std::vector<float> scores;
    int max_token_len = 0;
    std::unordered_map<std::string, int> ids;  // last of equal strings wins, as tokenizer.cpp:131-137 fills its map

    void index() {
        ids.clear();
        ids.reserve(vocab.size() * 2);
        for (size_t i = 0; i < vocab.size(); ++i) ids[vocab[i]] = static_cast<int>(i);
    }
    int lookup(const std::string& s) const {
        auto it = ids.find(s);
        return it == ids.end() ? -1 : it->second;
    }
};

extern "C" {

// load_tokenizer, tokenizer.cpp:15-55: int max_token_len, then per id float score, int length, bytes.
lpp_status lpp_tokenizer_load(lpp_tokenizer** out, const char* path, int vocab_size) {
    using lpp::fail;
    LPP_REQUIRE(out != nullptr && path != nullptr, "lpp_tokenizer_load: null argument");
    LPP_REQUIRE(vocab_size > 0, "lpp_tokenizer_load: vocab_size %d", vocab_size);
    *out = nullptr;
    FILE* f = std::fopen(path, "rb");
    if (f == nullptr) return fail(LPP_ERR_INVALID_ARG, "lpp_tokenizer_load: cannot open %s", path);
    lpp_tokenizer* t = new lpp_tokenizer;
    t->kind = LPP_TOKENIZER_SENTENCEPIECE;  // tokenizer.cpp:23: the file format is always this kind
    auto bad = [&](const char* what, int i) {
        lpp_status st = fail(LPP_ERR_INVALID_ARG, "lpp_tokenizer_load: %s: %s (entry %d)", path, what, i);
        std::fclose(f);
        delete t;
        return st;
    };
    if (std::fread(&t->max_token_len, sizeof(int), 1, f) != 1) return bad("no maximum token length", -1);
    t->vocab.resize(static_cast<size_t>(vocab_size));
    t->scores.resize(static_cast<size_t>(vocab_size));
    for (int i = 0; i < vocab_size; ++i) {
        int len = 0;
        if (std::fread(&t->scores[i], sizeof(float), 1, f) != 1 || std::fread(&len, sizeof(int), 1, f) != 1)
            return bad("file ends inside the vocabulary", i);
        if (len < 0 || len > (1 << 20)) return bad("implausible token length", i);
        t->vocab[i].resize(static_cast<size_t>(len));
        if (len > 0 && std::fread(&t->vocab[i][0], 1, static_cast<size_t>(len), f) != static_cast<size_t>(len))
            return bad("file ends inside a token", i);
    }
    std::fclose(f);
    t->index();
    *out = t;
    return LPP_OK;
}

// gguf_init_tokenizer, loader.cpp:648-699.
lpp_status lpp_tokenizer_from_gguf(lpp_tokenizer** out, const lpp_gguf* g) {
    LPP_REQUIRE(out != nullptr && g != nullptr, "lpp_tokenizer_from_gguf: null argument");
    *out = nullptr;
    lpp_tokenizer* t = new lpp_tokenizer;
    const lpp_status st = lpp::gguf_vocabulary(g, &t->kind, &t->vocab, &t->scores);
    if (st != LPP_OK) {
        delete t;
        return st;
    }
    for (const std::string& s : t->vocab)
        if (static_cast<int>(std::strlen(s.c_str())) > t->max_token_len) t->max_token_len = static_cast<int>(std::strlen(s.c_str()));
    t->index();
    *out = t;
    return LPP_OK;
}

lpp_status lpp_tokenizer_free(lpp_tokenizer* t) {
    delete t;
    return LPP_OK;
}

lpp_status lpp_tokenizer_info(const lpp_tokenizer* t, int* vocab_size, int* kind, int* max_token_len) {
    LPP_REQUIRE(t != nullptr, "lpp_tokenizer_info: null tokenizer");
    if (vocab_size) *vocab_size = static_cast<int>(t->vocab.size());
    if (kind) *kind = t->kind;
    if (max_token_len) *max_token_len = t->max_token_len;
    return LPP_OK;
}

// encode, tokenizer.cpp:148-235.
lpp_status lpp_tokenizer_encode(const lpp_tokenizer* t, const char* text, int* tokens, int max_tokens, int* n_tokens) {
    LPP_REQUIRE(t != nullptr && text != nullptr && n_tokens != nullptr, "lpp_tokenizer_encode: null argument");
    LPP_REQUIRE(max_tokens >= 0 && (max_tokens == 0 || tokens != nullptr), "lpp_tokenizer_encode: capacity %d", max_tokens);
    const bool bpe = t->kind == LPP_TOKENIZER_BPE;
    std::vector<int> cur;
    if (bpe) {  // :160-166
        const int bos = t->lookup("<|begin_of_text|>");
        if (bos != -1) cur.push_back(bos);
    } else if (t->vocab.size() > 1 && t->vocab[1] == "<s>") {  // :168-171
        cur.push_back(1);
    }
    const std::string marker = bpe ? "\xC4\xA0" : "\xE2\x96\x81";  // :179
    std::string processed = " ";  // :174-175
    processed += text;
    for (unsigned char ch : processed) {  // :181-203, byte by byte
        int id = t->lookup(ch == ' ' ? marker : std::string(1, static_cast<char>(ch)));
        if (id == -1) {
            char byte_token[8];
            std::snprintf(byte_token, sizeof byte_token, "<0x%02X>", ch);
            id = t->lookup(byte_token);
        }
        if (id != -1) cur.push_back(id);  // (the reference warns on stderr and drops the byte)
    }
    while (cur.size() >= 2) {  // :205-227 (the reference's loop bound underflows on an empty list)
        float best_score = -1e10f;
        int best_idx = -1, best_token = -1;
        for (size_t i = 0; i + 1 < cur.size(); ++i) {
            const int id = t->lookup(t->vocab[static_cast<size_t>(cur[i])] + t->vocab[static_cast<size_t>(cur[i + 1])]);
            if (id != -1 && t->scores[static_cast<size_t>(id)] > best_score) {
                best_score = t->scores[static_cast<size_t>(id)];
                best_idx = static_cast<int>(i);
                best_token = id;
            }
        }
        if (best_idx == -1) break;
        cur[static_cast<size_t>(best_idx)] = best_token;
        cur.erase(cur.begin() + best_idx + 1);
    }
    int n = 0;  // :229-234: what does not fit is dropped
    for (int id : cur)
        if (n < max_tokens) tokens[n++] = id;
    *n_tokens = n;
    return LPP_OK;
}

// decode_token, tokenizer.cpp:61-123.  At most 255 bytes, as the reference's buffer holds.
lpp_status lpp_tokenizer_decode(const lpp_tokenizer* t, int token_id, char* out, size_t capacity) {
    LPP_REQUIRE(t != nullptr && out != nullptr && capacity > 0, "lpp_tokenizer_decode: null argument");
    LPP_REQUIRE(token_id >= 0 && token_id < static_cast<int>(t->vocab.size()), "lpp_tokenizer_decode: id %d outside [0, %zu)",
                token_id, t->vocab.size());
    const char* raw = t->vocab[static_cast<size_t>(token_id)].c_str();  // up to the first NUL, as strlen sees it
    const size_t len = std::strlen(raw);
    std::string dst;
    if (len > 0 && raw[0] == '<' && raw[len - 1] == '>') {  // :70-84
        unsigned byte_val = 0;
        if (len == 6 && raw[1] == '0' && raw[2] == 'x' && std::sscanf(raw, "<0x%02X>", &byte_val) == 1)
            dst.assign(1, static_cast<char>(byte_val));
        // any other "<...>" entry prints as nothing
    } else {
        const bool bpe = t->kind == LPP_TOKENIZER_BPE;
        const unsigned char* s = reinterpret_cast<const unsigned char*>(raw);
        while (*s && dst.size() < 255) {  // :92-119
            if (bpe && s[0] == 0xC4 && s[1] == 0xA0) {
                dst.push_back(' ');
                s += 2;
            } else if (bpe && s[0] == 0xC4 && s[1] == 0x8A) {
                dst.push_back('\n');
                s += 2;
            } else if (!bpe && s[0] == 0xE2 && s[1] == 0x96 && s[2] == 0x81) {
                dst.push_back(' ');
                s += 3;
            } else {
                dst.push_back(static_cast<char>(*s++));
            }
        }
    }
    // a decoded byte token may be NUL: report the length the caller can rely on through the terminator only
    if (dst.size() + 1 > capacity) return lpp::fail(LPP_ERR_INVALID_ARG, "lpp_tokenizer_decode: %zu bytes do not fit %zu", dst.size() + 1, capacity);
    std::memcpy(out, dst.data(), dst.size());
    out[dst.size()] = '\0';
    return LPP_OK;
}

}  // extern "C"
