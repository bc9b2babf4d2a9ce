// lpp_gguf.cpp -- section D of lpp.h, GGUF half: the F32 / F16 reader of the
// reference (src/gguf.cpp, src/loader.cpp:196-641) as host code over a mapping of
// the file, and the upload of its tensors into an lpp_model in the stacked
// per-layer layout the decode path reads (binary16 matrices go up as they are).
//
// Format (versions 2 and 3, little endian): magic "GGUF", u32 version, u64 tensor
// count, u64 key/value count; the key/value pairs (string key, u32 type, value);
// the tensor descriptions (string name, u32 n_dims, u64 dims[n_dims], u32 type,
// u64 offset); padding to a multiple of 32; tensor data at the given offsets.  A
// string is a u64 length and that many bytes.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cerrno>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "lpp_internal.hpp"
#include "lpp_model.hpp"

namespace {

// value types of a key/value pair (gguf.h:20-34)
enum : uint32_t {
    kU8 = 0, kI8 = 1, kU16 = 2, kI16 = 3, kU32 = 4, kI32 = 5, kF32 = 6, kBool = 7, kString = 8, kArray = 9,
    kU64 = 10, kI64 = 11, kF64 = 12
};
constexpr uint32_t kMagic = 0x46554747u;  // gguf.h:8
constexpr size_t kAlignment = 32;         // gguf.cpp:259 (the reference does not read general.alignment)
constexpr int kSeqLenCap = 16384;         // loader.cpp:333-336

struct Cursor {
    const uint8_t* data;
    size_t pos, size;
    bool take(void* out, size_t n) {
        if (n > size - pos) return false;
        std::memcpy(out, data + pos, n);
        pos += n;
        return true;
    }
    bool skip(size_t n) {
        if (n > size - pos) return false;
        pos += n;
        return true;
    }
    bool string(std::string* out) {
        uint64_t len = 0;
        if (!take(&len, 8) || len > size - pos) return false;
        out->assign(reinterpret_cast<const char*>(data + pos), static_cast<size_t>(len));
        pos += static_cast<size_t>(len);
        return true;
    }
    // gguf.cpp:49-88
    bool skip_value(uint32_t type, int depth = 0) {
        switch (type) {
            case kU8: case kI8: case kBool: return skip(1);
            case kU16: case kI16: return skip(2);
            case kU32: case kI32: case kF32: return skip(4);
            case kU64: case kI64: case kF64: return skip(8);
            case kString: {
                uint64_t len = 0;
                return take(&len, 8) && len <= size - pos && skip(static_cast<size_t>(len));
            }
            case kArray: {
                uint32_t elem = 0;
                uint64_t count = 0;
                if (depth > 8 || !take(&elem, 4) || !take(&count, 8)) return false;
                for (uint64_t i = 0; i < count; ++i)
                    if (!skip_value(elem, depth + 1)) return false;
                return true;
            }
            default: return false;
        }
    }
};

struct Meta {
    std::string key;
    uint32_t type;
    size_t value_offset;
};

struct TensorInfo {
    std::string name;
    uint32_t n_dims;
    uint64_t dims[4];
    uint32_t type;
    uint64_t offset;
    size_t nelements;
};

size_t type_size(uint32_t ggml_type) { return ggml_type == LPP_GGML_F32 ? 4 : ggml_type == LPP_GGML_F16 ? 2 : 0; }

}  // namespace

struct lpp_gguf {
    void* map = nullptr;
    size_t size = 0;
    uint32_t version = 0;
    std::vector<Meta> meta;
    std::vector<TensorInfo> tensors;
    size_t data_start = 0;

    const Meta* find(const char* key, uint32_t type) const {  // gguf.cpp:91-98 + the getters' type check
        for (const Meta& m : meta)
            if (m.key == key) return m.type == type ? &m : nullptr;
        return nullptr;
    }
    const uint8_t* at(size_t off) const { return static_cast<const uint8_t*>(map) + off; }
    bool get_u32(const std::string& key, uint32_t* out) const {
        const Meta* m = find(key.c_str(), kU32);
        if (!m) return false;
        std::memcpy(out, at(m->value_offset), 4);
        return true;
    }
    bool get_f32(const std::string& key, float* out) const {
        const Meta* m = find(key.c_str(), kF32);
        if (!m) return false;
        std::memcpy(out, at(m->value_offset), 4);
        return true;
    }
    bool get_string(const std::string& key, std::string* out) const {
        const Meta* m = find(key.c_str(), kString);
        if (!m) return false;
        uint64_t len = 0;
        std::memcpy(&len, at(m->value_offset), 8);
        out->assign(reinterpret_cast<const char*>(at(m->value_offset + 8)), static_cast<size_t>(len));
        return true;
    }
    // number of elements of an array of strings, 0 when absent or of another kind (gguf.cpp:357-385)
    size_t string_array_count(const char* key) const {
        const Meta* m = find(key, kArray);
        if (!m) return 0;
        uint32_t elem = 0;
        uint64_t count = 0;
        std::memcpy(&elem, at(m->value_offset), 4);
        std::memcpy(&count, at(m->value_offset + 4), 8);
        return elem == kString ? static_cast<size_t>(count) : 0;
    }
    const TensorInfo* tensor(const std::string& name) const {
        for (const TensorInfo& t : tensors)
            if (t.name == name) return &t;
        return nullptr;
    }
    const void* data(const TensorInfo& t) const { return at(data_start + static_cast<size_t>(t.offset)); }
};

// The embedded vocabulary as gguf_init_tokenizer reads it (loader.cpp:648-699): kind from
// "tokenizer.ggml.model" ("gpt2" = byte-pair, anything else or absent = SentencePiece), strings
// from "tokenizer.ggml.tokens", scores from "tokenizer.ggml.scores" when there is one per token,
// zeros otherwise.  Used by lpp_tokenizer_from_gguf.
namespace lpp {
lpp_status gguf_vocabulary(const lpp_gguf* g, int* kind, std::vector<std::string>* tokens, std::vector<float>* scores) {
    std::string model;
    *kind = (g->get_string("tokenizer.ggml.model", &model) && model == "gpt2") ? LPP_TOKENIZER_BPE : LPP_TOKENIZER_SENTENCEPIECE;
    const size_t n = g->string_array_count("tokenizer.ggml.tokens");
    if (n == 0) return lpp::fail(LPP_ERR_INVALID_ARG, "lpp_tokenizer_from_gguf: no tokenizer.ggml.tokens");
    const Meta* m = g->find("tokenizer.ggml.tokens", kArray);
    size_t pos = m->value_offset + 12;
    tokens->resize(n);
    for (size_t i = 0; i < n; ++i) {  // bounds were checked when the file was opened
        uint64_t len = 0;
        std::memcpy(&len, g->at(pos), 8);
        (*tokens)[i].assign(reinterpret_cast<const char*>(g->at(pos + 8)), static_cast<size_t>(len));
        pos += 8 + static_cast<size_t>(len);
    }
    scores->assign(n, 0.0f);
    const Meta* sm = g->find("tokenizer.ggml.scores", kArray);
    if (sm != nullptr) {
        uint32_t elem = 0;
        uint64_t count = 0;
        std::memcpy(&elem, g->at(sm->value_offset), 4);
        std::memcpy(&count, g->at(sm->value_offset + 4), 8);
        if (elem == kF32 && count == n) std::memcpy(scores->data(), g->at(sm->value_offset + 12), n * sizeof(float));
    }
    return LPP_OK;
}
}  // namespace lpp

extern "C" {

lpp_status lpp_gguf_open(lpp_gguf** out, const char* path) {
    using lpp::fail;
    LPP_REQUIRE(out != nullptr && path != nullptr, "lpp_gguf_open: null argument");
    *out = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd == -1) return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_open: cannot open %s: %s", path, strerror(errno));
    struct stat sb;
    if (fstat(fd, &sb) == -1 || sb.st_size < 24) {
        close(fd);
        return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_open: %s is shorter than a GGUF header", path);
    }
    const size_t size = static_cast<size_t>(sb.st_size);
    void* map = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_open: mmap of %s failed", path);

    lpp_gguf* g = new lpp_gguf;
    g->map = map;
    g->size = size;
    auto bad = [&](const char* what) {
        lpp_status st = fail(LPP_ERR_INVALID_ARG, "lpp_gguf_open: %s: %s", path, what);
        munmap(map, size);
        delete g;
        return st;
    };
    Cursor c{static_cast<const uint8_t*>(map), 0, size};
    uint32_t magic = 0;
    uint64_t n_tensors = 0, n_meta = 0;
    if (!c.take(&magic, 4) || !c.take(&g->version, 4) || !c.take(&n_tensors, 8) || !c.take(&n_meta, 8))
        return bad("truncated header");
    if (magic != kMagic) return bad("not a GGUF file");
    if (g->version < 2 || g->version > 3) return bad("unsupported version (2 and 3 are read)");  // gguf.cpp:174-178
    if (n_meta > size || n_tensors > size) return bad("implausible counts");
    g->meta.resize(static_cast<size_t>(n_meta));
    for (Meta& m : g->meta) {  // gguf.cpp:189-214
        if (!c.string(&m.key) || !c.take(&m.type, 4)) return bad("truncated key/value list");
        m.value_offset = c.pos;
        if (!c.skip_value(m.type)) return bad("key/value pair of unknown type or past the end of the file");
    }
    g->tensors.resize(static_cast<size_t>(n_tensors));
    for (TensorInfo& t : g->tensors) {  // gguf.cpp:218-255
        if (!c.string(&t.name) || !c.take(&t.n_dims, 4)) return bad("truncated tensor list");
        if (t.n_dims < 1 || t.n_dims > 4) return bad("tensor with other than 1..4 dimensions");
        t.nelements = 1;
        for (uint32_t d = 0; d < t.n_dims; ++d) {
            if (!c.take(&t.dims[d], 8)) return bad("truncated tensor list");
            if (t.dims[d] == 0 || t.dims[d] > (1ull << 40) || t.nelements > (1ull << 62) / t.dims[d])
                return bad("implausible tensor dimension");
            t.nelements *= static_cast<size_t>(t.dims[d]);
        }
        if (!c.take(&t.type, 4) || !c.take(&t.offset, 8)) return bad("truncated tensor list");
    }
    g->data_start = (c.pos + kAlignment - 1) & ~(kAlignment - 1);  // gguf.cpp:259-261
    for (const TensorInfo& t : g->tensors) {
        const size_t bytes = t.nelements * type_size(t.type);  // 0 for the types this reader does not load
        if (g->data_start > size || t.offset > size - g->data_start || bytes > size - g->data_start - t.offset)
            return bad("tensor data past the end of the file");
    }
    *out = g;
    return LPP_OK;
}

lpp_status lpp_gguf_close(lpp_gguf* g) {
    if (g == nullptr) return LPP_OK;
    if (g->map != nullptr) munmap(g->map, g->size);
    delete g;
    return LPP_OK;
}

// gguf_extract_config (loader.cpp:213-339) + the precision test of gguf_init_weights (:426-433).
lpp_status lpp_gguf_config(const lpp_gguf* g, lpp_config* cfg) {
    using lpp::fail;
    LPP_REQUIRE(g != nullptr && cfg != nullptr, "lpp_gguf_config: null argument");
    std::string arch;
    if (!g->get_string("general.architecture", &arch))
        return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_config: missing general.architecture");
    const std::string prefix = arch + ".";
    auto need = [&](const char* name, int* out) -> lpp_status {
        uint32_t v = 0;
        if (!g->get_u32(prefix + name, &v))
            return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_config: missing %s%s (uint32)", prefix.c_str(), name);
        if (v == 0 || v > 0x7fffffffu) return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_config: %s%s = %u", prefix.c_str(), name, v);
        *out = static_cast<int>(v);
        return LPP_OK;
    };
    lpp_config c{};
    LPP_TRY(need("embedding_length", &c.dim));
    LPP_TRY(need("feed_forward_length", &c.hidden_dim));
    LPP_TRY(need("block_count", &c.n_layers));
    LPP_TRY(need("attention.head_count", &c.n_heads));
    uint32_t kv = 0;
    c.n_kv_heads = g->get_u32(prefix + "attention.head_count_kv", &kv) && kv > 0 ? static_cast<int>(kv) : c.n_heads;  // :273-277
    LPP_TRY(need("context_length", &c.seq_len));
    if (!g->get_f32(prefix + "rope.freq_base", &c.rope_base)) c.rope_base = 10000.0f;  // :289-292
    const size_t vocab = g->string_array_count("tokenizer.ggml.tokens");  // :297-303: the vocabulary is counted
    if (vocab == 0 || vocab > 0x7fffffffu) return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_config: missing tokenizer.ggml.tokens");
    c.vocab_size = static_cast<int>(vocab);
    if (c.seq_len > kSeqLenCap) c.seq_len = kSeqLenCap;  // :333-336
    const TensorInfo* q0 = g->tensor("blk.0.attn_q.weight");
    c.weight_precision = (q0 != nullptr && q0->type == LPP_GGML_F16) ? LPP_WEIGHT_FP16 : LPP_WEIGHT_FP32;
    if (c.dim % c.n_heads != 0 || c.n_heads % c.n_kv_heads != 0)
        return fail(LPP_ERR_INVALID_ARG, "lpp_gguf_config: dim %d, %d heads, %d kv heads do not divide", c.dim, c.n_heads,
                    c.n_kv_heads);
    *cfg = c;
    return LPP_OK;
}

lpp_status lpp_gguf_tensor(const lpp_gguf* g, const char* name, const void** data, int* ggml_type, size_t* nelements) {
    LPP_REQUIRE(g != nullptr && name != nullptr && data != nullptr && ggml_type != nullptr && nelements != nullptr,
                "lpp_gguf_tensor: null argument");
    const TensorInfo* t = g->tensor(name);
    if (t == nullptr) return lpp::fail(LPP_ERR_INVALID_ARG, "lpp_gguf_tensor: no tensor named %s", name);
    *data = g->data(*t);
    *ggml_type = static_cast<int>(t->type);
    *nelements = t->nelements;
    return LPP_OK;
}

// gguf_init_weights (loader.cpp:423-641): the named tensors into the stacked arrays.
lpp_status lpp_model_load_gguf(lpp_model** out, const lpp_gguf* g) {
    using lpp::fail;
    LPP_REQUIRE(out != nullptr && g != nullptr, "lpp_model_load_gguf: null argument");
    *out = nullptr;
    lpp_config cfg{};
    LPP_TRY(lpp_gguf_config(g, &cfg));
    lpp_model* m = nullptr;
    LPP_TRY(lpp_model_create(&m, &cfg));
    const bool f16_model = cfg.weight_precision == LPP_WEIGHT_FP16;
    const size_t dim = static_cast<size_t>(cfg.dim), hidden = static_cast<size_t>(cfg.hidden_dim);
    const size_t kv_dim = static_cast<size_t>(cfg.n_kv_heads) * (dim / static_cast<size_t>(cfg.n_heads));
    std::vector<float> widened;

    // One tensor of the file into [slot] of a stacked model tensor whose slices hold `count` elements.
    auto put = [&](const std::string& name, int tensor, size_t slot, size_t count, bool matrix) -> lpp_status {
        const TensorInfo* t = g->tensor(name);
        if (t == nullptr) return fail(LPP_ERR_INVALID_ARG, "lpp_model_load_gguf: missing %s", name.c_str());
        if (t->nelements != count)
            return fail(LPP_ERR_INVALID_ARG, "lpp_model_load_gguf: %s holds %zu elements, the shape needs %zu", name.c_str(),
                        t->nelements, count);
        if (t->type != LPP_GGML_F32 && t->type != LPP_GGML_F16)  // the reference zero-fills these (loader.cpp:395-400)
            return fail(LPP_ERR_UNSUPPORTED, "lpp_model_load_gguf: %s has ggml type %u; F32 and F16 are read", name.c_str(),
                        t->type);
        const bool as_f16 = matrix && f16_model;
        if (as_f16) {
            // binary16 matrices go to the device as they are (loader.cpp:405-419, 543-617)
            if (t->type != LPP_GGML_F16)
                return fail(LPP_ERR_UNSUPPORTED, "lpp_model_load_gguf: %s is F32 in a file whose blk.0.attn_q.weight is F16",
                            name.c_str());
            return lpp_model_upload(m, tensor, slot * count * 2, g->data(*t), count * 2);
        }
        if (t->type == LPP_GGML_F32) return lpp_model_upload(m, tensor, slot * count * 4, g->data(*t), count * 4);
        widened.resize(count);  // exact widening, loader.cpp:346-379, 391-394
        LPP_TRY(lpp_f16_to_f32_host(widened.data(), static_cast<const lpp_half*>(g->data(*t)), count));
        return lpp_model_upload(m, tensor, slot * count * 4, widened.data(), count * 4);
    };
    auto load_all = [&]() -> lpp_status {
        LPP_TRY(put("token_embd.weight", LPP_T_TOKEN_EMBEDDING, 0, static_cast<size_t>(cfg.vocab_size) * dim, false));
        LPP_TRY(put("output_norm.weight", LPP_T_RMS_FINAL, 0, dim, false));
        for (int l = 0; l < cfg.n_layers; ++l) {
            const std::string b = "blk." + std::to_string(l) + ".";
            const size_t s = static_cast<size_t>(l);
            LPP_TRY(put(b + "attn_norm.weight", LPP_T_RMS_ATT, s, dim, false));
            LPP_TRY(put(b + "attn_q.weight", LPP_T_WQ, s, dim * dim, true));
            LPP_TRY(put(b + "attn_k.weight", LPP_T_WK, s, kv_dim * dim, true));
            LPP_TRY(put(b + "attn_v.weight", LPP_T_WV, s, kv_dim * dim, true));
            LPP_TRY(put(b + "attn_output.weight", LPP_T_WO, s, dim * dim, true));
            LPP_TRY(put(b + "ffn_norm.weight", LPP_T_RMS_FFN, s, dim, false));
            LPP_TRY(put(b + "ffn_gate.weight", LPP_T_W1, s, hidden * dim, true));
            LPP_TRY(put(b + "ffn_down.weight", LPP_T_W2, s, dim * hidden, true));
            LPP_TRY(put(b + "ffn_up.weight", LPP_T_W3, s, hidden * dim, true));
        }
        // loader.cpp:459-468, 619-632: a separate classifier when the file has one, else the embedding
        if (g->tensor("output.weight") != nullptr)
            return put("output.weight", LPP_T_WCLS, 0, static_cast<size_t>(cfg.vocab_size) * dim, true);
        return lpp_model_tie_classifier(m);
    };
    const lpp_status st = load_all();
    if (st != LPP_OK) {
        lpp_model_destroy(m);
        return st;
    }
    *out = m;
    return LPP_OK;
}

}  // extern "C"
