// ref_shim.cpp -- C-callable doorway into the *compiled reference* CPU path.
//
// TEST INFRASTRUCTURE ONLY.  This file holds no arithmetic of its own: it
// includes the reference's headers where they lie (the Makefile passes
// -I/root/reference/src) and is linked with the reference's ops.cpp and
// model.cpp, compiled untouched with the reference's flags (CMakeLists.txt:24:
// -O3 -Wall -Wextra).  The resulting oracle/_ref/liblpp_ref.so is used to
// prove the restated oracle (lpp_oracle.c) bit-identical to the reference, to
// write golden vectors, and as the "reference" CPU baseline of the benchmark.
#include <stdlib.h>
#include <string.h>

#include "model.h"
#include "loader.h"
#include "ops.h"
#include "tokenizer.h"

// model.h still declares the old 4-argument sample(); the definition in
// model.cpp:256 takes seven.  Declare what is actually defined.
int sample(float* logits, int vocab_size, float temperature, float topp,
           float penalty, int* history, int history_len);

namespace {

struct RefModel {
    Config cfg;
    transformerWeights w;
    RunState s;
};

}  // namespace

extern "C" {

void ref_naive_matmul(float* out, float* x, float* w, int n, int d) { naive_matmul(out, x, w, n, d); }
void ref_rmsnorm(float* out, float* x, float* weight, int n) { RMSNorm(out, x, weight, n); }
void ref_rope(float* q, float* k, int pos, int dim, int kv_dim, int head_size, float base) {
    rope(q, k, pos, dim, kv_dim, head_size, base);
}
void ref_softmax(float* x, int size) { softmax(x, size); }
void ref_swiglu(float* hb, float* h1, float* h3, int size) { swiglu(hb, h1, h3, size); }

// sample() draws rand()/RAND_MAX itself; seed it here so a caller can replay the
// same libc stream and hand the oracle the identical r.
void ref_srand(unsigned seed) { srand(seed); }
float ref_next_uniform(void) { return (float)rand() / (float)RAND_MAX; }
int ref_sample(float* logits, int vocab, float temperature, float topp, float penalty,
               int* history, int history_len) {
    return sample(logits, vocab, temperature, topp, penalty, history, history_len);
}

// Model handle: the caller keeps ownership of every weight array (fp32, stacked
// per layer in the reference's layout); RunState comes from the reference's own
// malloc_run_state.
void* ref_model_create(int dim, int hidden_dim, int n_layers, int n_heads, int n_kv_heads,
                       int vocab_size, int seq_len, float rope_base,
                       float* token_embedding_table, float* rms_att_weight, float* wq, float* wk,
                       float* wv, float* wo, float* rms_ffn_weight, float* w1, float* w2,
                       float* w3, float* rms_final_weight, float* w_cls) {
    RefModel* m = (RefModel*)calloc(1, sizeof(RefModel));
    if (!m) return nullptr;
    m->cfg.dim = dim;
    m->cfg.hidden_dim = hidden_dim;
    m->cfg.n_layers = n_layers;
    m->cfg.n_heads = n_heads;
    m->cfg.n_kv_heads = n_kv_heads;
    m->cfg.vocab_size = vocab_size;
    m->cfg.seq_len = seq_len;
    m->cfg.rope_base = rope_base;
    m->cfg.weight_precision = WEIGHT_FP32;
    m->w.token_embedding_table = token_embedding_table;
    m->w.rms_att_weight = rms_att_weight;
    m->w.wq = wq;
    m->w.wk = wk;
    m->w.wv = wv;
    m->w.wo = wo;
    m->w.rms_ffn_weight = rms_ffn_weight;
    m->w.w1 = w1;
    m->w.w2 = w2;
    m->w.w3 = w3;
    m->w.rms_final_weight = rms_final_weight;
    m->w.w_cls = w_cls;
    malloc_run_state(&m->s, &m->cfg);
    return m;
}

void ref_model_destroy(void* h) {
    RefModel* m = (RefModel*)h;
    if (!m) return;
    free_run_state(&m->s);
    free(m);
}

int ref_forward(void* h, int token, int pos, float temperature, float topp, float penalty,
                int* history, int history_len) {
    RefModel* m = (RefModel*)h;
    return forward(token, pos, &m->s, &m->w, &m->cfg, temperature, topp, penalty, history,
                   history_len);
}

void ref_attention(void* h, int layer, int pos) {
    RefModel* m = (RefModel*)h;
    attention(&m->s, &m->w, &m->cfg, layer, pos);
}

void ref_transformer_block(void* h, int layer, int pos) {
    RefModel* m = (RefModel*)h;
    transformer_block(&m->s, &m->w, &m->cfg, layer, pos);
}

// Buffer access for comparisons: 0 x, 1 xb, 2 xb2, 3 hb, 4 he, 5 q, 6 k, 7 v, 8 att,
// 9 logits, 10 key_cache, 11 value_cache.
float* ref_state_buffer(void* h, int which) {
    RefModel* m = (RefModel*)h;
    switch (which) {
        case 0: return m->s.x;
        case 1: return m->s.xb;
        case 2: return m->s.xb2;
        case 3: return m->s.hb;
        case 4: return m->s.he;
        case 5: return m->s.q;
        case 6: return m->s.k;
        case 7: return m->s.v;
        case 8: return m->s.att;
        case 9: return m->s.logits;
        case 10: return m->s.key_cache;
        case 11: return m->s.value_cache;
        default: return nullptr;
    }
}


// load_model_file + checkpoint_init_weights (loader.cpp:134-172, 18-66) on a file on
// disk: the header fields as the reference reads them and where it points each
// tensor, in floats from the first weight.  Returns 0, or -1 when the file cannot
// be opened.
int ref_checkpoint_layout(const char* path, int* header7, float* rope_base, long long* offsets12) {
    Config cfg;
    size_t file_size = 0;
    float* data = load_model_file(path, &cfg, &file_size);
    if (!data) return -1;
    transformerWeights w;
    memset(&w, 0, sizeof(w));
    checkpoint_init_weights(&w, &cfg, data);
    header7[0] = cfg.dim; header7[1] = cfg.hidden_dim; header7[2] = cfg.n_layers; header7[3] = cfg.n_heads;
    header7[4] = cfg.n_kv_heads; header7[5] = cfg.vocab_size; header7[6] = cfg.seq_len;
    *rope_base = cfg.rope_base;
    float* t[12] = {w.token_embedding_table, w.rms_att_weight, w.wq, w.wk, w.wv, w.wo, w.rms_ffn_weight,
                    w.w1, w.w2, w.w3, w.rms_final_weight, w.w_cls};
    for (int i = 0; i < 12; ++i) offsets12[i] = (long long)(t[i] - data);
    free_model_file(data, file_size);
    return 0;
}

// gguf_open + gguf_extract_config + gguf_init_weights (gguf.cpp:125-266, loader.cpp:213-339,
// 423-541, CPU build): the reference's own reading of a GGUF file.  config9 receives the
// nine Config fields (rope_base as its bit pattern); weights12 the host arrays the loader
// allocated (fp32, stacked per layer).  Returns a handle for ref_gguf_free, or null.
void* ref_gguf_load(const char* path, int* config9, float** weights12) {
    GGUFFile* f = gguf_open(path);
    if (!f) return nullptr;
    RefModel* m = (RefModel*)calloc(1, sizeof(RefModel));
    if (!m || !gguf_extract_config(f, &m->cfg) || !gguf_init_weights(f, &m->w, &m->cfg)) {
        gguf_close(f);
        free(m);
        return nullptr;
    }
    gguf_close(f);
    config9[0] = m->cfg.dim; config9[1] = m->cfg.hidden_dim; config9[2] = m->cfg.n_layers;
    config9[3] = m->cfg.n_heads; config9[4] = m->cfg.n_kv_heads; config9[5] = m->cfg.vocab_size;
    config9[6] = m->cfg.seq_len; memcpy(&config9[7], &m->cfg.rope_base, 4);
    config9[8] = (int)m->cfg.weight_precision;
    float* t[12] = {m->w.token_embedding_table, m->w.rms_att_weight, m->w.wq, m->w.wk, m->w.wv, m->w.wo,
                    m->w.rms_ffn_weight, m->w.w1, m->w.w2, m->w.w3, m->w.rms_final_weight, m->w.w_cls};
    for (int i = 0; i < 12; ++i) weights12[i] = t[i];
    return m;
}

void ref_gguf_free(void* h) {
    RefModel* m = (RefModel*)h;
    if (!m) return;
    if (m->w.w_cls != m->w.token_embedding_table) free(m->w.w_cls);
    float* t[11] = {m->w.token_embedding_table, m->w.rms_att_weight, m->w.wq, m->w.wk, m->w.wv, m->w.wo,
                    m->w.rms_ffn_weight, m->w.w1, m->w.w2, m->w.w3, m->w.rms_final_weight};
    for (int i = 0; i < 11; ++i) free(t[i]);
    free(m);
}

// The reference's tokenizer (tokenizer.cpp; gguf_init_tokenizer, loader.cpp:648-699).
// Its string-to-id map is a file-scope static built from the first vocabulary it
// sees: load this library afresh (from a copy of the file) for every vocabulary.
void* ref_tokenizer_load(const char* path, int vocab_size) {
    Tokenizer* t = (Tokenizer*)calloc(1, sizeof(Tokenizer));
    load_tokenizer(t, path, vocab_size);  // exits the process on a malformed file
    return t;
}
void* ref_tokenizer_from_gguf(const char* path) {
    GGUFFile* f = gguf_open(path);
    if (!f) return nullptr;
    Tokenizer* t = (Tokenizer*)calloc(1, sizeof(Tokenizer));
    const bool ok = gguf_init_tokenizer(f, t);
    gguf_close(f);
    if (!ok) {
        free(t);
        return nullptr;
    }
    return t;
}
int ref_tokenizer_kind(void* h) { return (int)((Tokenizer*)h)->type; }
int ref_tokenizer_vocab_size(void* h) { return ((Tokenizer*)h)->vocab_size; }
int ref_tokenizer_max_token_len(void* h) { return ((Tokenizer*)h)->max_token_len; }
float ref_tokenizer_score(void* h, int i) { return ((Tokenizer*)h)->vocab_scores[i]; }
int ref_encode(void* h, const char* text, int* tokens, int max_tokens) {
    int n = 0;
    encode((Tokenizer*)h, text, tokens, &n, max_tokens);
    return n;
}
const char* ref_decode(void* h, int id) { return decode_token((Tokenizer*)h, id); }
}  // extern "C"
