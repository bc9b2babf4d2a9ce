// Test harness around the reference's own forward() (src/model.cpp:342-371, USE_CUDA branch) built against
// liblpp_hip.so: creates its Config / RunState / transformerWeights, puts the weights on the device the way the
// reference's loader does (loader.cpp:543-617: one allocation per tensor, stacked [L][rows][cols]), and calls
// forward().  No arithmetic here; test infrastructure only.
#include <string.h>

#include "model.h"

namespace {
struct Harness {
    Config cfg;
    RunState state;
    transformerWeights w;
    float* host_embedding;
};
}  // namespace

extern "C" {

void* rol_create(int dim, int hidden_dim, int n_layers, int n_heads, int n_kv_heads, int vocab_size, int seq_len,
                 float rope_base, int weight_precision) {
    Harness* h = new Harness;
    memset(&h->w, 0, sizeof h->w);
    memset(&h->state, 0, sizeof h->state);
    h->cfg = Config{dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len, rope_base,
                    static_cast<WeightPrecision>(weight_precision)};
    malloc_run_state(&h->state, &h->cfg);
    h->host_embedding = nullptr;
    return h;
}

// which: 0 embedding (fp32, kept on the host too: forward() copies one row per token), 1 rms_att, 2 wq, 3 wk,
// 4 wv, 5 wo, 6 rms_ffn, 7 w1, 8 w2, 9 w3, 10 rms_final, 11 w_cls
int rol_upload(void* handle, int which, const void* host, size_t bytes) {
    Harness* h = static_cast<Harness*>(handle);
    void* d = nullptr;
    if (lpp_malloc(&d, bytes) != LPP_OK) return 1;
    if (lpp_memcpy_h2d(d, host, bytes) != LPP_OK) return 2;
    transformerWeights& w = h->w;
    switch (which) {
        case 0:
            w.d_token_embedding_table = static_cast<float*>(d);
            h->host_embedding = new float[bytes / sizeof(float)];
            memcpy(h->host_embedding, host, bytes);
            w.token_embedding_table = h->host_embedding;
            break;
        case 1: w.d_rms_att_weight = static_cast<float*>(d); break;
        case 2: w.d_wq = d; break;
        case 3: w.d_wk = d; break;
        case 4: w.d_wv = d; break;
        case 5: w.d_wo = d; break;
        case 6: w.d_rms_ffn_weight = static_cast<float*>(d); break;
        case 7: w.d_w1 = d; break;
        case 8: w.d_w2 = d; break;
        case 9: w.d_w3 = d; break;
        case 10: w.d_rms_final_weight = static_cast<float*>(d); break;
        case 11: w.d_w_cls = d; break;
        default: return 3;
    }
    return 0;
}

// The reference's forward(), greedy (temperature 0, no penalty); the logits it left on the device come back too.
int rol_forward(void* handle, int token, int pos, float* logits_out) {
    Harness* h = static_cast<Harness*>(handle);
    const int next = forward(token, pos, &h->state, &h->w, &h->cfg, 0.0f, 0.9f, 1.0f, nullptr, 0);
    if (logits_out != nullptr) lpp_memcpy_d2h(logits_out, h->state.d_logits, h->cfg.vocab_size * sizeof(float));
    return next;
}

void rol_destroy(void* handle) {
    Harness* h = static_cast<Harness*>(handle);
    free_run_state(&h->state);
    void* all[] = {h->w.d_token_embedding_table, h->w.d_rms_att_weight, h->w.d_wq, h->w.d_wk, h->w.d_wv, h->w.d_wo,
                   h->w.d_rms_ffn_weight,        h->w.d_w1,             h->w.d_w2, h->w.d_w3, h->w.d_rms_final_weight,
                   h->w.d_w_cls};
    for (void* p : all) lpp_free(p);
    delete[] h->host_embedding;
    delete h;
}

}  // extern "C"
