// lpp_model.cpp -- section B of lpp.h: the host side of the decode loop.
//
// Mirrors malloc_run_state / free_run_state / attention / transformer_block /
// forward (reference src/model.cpp:18-241, 342-371) and the generation loop of
// src/main.cpp:158-223.  LPP_PATH_OPS issues the twelve operators in exactly
// the reference's order through the C ABI; the fused paths hand a whole token
// to fused_decode.hip.
#include "lpp_model.hpp"

#include <chrono>
#include <cmath>
#include <cstring>
#include <new>
#include <vector>

using lpp::fail;

namespace lpp {

size_t tensor_bytes(const lpp_config& c, int tensor) {
    const size_t dim = c.dim, hidden = c.hidden_dim, L = c.n_layers, vocab = c.vocab_size;
    const size_t kv_dim = static_cast<size_t>(c.dim) * c.n_kv_heads / c.n_heads;
    const size_t wb = (c.weight_precision == LPP_WEIGHT_FP16) ? 2 : 4;
    switch (tensor) {
        case LPP_T_TOKEN_EMBEDDING: return vocab * dim * 4;
        case LPP_T_RMS_ATT: return L * dim * 4;
        case LPP_T_WQ: return L * dim * dim * wb;
        case LPP_T_WK: return L * kv_dim * dim * wb;
        case LPP_T_WV: return L * kv_dim * dim * wb;
        case LPP_T_WO: return L * dim * dim * wb;
        case LPP_T_RMS_FFN: return L * dim * 4;
        case LPP_T_W1: return L * hidden * dim * wb;
        case LPP_T_W2: return L * dim * hidden * wb;
        case LPP_T_W3: return L * hidden * dim * wb;
        case LPP_T_RMS_FINAL: return dim * 4;
        case LPP_T_WCLS: return vocab * dim * wb;
        default: return 0;
    }
}

namespace {

template <typename T>
lpp_status dev_alloc(T** p, size_t count, bool zero) {
    void* raw = nullptr;
    LPP_TRY(lpp_malloc(&raw, count * sizeof(T)));
    *p = static_cast<T*>(raw);
    if (zero && count) LPP_TRY(lpp_memset(raw, 0, count * sizeof(T)));
    return LPP_OK;
}

// WEIGHT_PTR of model.cpp:12-13: element offset scaled by the weight width.
inline const void* weight_at(const lpp_model* m, int tensor, size_t elem_offset) {
    const size_t wb = (m->cfg.weight_precision == LPP_WEIGHT_FP16) ? 2 : 4;
    return static_cast<const char*>(m->w[tensor]) + elem_offset * wb;
}

lpp_status check_ready(const lpp_model* m) {
    if (m == nullptr) return fail(LPP_ERR_INVALID_ARG, "null model");
    for (int t = 0; t < LPP_T_COUNT; ++t)
        if (!m->w_loaded[t])
            return fail(LPP_ERR_STATE, "weight tensor %d has not been uploaded", t);
    return LPP_OK;
}

}  // namespace
}  // namespace lpp

extern "C" {

lpp_status lpp_model_create(lpp_model** out, const lpp_config* cfg) {
    LPP_REQUIRE(out && cfg, "lpp_model_create: null argument");
    *out = nullptr;
    const lpp_config& c = *cfg;
    LPP_REQUIRE(c.dim > 0 && c.hidden_dim > 0 && c.n_layers > 0 && c.n_heads > 0 && c.n_kv_heads > 0 &&
                    c.vocab_size > 0 && c.seq_len > 0,
                "lpp_model_create: every Config field must be positive");
    LPP_REQUIRE(c.dim % c.n_heads == 0, "lpp_model_create: dim %d not divisible by n_heads %d", c.dim, c.n_heads);
    LPP_REQUIRE(c.n_heads % c.n_kv_heads == 0, "lpp_model_create: n_heads %d not divisible by n_kv_heads %d",
                c.n_heads, c.n_kv_heads);
    LPP_REQUIRE((c.dim / c.n_heads) % 2 == 0, "lpp_model_create: head size %d must be even", c.dim / c.n_heads);
    if (c.weight_precision != LPP_WEIGHT_FP32 && c.weight_precision != LPP_WEIGHT_FP16)
        return fail(LPP_ERR_UNSUPPORTED, "lpp_model_create: weight_precision %d is not implemented",
                    c.weight_precision);
    LPP_TRY(lpp_init(0));

    lpp_model* m = new (std::nothrow) lpp_model();
    if (!m) return fail(LPP_ERR_OOM, "lpp_model_create: host allocation failed");
    m->cfg = c;
    m->head_size = c.dim / c.n_heads;
    m->kv_dim = c.dim * c.n_kv_heads / c.n_heads;
    m->gqa = c.n_heads / c.n_kv_heads;

    lpp_status st = LPP_OK;
    auto guard = [&](lpp_status s) {
        if (st == LPP_OK) st = s;
        return s == LPP_OK;
    };
    for (int t = 0; t < LPP_T_COUNT && st == LPP_OK; ++t) {
        m->w_bytes[t] = lpp::tensor_bytes(c, t);
        guard(lpp_malloc(&m->w[t], m->w_bytes[t]));
    }
    const size_t cache = static_cast<size_t>(c.n_layers) * c.seq_len * m->kv_dim;
    // model.cpp:58-80
    guard(lpp::dev_alloc(&m->x, c.dim, true)) && guard(lpp::dev_alloc(&m->xb, c.dim, true)) &&
        guard(lpp::dev_alloc(&m->xb2, c.dim, true)) && guard(lpp::dev_alloc(&m->hb, c.hidden_dim, true)) &&
        guard(lpp::dev_alloc(&m->he, c.hidden_dim, true)) && guard(lpp::dev_alloc(&m->q, c.dim, true)) &&
        guard(lpp::dev_alloc(&m->k, m->kv_dim, true)) && guard(lpp::dev_alloc(&m->v, m->kv_dim, true)) &&
        guard(lpp::dev_alloc(&m->att, static_cast<size_t>(c.n_heads) * c.seq_len, true)) &&
        guard(lpp::dev_alloc(&m->logits, c.vocab_size, true)) &&
        guard(lpp::dev_alloc(&m->key_cache, cache, true)) && guard(lpp::dev_alloc(&m->value_cache, cache, true)) &&
        guard(lpp::dev_alloc(&m->sampled_token, 1, true)) && guard(lpp::dev_alloc(&m->history, c.seq_len, true));
    if (st == LPP_OK) {
        uint16_t* ws = nullptr;
        guard(lpp::dev_alloc(&ws, c.hidden_dim > c.dim ? c.hidden_dim : c.dim, true));
        m->workspace_f16 = ws;
    }
    if (st == LPP_OK) guard(lpp::rope_table(m->head_size, c.rope_base, c.seq_len, &m->rope));
    if (st == LPP_OK) guard(lpp::fused_prepare(m));
    if (st == LPP_OK && hipEventCreate(&m->ev_a) != hipSuccess) st = fail(LPP_ERR_HIP, "hipEventCreate failed");
    if (st == LPP_OK && hipEventCreate(&m->ev_b) != hipSuccess) st = fail(LPP_ERR_HIP, "hipEventCreate failed");
    if (st == LPP_OK) guard(lpp_synchronize());
    if (st != LPP_OK) {
        char keep[512];
        std::strncpy(keep, lpp_last_error(), sizeof keep - 1);
        keep[sizeof keep - 1] = 0;
        lpp_model_destroy(m);
        return fail(st, "%s", keep);
    }
    *out = m;
    return LPP_OK;
}

lpp_status lpp_model_destroy(lpp_model* m) {
    if (!m) return LPP_OK;
    (void)hipStreamSynchronize(lpp::stream());
    lpp::fused_release(m);
    lpp::prefill_release(m);
    for (int t = 0; t < LPP_T_COUNT; ++t) lpp_free(m->w[t]);
    lpp_free(m->x); lpp_free(m->xb); lpp_free(m->xb2); lpp_free(m->hb); lpp_free(m->he);
    lpp_free(m->q); lpp_free(m->k); lpp_free(m->v); lpp_free(m->att); lpp_free(m->logits);
    lpp_free(m->key_cache); lpp_free(m->value_cache); lpp_free(m->workspace_f16);
    lpp_free(m->sampled_token); lpp_free(m->history);
    if (m->ev_a) (void)hipEventDestroy(m->ev_a);
    if (m->ev_b) (void)hipEventDestroy(m->ev_b);
    delete m;
    return LPP_OK;
}

lpp_status lpp_model_tensor_bytes(const lpp_model* m, int tensor, size_t* bytes) {
    LPP_REQUIRE(m && bytes, "lpp_model_tensor_bytes: null argument");
    LPP_REQUIRE(tensor >= 0 && tensor < LPP_T_COUNT, "lpp_model_tensor_bytes: tensor id %d", tensor);
    *bytes = m->w_bytes[tensor];
    return LPP_OK;
}

lpp_status lpp_model_upload(lpp_model* m, int tensor, size_t byte_offset, const void* host_src, size_t bytes) {
    LPP_REQUIRE(m && host_src, "lpp_model_upload: null argument");
    LPP_REQUIRE(tensor >= 0 && tensor < LPP_T_COUNT, "lpp_model_upload: tensor id %d", tensor);
    LPP_REQUIRE(byte_offset <= m->w_bytes[tensor] && bytes <= m->w_bytes[tensor] - byte_offset,
                "lpp_model_upload: [%zu, +%zu) exceeds tensor %d of %zu bytes", byte_offset, bytes, tensor,
                m->w_bytes[tensor]);
    LPP_TRY(lpp_memcpy_h2d(static_cast<char*>(m->w[tensor]) + byte_offset, host_src, bytes));
    if (byte_offset + bytes == m->w_bytes[tensor]) m->w_loaded[tensor] = true;
    return LPP_OK;
}

lpp_status lpp_model_tie_classifier(lpp_model* m) {
    LPP_REQUIRE(m != nullptr, "lpp_model_tie_classifier: null model");
    if (!m->w_loaded[LPP_T_TOKEN_EMBEDDING])
        return fail(LPP_ERR_STATE, "lpp_model_tie_classifier: embedding table not uploaded yet");
    const size_t total = static_cast<size_t>(m->cfg.vocab_size) * m->cfg.dim;
    if (m->cfg.weight_precision == LPP_WEIGHT_FP16) {
        // loader.cpp:621-627: binary16 copy of the fp32 table, cast on the device.
        const size_t step = 1u << 28;
        for (size_t off = 0; off < total; off += step) {
            const size_t n = (total - off < step) ? total - off : step;
            LPP_TRY(lpp_convert_f32_to_f16(static_cast<lpp_half*>(m->w[LPP_T_WCLS]) + off,
                                           static_cast<const float*>(m->w[LPP_T_TOKEN_EMBEDDING]) + off,
                                           static_cast<int>(n)));
        }
    } else {
        LPP_TRY(lpp_memcpy_d2d(m->w[LPP_T_WCLS], m->w[LPP_T_TOKEN_EMBEDDING], total * 4));
    }
    LPP_TRY(lpp_synchronize());
    m->w_loaded[LPP_T_WCLS] = true;
    return LPP_OK;
}

lpp_status lpp_model_tensor_ptr(lpp_model* m, int tensor, void** d_ptr) {
    LPP_REQUIRE(m && d_ptr, "lpp_model_tensor_ptr: null argument");
    LPP_REQUIRE(tensor >= 0 && tensor < LPP_T_COUNT, "lpp_model_tensor_ptr: tensor id %d", tensor);
    *d_ptr = m->w[tensor];
    return LPP_OK;
}

lpp_status lpp_model_buffer_ptr(lpp_model* m, int buffer, void** d_ptr, size_t* bytes) {
    LPP_REQUIRE(m && d_ptr, "lpp_model_buffer_ptr: null argument");
    const lpp_config& c = m->cfg;
    const size_t cache = static_cast<size_t>(c.n_layers) * c.seq_len * m->kv_dim;
    void* p = nullptr;
    size_t n = 0;
    switch (buffer) {
        case LPP_B_X: p = m->x; n = c.dim * 4u; break;
        case LPP_B_XB: p = m->xb; n = c.dim * 4u; break;
        case LPP_B_XB2: p = m->xb2; n = c.dim * 4u; break;
        case LPP_B_HB: p = m->hb; n = c.hidden_dim * 4u; break;
        case LPP_B_HE: p = m->he; n = c.hidden_dim * 4u; break;
        case LPP_B_Q: p = m->q; n = c.dim * 4u; break;
        case LPP_B_K: p = m->k; n = m->kv_dim * 4u; break;
        case LPP_B_V: p = m->v; n = m->kv_dim * 4u; break;
        case LPP_B_ATT: p = m->att; n = static_cast<size_t>(c.n_heads) * c.seq_len * 4u; break;
        case LPP_B_LOGITS: p = m->logits; n = c.vocab_size * 4u; break;
        case LPP_B_KEY_CACHE: p = m->key_cache; n = cache * 2u; break;
        case LPP_B_VALUE_CACHE: p = m->value_cache; n = cache * 2u; break;
        default: return fail(LPP_ERR_INVALID_ARG, "lpp_model_buffer_ptr: buffer id %d", buffer);
    }
    *d_ptr = p;
    if (bytes) *bytes = n;
    return LPP_OK;
}

lpp_status lpp_model_set_path(lpp_model* m, int path) {
    LPP_REQUIRE(m != nullptr, "lpp_model_set_path: null model");
    LPP_REQUIRE(path == LPP_PATH_OPS || path == LPP_PATH_FUSED || path == LPP_PATH_PERSISTENT,
                "lpp_model_set_path: path %d", path);
    if (path == LPP_PATH_PERSISTENT)
        if (const char* why = lpp::dataflow_unsupported_reason(m)) return lpp::fail(LPP_ERR_UNSUPPORTED, "%s", why);
    m->path = path;
    return LPP_OK;
}

lpp_status lpp_model_set_spin_limit(lpp_model* m, unsigned polls) {
    LPP_REQUIRE(m != nullptr && polls > 0u, "lpp_model_set_spin_limit: null model or zero bound");
    m->spin_limit = polls;
    return LPP_OK;
}

lpp_status lpp_model_set_sequence_base(lpp_model* m, unsigned base) {
    LPP_REQUIRE(m != nullptr, "lpp_model_set_sequence_base: null model");
    m->df_base = base;
    return LPP_OK;
}

lpp_status lpp_model_reset(lpp_model* m) {
    LPP_REQUIRE(m != nullptr, "lpp_model_reset: null model");
    const size_t cache = static_cast<size_t>(m->cfg.n_layers) * m->cfg.seq_len * m->kv_dim;
    LPP_TRY(lpp_memset(m->key_cache, 0, cache * 2));
    LPP_TRY(lpp_memset(m->value_cache, 0, cache * 2));
    return lpp_synchronize();
}

// model.cpp:121-160, CUDA branch.
lpp_status lpp_attention(lpp_model* m, int layer, int pos) {
    LPP_TRY(lpp::check_ready(m));
    const lpp_config& c = m->cfg;
    LPP_REQUIRE(layer >= 0 && layer < c.n_layers, "lpp_attention: layer %d", layer);
    LPP_REQUIRE(pos >= 0 && pos < c.seq_len, "lpp_attention: pos %d outside [0, %d)", pos, c.seq_len);
    const int dim = c.dim, kv_dim = m->kv_dim, hs = m->head_size;
    const size_t off_qkv = static_cast<size_t>(layer) * dim * dim;
    const size_t off_kv = static_cast<size_t>(layer) * kv_dim * dim;
    const int prec = c.weight_precision;

    LPP_TRY(lpp_gemv(m->q, m->xb, lpp::weight_at(m, LPP_T_WQ, off_qkv), m->workspace_f16, dim, dim, prec));
    LPP_TRY(lpp_gemv(m->k, m->xb, lpp::weight_at(m, LPP_T_WK, off_kv), m->workspace_f16, kv_dim, dim, prec));
    LPP_TRY(lpp_gemv(m->v, m->xb, lpp::weight_at(m, LPP_T_WV, off_kv), m->workspace_f16, kv_dim, dim, prec));
    LPP_TRY(lpp_rope(m->q, m->k, pos, dim, kv_dim, hs, c.rope_base));
    LPP_TRY(lpp_scatter_kv(m->key_cache, m->value_cache, m->k, m->v, layer, pos, c.n_kv_heads, hs, c.seq_len));
    LPP_TRY(lpp_multihead_gemv(m->att, m->q, m->key_cache, layer, pos, c.n_heads, c.n_kv_heads, hs, c.seq_len));
    const float scale = 1.0f / sqrtf(static_cast<float>(hs));
    LPP_TRY(lpp_scale_multihead(m->att, scale, c.n_heads, pos + 1, c.seq_len));
    LPP_TRY(lpp_softmax_multihead(m->att, m->att, c.n_heads, pos + 1, c.seq_len));
    const size_t layer_v = static_cast<size_t>(layer) * kv_dim * c.seq_len;
    LPP_TRY(lpp_aggregation_multihead(m->xb, m->value_cache + layer_v, m->att, c.n_heads, pos + 1, hs, m->gqa,
                                      c.seq_len));
    LPP_TRY(lpp_gemv(m->xb2, m->xb, lpp::weight_at(m, LPP_T_WO, off_qkv), m->workspace_f16, dim, dim, prec));
    return LPP_OK;
}

// model.cpp:205-226, CUDA branch.
lpp_status lpp_transformer_block(lpp_model* m, int layer, int pos) {
    LPP_TRY(lpp::check_ready(m));
    const lpp_config& c = m->cfg;
    LPP_REQUIRE(layer >= 0 && layer < c.n_layers, "lpp_transformer_block: layer %d", layer);
    const int dim = c.dim, hidden = c.hidden_dim;
    const size_t off_ffn = static_cast<size_t>(layer) * hidden * dim;
    const size_t off_norm = static_cast<size_t>(layer) * dim;
    const int prec = c.weight_precision;
    const float* rms_att = static_cast<const float*>(m->w[LPP_T_RMS_ATT]) + off_norm;
    const float* rms_ffn = static_cast<const float*>(m->w[LPP_T_RMS_FFN]) + off_norm;

    LPP_TRY(lpp_rmsnorm(m->xb, m->x, rms_att, dim));
    LPP_TRY(lpp_attention(m, layer, pos));
    LPP_TRY(lpp_residual_add(m->x, m->x, m->xb2, dim));
    LPP_TRY(lpp_rmsnorm(m->xb, m->x, rms_ffn, dim));
    LPP_TRY(lpp_gemv(m->hb, m->xb, lpp::weight_at(m, LPP_T_W1, off_ffn), m->workspace_f16, hidden, dim, prec));
    LPP_TRY(lpp_gemv(m->he, m->xb, lpp::weight_at(m, LPP_T_W3, off_ffn), m->workspace_f16, hidden, dim, prec));
    LPP_TRY(lpp_swiglu(m->hb, m->hb, m->he, hidden));
    LPP_TRY(lpp_gemv(m->xb2, m->hb, lpp::weight_at(m, LPP_T_W2, off_ffn), m->workspace_f16, dim, hidden, prec));
    LPP_TRY(lpp_residual_add(m->x, m->x, m->xb2, dim));
    return LPP_OK;
}

namespace {

// model.cpp:342-371 on the operator path.  The embedding row is gathered from
// the device-resident table instead of crossing PCIe each token.
lpp_status forward_ops(lpp_model* m, int token, int pos, float temperature, float topp, float penalty,
                       const int* history, int history_len, float r, int* next_token) {
    const lpp_config& c = m->cfg;
    const float* row = static_cast<const float*>(m->w[LPP_T_TOKEN_EMBEDDING]) + static_cast<size_t>(token) * c.dim;
    LPP_TRY(lpp_memcpy_d2d(m->x, row, static_cast<size_t>(c.dim) * 4));
    for (int layer = 0; layer < c.n_layers; ++layer) LPP_TRY(lpp_transformer_block(m, layer, pos));
    LPP_TRY(lpp_rmsnorm(m->x, m->x, static_cast<const float*>(m->w[LPP_T_RMS_FINAL]), c.dim));
    LPP_TRY(lpp_gemv(m->logits, m->x, m->w[LPP_T_WCLS], m->workspace_f16, c.vocab_size, c.dim, c.weight_precision));
    const bool use_history = penalty > 1.0f && history != nullptr && history_len > 0;
    if (use_history) {
        LPP_REQUIRE(history_len <= c.seq_len, "lpp_forward: history_len %d exceeds seq_len %d", history_len, c.seq_len);
        LPP_TRY(lpp_memcpy_h2d(m->history, history, static_cast<size_t>(history_len) * sizeof(int)));
    }
    LPP_TRY(lpp_sample(m->logits, c.vocab_size, temperature, topp, penalty, use_history ? m->history : nullptr,
                       history_len, m->sampled_token, nullptr, r));
    LPP_TRY(lpp_memcpy_d2h(next_token, m->sampled_token, sizeof(int)));
    return LPP_OK;
}

}  // namespace

}  // extern "C"

// Stand-alone timing of the operators of section A as forward_ops launches them at position `pos`: every class is
// launched as often as one token launches it (one launch per layer, so successive launches stream different weights),
// `reps` tokens' worth between two events on the launch stream.  bytes = what the operator has to move at least once
// (weights or cache rows once, vectors in and out).  The run state is left holding whatever the operators wrote.
lpp_status lpp::ops_profile(lpp_model* m, int pos, int reps, lpp_kernel_time* out, int capacity, int* count) {
    const lpp_config& c = m->cfg;
    const int L = c.n_layers, dim = c.dim, kv = m->kv_dim, hidden = c.hidden_dim, hs = m->head_size, prec = c.weight_precision;
    const double wb = prec == LPP_WEIGHT_FP16 ? 2.0 : 4.0;
    const int npos = pos + 1;
    hipStream_t s = lpp::stream();
    int n = 0;
    auto timed = [&](const char* name, int per_token, double bytes, auto launch_layer) -> lpp_status {
        for (int l = 0; l < (per_token > 0 ? L : 1); ++l) LPP_TRY(launch_layer(l));  // warm-up: code objects, tables
        LPP_HIP(hipStreamSynchronize(s));
        LPP_HIP(hipEventRecord(m->ev_a, s));
        int launches = 0;
        for (int r = 0; r < reps; ++r)
            for (int l = 0; l < L; ++l) {
                const int before = launches;
                LPP_TRY(launch_layer(l));
                launches = before + 1;
            }
        LPP_HIP(hipEventRecord(m->ev_b, s));
        LPP_HIP(hipEventSynchronize(m->ev_b));
        float ms = 0.0f;
        LPP_HIP(hipEventElapsedTime(&ms, m->ev_a, m->ev_b));
        if (n < capacity) {
            std::snprintf(out[n].name, sizeof out[n].name, "%s", name);
            out[n].launches_per_token = per_token;
            out[n].avg_ms = static_cast<double>(ms) / launches;
            out[n].bytes_per_launch = bytes;
        }
        ++n;
        return LPP_OK;
    };
    auto gemv_bytes = [&](double rows, double cols) { return rows * cols * wb + 4.0 * cols + 4.0 * rows; };
    const float* rms_att = static_cast<const float*>(m->w[LPP_T_RMS_ATT]);
    LPP_TRY(lpp_memset(m->att, 0, static_cast<size_t>(c.n_heads) * c.seq_len * sizeof(float)));
    LPP_TRY(timed("gemv Wq", L, gemv_bytes(dim, dim), [&](int l) {
        return lpp_gemv(m->q, m->xb, lpp::weight_at(m, LPP_T_WQ, static_cast<size_t>(l) * dim * dim), m->workspace_f16, dim, dim, prec);
    }));
    LPP_TRY(timed("gemv Wk, Wv", 2 * L, gemv_bytes(kv, dim), [&](int l) {
        return lpp_gemv(m->k, m->xb, lpp::weight_at(m, (l & 1) ? LPP_T_WV : LPP_T_WK, static_cast<size_t>(l) * kv * dim), m->workspace_f16, kv, dim, prec);
    }));
    LPP_TRY(timed("gemv Wo", L, gemv_bytes(dim, dim), [&](int l) {
        return lpp_gemv(m->xb2, m->xb, lpp::weight_at(m, LPP_T_WO, static_cast<size_t>(l) * dim * dim), m->workspace_f16, dim, dim, prec);
    }));
    LPP_TRY(timed("gemv W1, W3", 2 * L, gemv_bytes(hidden, dim), [&](int l) {
        return lpp_gemv(m->hb, m->xb, lpp::weight_at(m, (l & 1) ? LPP_T_W3 : LPP_T_W1, static_cast<size_t>(l) * hidden * dim), m->workspace_f16, hidden, dim, prec);
    }));
    LPP_TRY(timed("gemv W2", L, gemv_bytes(dim, hidden), [&](int l) {
        return lpp_gemv(m->xb2, m->hb, lpp::weight_at(m, LPP_T_W2, static_cast<size_t>(l) * hidden * dim), m->workspace_f16, dim, hidden, prec);
    }));
    LPP_TRY(timed("gemv classifier", 1, gemv_bytes(c.vocab_size, dim), [&](int) {
        return lpp_gemv(m->logits, m->x, m->w[LPP_T_WCLS], m->workspace_f16, c.vocab_size, dim, prec);
    }));
    LPP_TRY(timed("convert_f32_to_f16", 0, 6.0 * hidden, [&](int) {  // (never launched by forward: x stays fp32)
        return lpp_convert_f32_to_f16(static_cast<lpp_half*>(m->workspace_f16), m->hb, hidden);
    }));
    LPP_TRY(timed("rmsnorm", 2 * L + 1, 12.0 * dim, [&](int l) { return lpp_rmsnorm(m->xb, m->x, rms_att + static_cast<size_t>(l) * dim, dim); }));
    LPP_TRY(timed("rope", L, 8.0 * (dim + kv), [&](int) { return lpp_rope(m->q, m->k, pos, dim, kv, hs, c.rope_base); }));
    LPP_TRY(timed("scatter_kv", L, 12.0 * kv, [&](int l) {
        return lpp_scatter_kv(m->key_cache, m->value_cache, m->k, m->v, l, pos, c.n_kv_heads, hs, c.seq_len);
    }));
    LPP_TRY(timed("multihead_gemv", L, 2.0 * kv * npos + 4.0 * dim + 4.0 * c.n_heads * npos, [&](int l) {
        return lpp_multihead_gemv(m->att, m->q, m->key_cache, l, pos, c.n_heads, c.n_kv_heads, hs, c.seq_len);
    }));
    LPP_TRY(timed("scale_multihead", L, 8.0 * c.n_heads * npos, [&](int) {
        return lpp_scale_multihead(m->att, 1.0f / sqrtf(static_cast<float>(hs)), c.n_heads, npos, c.seq_len);
    }));
    LPP_TRY(timed("softmax_multihead", L, 8.0 * c.n_heads * npos, [&](int) {
        return lpp_softmax_multihead(m->att, m->att, c.n_heads, npos, c.seq_len);
    }));
    LPP_TRY(timed("aggregation_multihead", L, 2.0 * kv * npos + 4.0 * c.n_heads * npos + 4.0 * dim, [&](int l) {
        return lpp_aggregation_multihead(m->xb, m->value_cache + static_cast<size_t>(l) * kv * c.seq_len, m->att, c.n_heads, npos, hs,
                                         m->gqa, c.seq_len);
    }));
    LPP_TRY(timed("residual_add", 2 * L, 12.0 * dim, [&](int) { return lpp_residual_add(m->x, m->x, m->xb2, dim); }));
    LPP_TRY(timed("swiglu", L, 12.0 * hidden, [&](int) { return lpp_swiglu(m->hb, m->hb, m->he, hidden); }));
    LPP_TRY(timed("sample", 1, 8.0 * c.vocab_size, [&](int) {
        return lpp_sample(m->logits, c.vocab_size, 0.8f, 1.0f, 1.0f, nullptr, 0, m->sampled_token, nullptr, 0.5f);
    }));
    *count = n < capacity ? n : capacity;
    return LPP_OK;
}

extern "C" {

lpp_status lpp_forward(lpp_model* m, int token, int pos, float temperature, float topp, float penalty,
                       const int* history, int history_len, float r, int* next_token) {
    LPP_TRY(lpp::check_ready(m));
    LPP_REQUIRE(next_token != nullptr, "lpp_forward: null output");
    LPP_REQUIRE(token >= 0 && token < m->cfg.vocab_size, "lpp_forward: token %d outside [0, %d)", token,
                m->cfg.vocab_size);
    LPP_REQUIRE(pos >= 0 && pos < m->cfg.seq_len, "lpp_forward: pos %d outside [0, %d)", pos, m->cfg.seq_len);
    LPP_REQUIRE(history_len >= 0, "lpp_forward: history_len %d", history_len);
    if (m->path == LPP_PATH_OPS)
        return forward_ops(m, token, pos, temperature, topp, penalty, history, history_len, r, next_token);
    return lpp::fused_forward(m, token, pos, temperature, penalty, history, history_len, r, next_token);
}

lpp_status lpp_generate(lpp_model* m, int first_token, int start_pos, int n_steps, float temperature, float topp,
                        float penalty, int* history, int* history_len, int history_cap, const float* uniforms,
                        int* out_tokens, lpp_gen_stats* stats) {
    LPP_TRY(lpp::check_ready(m));
    LPP_REQUIRE(n_steps >= 0 && out_tokens != nullptr, "lpp_generate: n_steps %d / null output", n_steps);
    LPP_REQUIRE(start_pos >= 0 && start_pos + n_steps <= m->cfg.seq_len,
                "lpp_generate: positions [%d, %d) exceed seq_len %d", start_pos, start_pos + n_steps, m->cfg.seq_len);
    LPP_REQUIRE(first_token >= 0 && first_token < m->cfg.vocab_size, "lpp_generate: first_token %d", first_token);
    LPP_REQUIRE(temperature == 0.0f || uniforms != nullptr, "lpp_generate: uniforms required when temperature != 0");
    int local_len = 0;
    if (history_len == nullptr) history_len = &local_len;
    LPP_REQUIRE(history_cap >= 0 && *history_len >= 0 && *history_len <= history_cap,
                "lpp_generate: history_len %d / capacity %d", *history_len, history_cap);
    LPP_REQUIRE(history_cap == 0 || history != nullptr, "lpp_generate: null history with capacity %d", history_cap);
    LPP_REQUIRE(history_cap <= m->cfg.seq_len, "lpp_generate: history capacity %d exceeds seq_len %d", history_cap,
                m->cfg.seq_len);
    if (stats) std::memset(stats, 0, sizeof *stats);
    if (m->path != LPP_PATH_OPS)
        return lpp::fused_generate(m, first_token, start_pos, n_steps, temperature, penalty, history, history_len,
                                   history_cap, uniforms, out_tokens, stats);

    hipStream_t s = lpp::stream();
    LPP_HIP(hipEventRecord(m->ev_a, s));
    const auto t0 = std::chrono::steady_clock::now();
    int token = first_token;
    for (int i = 0; i < n_steps; ++i) {
        const float r = uniforms ? uniforms[i] : 0.0f;
        LPP_TRY(forward_ops(m, token, start_pos + i, temperature, topp, penalty, history, *history_len, r, &token));
        out_tokens[i] = token;
        // main.cpp:203-208
        if (history_cap > 0) {
            if (*history_len < history_cap) {
                history[(*history_len)++] = token;
            } else {
                std::memmove(history, history + 1, static_cast<size_t>(history_cap - 1) * sizeof(int));
                history[history_cap - 1] = token;
            }
        }
    }
    const auto t1 = std::chrono::steady_clock::now();
    LPP_HIP(hipEventRecord(m->ev_b, s));
    LPP_HIP(hipEventSynchronize(m->ev_b));
    if (stats) {
        float ms = 0.0f;
        LPP_HIP(hipEventElapsedTime(&ms, m->ev_a, m->ev_b));
        stats->wall_seconds = std::chrono::duration<double>(t1 - t0).count();
        stats->device_ms = ms;
        stats->tokens = n_steps;
    }
    return LPP_OK;
}

}  // extern "C"
