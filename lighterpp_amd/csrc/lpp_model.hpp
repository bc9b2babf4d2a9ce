// lpp_model.hpp -- the model object behind section B of lpp.h.
#pragma once

#include <hip/hip_runtime.h>

#include <vector>

#include "lpp_internal.hpp"

// Everything forward() touches, resident in HBM.  Field names follow
// transformerWeights and RunState (reference src/model.h:34-115).
namespace lpp {
struct StepParams;
}

struct lpp_model {
    lpp_config cfg{};
    int kv_dim = 0;
    int head_size = 0;
    int gqa = 0;
    int path = LPP_PATH_OPS;

    // Weights, stacked per layer: [L][rows][cols].  Matrices are binary16 or fp32
    // according to cfg.weight_precision; embedding and norm gains are fp32.
    void* w[LPP_T_COUNT] = {};
    size_t w_bytes[LPP_T_COUNT] = {};
    bool w_loaded[LPP_T_COUNT] = {};

    // Run state (model.h:96-114).
    float* x = nullptr;
    float* xb = nullptr;
    float* xb2 = nullptr;
    float* hb = nullptr;
    float* he = nullptr;
    float* q = nullptr;
    float* k = nullptr;
    float* v = nullptr;
    float* att = nullptr;
    float* logits = nullptr;
    uint16_t* key_cache = nullptr;    // [L][n_kv_heads][seq_len][head_size]
    uint16_t* value_cache = nullptr;
    void* workspace_f16 = nullptr;    // kept for the operator signature; unused
    int* sampled_token = nullptr;     // [1]
    int* history = nullptr;           // [seq_len]

    // Fused paths: per-token scalars live on the device so that a recorded
    // graph can be replayed without touching its nodes.
    struct lpp::StepParams* step = nullptr;       // device
    struct lpp::StepParams* step_host = nullptr;  // pinned host mirror
    int* pinned_tokens = nullptr;            // pinned host landing area for sampled ids
    int* pinned_tokens_dev = nullptr;        // the same memory as the device addresses it
    float* att_partial = nullptr;            // split-context attention partials
    float* work_logits = nullptr;            // sampler working copy of the logits
    unsigned* sync_words = nullptr;          // arrival counters of the attention combine; abort flag
    float* sample_scratch = nullptr;         // 4 x kMaxChunks words
    float* gen_uniforms = nullptr;           // device copy of the per-step draws
    int gen_cap = 0;
    void* tagged = nullptr;                  // value+sequence-number vectors of the persistent kernel
    void* df_rows[3] = {nullptr, nullptr, nullptr};  // row lists of the persistent kernel's streaming wavefronts: [0] every row
    int df_row_stride[3] = {0, 0, 0};        // streamed, [1] with parked gate/up rows left out (short contexts), [2] the
                                             // same for the plan that splits a context over an XCD
    const void* df_rows_key[12] = {};        // weight addresses the lists were built from
    int* df_gu_first[3] = {nullptr, nullptr, nullptr};  // device tables of the gate/up partition the lists were built for
    std::vector<float> df_gu_weight;         // per workgroup: its share of the hidden units relative to an even deal
    bool df_calibrated = false;              // a traced token has set df_gu_weight (or could not)
    // Host's own count of the step record for the persistent path: everything but the token id
    // is known before a launch and travels as kernel arguments.
    int df_pos = 0, df_history_len = 0, df_history_cap = 0, df_step_index = 0, df_freeze = 0;
    float df_temperature = 0.0f, df_penalty = 1.0f, df_r = 0.0f;
    const float* df_uniforms_host = nullptr; // per-step draws of the generate call in progress (host memory)
    unsigned df_base = 0;                    // sequence-number base of the next persistent launch
    int df_trace_stride = 0;                 // timeline words per workgroup when every workgroup is traced (0: workgroup 0 only)
    int persist_grid = 0;                    // workgroups of the persistent kernel (0: not sized yet)
    unsigned df_ticket_base = 0;             // what the per-XCD workgroup counters read before the next persistent launch
    int df_xcc = 0;                          // XCDs the persistent kernel's workgroups go round (1: near copies off; 0: not probed)
    unsigned df_options_epoch = 0;           // test_options_epoch() the plans and lists were made under
    unsigned spin_limit = 1u << 20;          // polls a wait for tagged inputs may take before giving up
    const float2* rope = nullptr;            // [seq_len][head_size/2] (cos, sin)
    int max_splits = 1;
    bool fused_ok = false;                   // shape supported by the fused kernels
    char fused_why[160] = "";

    void* pf_buf[12] = {};                   // batched prefill: activations of a chunk of tokens (prefill.hip)
    int pf_cap = 0;                          // tokens those buffers hold
    int pf_mode = 0;                         // LPP_PREFILL_EXACT / LPP_PREFILL_FAST

    hipGraphExec_t graph_exec[2] = {nullptr, nullptr};  // [0] without, [1] with uniforms/out arrays
    hipEvent_t ev_a = nullptr, ev_b = nullptr;
};

namespace lpp {

// Per-token scalars the fused kernels read from device memory, so that a
// recorded graph can be replayed without touching its nodes.
struct StepParams {
    int token;         // input token id; replaced by the sampled id at the end of the step
    int pos;           // position of this token; advanced at the end of the step
    int history_len;   // valid entries in the device penalty window
    int history_cap;   // capacity of the window (0: no window kept)
    int history_next;  // ring slot the next sampled id goes to
    int step_index;    // index into uniforms[] / out_tokens[]
    float temperature;
    float penalty;
    float r;           // uniform draw when no uniforms[] array is attached
    unsigned epoch;    // unused (kept so the record's layout stays put)
    int error;         // set by a kernel that gave up (bounded waits)
    int freeze;        // nonzero: a step leaves token/position/window as they are (timing replays)
};

size_t tensor_bytes(const lpp_config& c, int tensor);

// Implemented in prefill.hip: frees the batched prefill's buffers.
void prefill_release(lpp_model* m);

// Implemented in dataflow_decode.hip: why LPP_PATH_PERSISTENT cannot take this model's shape, or nullptr.
const char* dataflow_unsupported_reason(const lpp_model* m);

// Implemented in lpp_model.cpp: stand-alone timing of the operators of lpp.h section A (lpp_profile_kernels on LPP_PATH_OPS).
lpp_status ops_profile(lpp_model* m, int pos, int reps, lpp_kernel_time* out, int capacity, int* count);

// Implemented in fused_decode.hip.
lpp_status fused_prepare(lpp_model* m);
lpp_status fused_release(lpp_model* m);
// forward() and the generation loop on LPP_PATH_FUSED / LPP_PATH_PERSISTENT.
lpp_status fused_forward(lpp_model* m, int token, int pos, float temperature, float penalty,
                         const int* history, int history_len, float r, int* next_token);
lpp_status fused_generate(lpp_model* m, int first_token, int start_pos, int n_steps, float temperature,
                          float penalty, int* history, int* history_len, int history_cap,
                          const float* uniforms, int* out_tokens, lpp_gen_stats* stats);

}  // namespace lpp
