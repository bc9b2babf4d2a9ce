// fused_decode.hip -- LPP_PATH_FUSED: one token of forward() (reference
// src/model.cpp:342-371) as 5 launches per layer + classifier + sampler steps,
// recorded once into a HIP graph and replayed per token.  All per-token
// scalars (token, position, penalty window, uniform draw) live in device
// memory, so the graph is never patched; the sampled id is fed back on the
// device, and the host only collects 4 bytes per token.
#include <chrono>
#include <cstring>
#include <vector>

#include "decode_phases.hpp"

namespace lpp {
namespace {

using namespace ph;

constexpr int kThreads = 256;
constexpr int kWavesPerWg = kThreads / dev::kWave;

struct NoWait {
    __device__ __forceinline__ void operator()() const {}
};

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_qkv(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    phase_qkv<kF16, 2>(a, layer, blockIdx.x, gridDim.x, lds, NoWait{});
}

__global__ __launch_bounds__(kThreads) void k_attention(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    phase_attention(a, layer, blockIdx.x, gridDim.x, lds, NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_oproj(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    const int wbytes = kF16 ? 2 : 4;
    const char* w = a.wo + static_cast<size_t>(layer) * a.dim * a.dim * wbytes;
    phase_proj_residual<kF16, 2>(w, a.dim, a.dim, a.xb, layer_input(a, layer), a.x, blockIdx.x, gridDim.x, lds,
                                 NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_gateup(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    phase_gateup<kF16, 2>(a, layer, blockIdx.x, gridDim.x, lds, NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_down(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    const int wbytes = kF16 ? 2 : 4;
    const char* w = a.w2 + static_cast<size_t>(layer) * a.dim * a.hidden * wbytes;
    phase_proj_residual<kF16, 1>(w, a.dim, a.hidden, a.hb, a.x, a.x, blockIdx.x, gridDim.x, lds, NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_lmhead(DecodeArgs a) {
    extern __shared__ __align__(16) float lds[];
    phase_lmhead<kF16, 4>(a, blockIdx.x, gridDim.x, lds, NoWait{});
}

// Sampler steps; one workgroup per vocabulary chunk.
__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_scale(DecodeArgs a, int chunk) {
    const StepParams* sp = a.step;
    smp::scale_max_chunk(a.logits, a.work, a.vocab, chunk, blockIdx.x, sp->temperature, sp->penalty,
                         sp->history_len > 0 ? a.history : nullptr, sp->history_len, a.sample_scratch);
}

__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_exp(DecodeArgs a, int chunk, int nchunks) {
    if (a.step->temperature == 0.0f) {
        // model.cpp:272-283: greedy; one workgroup finishes the token.
        if (blockIdx.x == 0) {
            const int tok = smp::argmax_over_chunks(nchunks, a.sample_scratch);
            if (threadIdx.x == 0) a.sampled[0] = tok;
        }
        return;
    }
    smp::exp_sum_chunk(a.work, a.vocab, chunk, nchunks, blockIdx.x, a.sample_scratch);
}

__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_norm(DecodeArgs a, int chunk, int nchunks) {
    if (a.step->temperature == 0.0f) return;
    smp::normalise_chunk(a.work, a.vocab, chunk, nchunks, blockIdx.x, a.sample_scratch);
    if (blockIdx.x == 0 && threadIdx.x == 0) a.sampled[0] = a.vocab - 1;  // model.cpp:302
}

__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_search(DecodeArgs a, int chunk) {
    if (a.step->temperature == 0.0f) return;
    smp::cdf_search_chunk(a.work, a.vocab, chunk, blockIdx.x, step_uniform(a), a.sample_scratch, a.sampled);
}

__global__ void k_finish(DecodeArgs a) {
    if (threadIdx.x == 0 && blockIdx.x == 0) finish_token(a, a.sampled[0]);
}

DecodeArgs make_args(const lpp_model* m, bool with_arrays) {
    DecodeArgs a{};
    const lpp_config& c = m->cfg;
    a.dim = c.dim;
    a.hidden = c.hidden_dim;
    a.n_layers = c.n_layers;
    a.n_heads = c.n_heads;
    a.n_kv_heads = c.n_kv_heads;
    a.head_size = m->head_size;
    a.kv_dim = m->kv_dim;
    a.vocab = c.vocab_size;
    a.seq_len = c.seq_len;
    a.gqa = m->gqa;
    a.max_splits = m->max_splits;
    a.emb = static_cast<const float*>(m->w[LPP_T_TOKEN_EMBEDDING]);
    a.rms_att = static_cast<const float*>(m->w[LPP_T_RMS_ATT]);
    a.wq = static_cast<const char*>(m->w[LPP_T_WQ]);
    a.wk = static_cast<const char*>(m->w[LPP_T_WK]);
    a.wv = static_cast<const char*>(m->w[LPP_T_WV]);
    a.wo = static_cast<const char*>(m->w[LPP_T_WO]);
    a.rms_ffn = static_cast<const float*>(m->w[LPP_T_RMS_FFN]);
    a.w1 = static_cast<const char*>(m->w[LPP_T_W1]);
    a.w2 = static_cast<const char*>(m->w[LPP_T_W2]);
    a.w3 = static_cast<const char*>(m->w[LPP_T_W3]);
    a.rms_final = static_cast<const float*>(m->w[LPP_T_RMS_FINAL]);
    a.wcls = static_cast<const char*>(m->w[LPP_T_WCLS]);
    a.x = m->x;
    a.xb = m->xb;
    a.q = m->q;
    a.k = m->k;
    a.v = m->v;
    a.hb = m->hb;
    a.logits = m->logits;
    a.work = m->work_logits;
    a.key_cache = m->key_cache;
    a.value_cache = m->value_cache;
    a.att_partial = m->att_partial;
    a.att_count = m->sync_words;
    a.rope = m->rope;
    a.step = m->step;
    a.history = m->history;
    a.uniforms = with_arrays ? m->gen_uniforms : nullptr;
    a.out_tokens = with_arrays ? m->gen_tokens : nullptr;
    a.sampled = m->sampled_token;
    float* sc = m->sample_scratch;
    a.sample_scratch = smp::SampleScratch{sc, reinterpret_cast<int*>(sc + smp::kMaxChunks),
                                          sc + 2 * smp::kMaxChunks, sc + 3 * smp::kMaxChunks};
    return a;
}

int blocks_for_tiles(int ntiles) {
    int blocks = (ntiles + kWavesPerWg - 1) / kWavesPerWg;
    const int cap = compute_units() * 8;
    if (blocks > cap) blocks = cap;
    return blocks < 1 ? 1 : blocks;
}

// Enqueue every launch of one token on `s`.
template <bool kF16>
lpp_status enqueue_token(const lpp_model* m, const DecodeArgs& a, hipStream_t s) {
    const lpp_config& c = m->cfg;
    const size_t lds_dim = static_cast<size_t>((c.dim + 7) & ~7) * 4;
    const size_t lds_hidden = static_cast<size_t>((c.hidden_dim + 7) & ~7) * 4;
    const size_t lds_att = static_cast<size_t>(attention_lds_floats(m->gqa, m->head_size, kThreads)) * 4;
    const int qkv_tiles = (c.dim + 2 * m->kv_dim + 1) / 2;
    const int o_tiles = (c.dim + 1) / 2;
    const int gu_tiles = (c.hidden_dim + 1) / 2;
    const int down_tiles = c.dim;
    const int lm_tiles = (c.vocab_size + 3) / 4;
    const int att_blocks = c.n_kv_heads * m->max_splits;
    for (int layer = 0; layer < c.n_layers; ++layer) {
        hipLaunchKernelGGL((k_qkv<kF16>), dim3(blocks_for_tiles(qkv_tiles)), dim3(kThreads), lds_dim, s, a, layer);
        hipLaunchKernelGGL(k_attention, dim3(att_blocks), dim3(kThreads), lds_att, s, a, layer);
        hipLaunchKernelGGL((k_oproj<kF16>), dim3(blocks_for_tiles(o_tiles)), dim3(kThreads), lds_dim, s, a, layer);
        hipLaunchKernelGGL((k_gateup<kF16>), dim3(blocks_for_tiles(gu_tiles)), dim3(kThreads), lds_dim, s, a, layer);
        hipLaunchKernelGGL((k_down<kF16>), dim3(blocks_for_tiles(down_tiles)), dim3(kThreads), lds_hidden, s, a,
                           layer);
    }
    hipLaunchKernelGGL((k_lmhead<kF16>), dim3(blocks_for_tiles(lm_tiles)), dim3(kThreads), lds_dim, s, a);
    const int chunk = smp::chunk_size_for(c.vocab_size);
    const int nchunks = (c.vocab_size + chunk - 1) / chunk;
    hipLaunchKernelGGL(k_sample_scale, dim3(nchunks), dim3(smp::kSampleThreads), 0, s, a, chunk);
    hipLaunchKernelGGL(k_sample_exp, dim3(nchunks), dim3(smp::kSampleThreads), 0, s, a, chunk, nchunks);
    hipLaunchKernelGGL(k_sample_norm, dim3(nchunks), dim3(smp::kSampleThreads), 0, s, a, chunk, nchunks);
    hipLaunchKernelGGL(k_sample_search, dim3(nchunks), dim3(smp::kSampleThreads), 0, s, a, chunk);
    hipLaunchKernelGGL(k_finish, dim3(1), dim3(64), 0, s, a);
    LPP_CHECK_LAUNCH("fused token");
    return LPP_OK;
}

lpp_status enqueue_token_any(const lpp_model* m, const DecodeArgs& a, hipStream_t s) {
    return m->cfg.weight_precision == LPP_WEIGHT_FP16 ? enqueue_token<true>(m, a, s)
                                                      : enqueue_token<false>(m, a, s);
}

// Record the token into a graph once per (model, with_arrays) and keep the
// executable; replays take no arguments because everything variable is read
// from device memory.
lpp_status token_graph(lpp_model* m, bool with_arrays, hipGraphExec_t* exec) {
    const int slot = with_arrays ? 1 : 0;
    if (m->graph_exec[slot] == nullptr) {
        hipStream_t s = stream();
        const DecodeArgs a = make_args(m, with_arrays);
        hipGraph_t graph = nullptr;
        LPP_HIP(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
        lpp_status st = enqueue_token_any(m, a, s);
        hipError_t e = hipStreamEndCapture(s, &graph);
        if (st != LPP_OK) {
            if (graph) (void)hipGraphDestroy(graph);
            return st;
        }
        if (e != hipSuccess) return fail(LPP_ERR_HIP, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
        e = hipGraphInstantiate(&m->graph_exec[slot], graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (e != hipSuccess) return fail(LPP_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    *exec = m->graph_exec[slot];
    return LPP_OK;
}

void drop_graphs(lpp_model* m) {
    for (auto& g : m->graph_exec) {
        if (g) (void)hipGraphExecDestroy(g);
        g = nullptr;
    }
}

lpp_status require_fused(const lpp_model* m) {
    if (!m->fused_ok) return fail(LPP_ERR_UNSUPPORTED, "fused decode path unavailable for this shape: %s", m->fused_why);
    if (m->path == LPP_PATH_PERSISTENT)
        return fail(LPP_ERR_UNSUPPORTED, "LPP_PATH_PERSISTENT is not built into this library");
    return LPP_OK;
}

lpp_status ensure_gen_capacity(lpp_model* m, int n_steps) {
    if (n_steps <= m->gen_cap) return LPP_OK;
    int want = m->gen_cap > 0 ? m->gen_cap : 1024;
    while (want < n_steps) want *= 2;
    LPP_HIP(hipStreamSynchronize(stream()));
    drop_graphs(m);  // the recorded kernels hold the old array addresses
    lpp_free(m->gen_uniforms);
    lpp_free(m->gen_tokens);
    m->gen_uniforms = nullptr;
    m->gen_tokens = nullptr;
    m->gen_cap = 0;
    void* p = nullptr;
    LPP_TRY(lpp_malloc(&p, static_cast<size_t>(want) * sizeof(float)));
    m->gen_uniforms = static_cast<float*>(p);
    LPP_TRY(lpp_malloc(&p, static_cast<size_t>(want) * sizeof(int)));
    m->gen_tokens = static_cast<int*>(p);
    if (m->pinned_tokens) (void)hipHostFree(m->pinned_tokens);
    m->pinned_tokens = nullptr;
    if (hipHostMalloc(reinterpret_cast<void**>(&m->pinned_tokens), static_cast<size_t>(want) * sizeof(int),
                      hipHostMallocDefault) != hipSuccess)
        return fail(LPP_ERR_OOM, "pinned token buffer allocation failed");
    m->pinned_tokens_cap = want;
    m->gen_cap = want;
    return LPP_OK;
}

}  // namespace

lpp_status fused_prepare(lpp_model* m) {
    const lpp_config& c = m->cfg;
    m->fused_ok = true;
    auto reject = [&](const char* why) {
        m->fused_ok = false;
        std::strncpy(m->fused_why, why, sizeof m->fused_why - 1);
    };
    const int per = (c.weight_precision == LPP_WEIGHT_FP16) ? 8 : 4;
    if (m->head_size % 8 != 0 || m->head_size > 128) reject("head_size must be a multiple of 8, at most 128");
    else if (m->gqa > kMaxGqa) reject("more than 8 query heads per KV head");
    else if (c.dim % per != 0 || c.hidden_dim % per != 0) reject("dim and hidden_dim must fill whole 16-byte weight loads");
    else if (c.hidden_dim > 16384 || c.dim > 16384) reject("activation vector does not fit the 64 KiB LDS stage");

    // About 64 positions per split once the context is long; at most 32 splits.
    int splits = c.seq_len / 64;
    if (splits < 1) splits = 1;
    if (splits > 32) splits = 32;
    m->max_splits = splits;

    void* p = nullptr;
    LPP_TRY(lpp_malloc(&p, sizeof(StepParams)));
    m->step = static_cast<StepParams*>(p);
    LPP_TRY(lpp_memset(m->step, 0, sizeof(StepParams)));
    if (hipHostMalloc(reinterpret_cast<void**>(&m->step_host), sizeof(StepParams), hipHostMallocDefault) != hipSuccess)
        return fail(LPP_ERR_OOM, "pinned StepParams allocation failed");
    std::memset(m->step_host, 0, sizeof(StepParams));
    const size_t partial = static_cast<size_t>(c.n_heads) * splits * (m->head_size + 2);
    LPP_TRY(lpp_malloc(&p, partial * sizeof(float)));
    m->att_partial = static_cast<float*>(p);
    LPP_TRY(lpp_malloc(&p, static_cast<size_t>(c.vocab_size) * sizeof(float)));
    m->work_logits = static_cast<float*>(p);
    LPP_TRY(lpp_malloc(&p, 256 * sizeof(unsigned)));
    m->sync_words = static_cast<unsigned*>(p);
    LPP_TRY(lpp_memset(m->sync_words, 0, 256 * sizeof(unsigned)));
    LPP_TRY(lpp_malloc(&p, 4 * smp::kMaxChunks * sizeof(float)));
    m->sample_scratch = static_cast<float*>(p);
    for (auto& e : m->ev_tok)
        if (hipEventCreate(&e) != hipSuccess) return fail(LPP_ERR_HIP, "hipEventCreate failed");
    return LPP_OK;
}

lpp_status fused_release(lpp_model* m) {
    drop_graphs(m);
    lpp_free(m->step);
    if (m->step_host) (void)hipHostFree(m->step_host);
    if (m->pinned_tokens) (void)hipHostFree(m->pinned_tokens);
    lpp_free(m->att_partial);
    lpp_free(m->work_logits);
    lpp_free(m->sync_words);
    lpp_free(m->sample_scratch);
    lpp_free(m->gen_uniforms);
    lpp_free(m->gen_tokens);
    for (auto& e : m->ev_tok)
        if (e) (void)hipEventDestroy(e);
    return LPP_OK;
}

lpp_status fused_forward(lpp_model* m, int token, int pos, float temperature, float penalty, const int* history,
                         int history_len, float r, int* next_token) {
    LPP_TRY(require_fused(m));
    hipStream_t s = stream();
    const bool use_history = penalty > 1.0f && history != nullptr && history_len > 0;
    if (use_history)
        LPP_REQUIRE(history_len <= m->cfg.seq_len, "lpp_forward: history_len %d exceeds seq_len %d", history_len,
                    m->cfg.seq_len);
    StepParams& sp = *m->step_host;
    std::memset(&sp, 0, sizeof sp);
    sp.token = token;
    sp.pos = pos;
    sp.history_len = use_history ? history_len : 0;
    sp.history_cap = 0;  // the caller owns the window (model.cpp:361-363 uploads it per call)
    sp.temperature = temperature;
    sp.penalty = penalty;
    sp.r = r;
    LPP_HIP(hipMemcpyAsync(m->step, &sp, sizeof sp, hipMemcpyHostToDevice, s));
    if (use_history)
        LPP_HIP(hipMemcpyAsync(m->history, history, static_cast<size_t>(history_len) * sizeof(int),
                               hipMemcpyHostToDevice, s));
    hipGraphExec_t exec = nullptr;
    LPP_TRY(token_graph(m, false, &exec));
    LPP_HIP(hipGraphLaunch(exec, s));
    LPP_HIP(hipMemcpyAsync(next_token, m->sampled_token, sizeof(int), hipMemcpyDeviceToHost, s));
    LPP_HIP(hipStreamSynchronize(s));
    return LPP_OK;
}

lpp_status fused_generate(lpp_model* m, int first_token, int start_pos, int n_steps, float temperature,
                          float penalty, int* history, int* history_len, int history_cap, const float* uniforms,
                          int* out_tokens, lpp_gen_stats* stats) {
    LPP_TRY(require_fused(m));
    if (n_steps == 0) return LPP_OK;
    hipStream_t s = stream();
    LPP_TRY(ensure_gen_capacity(m, n_steps));
    StepParams& sp = *m->step_host;
    std::memset(&sp, 0, sizeof sp);
    sp.token = first_token;
    sp.pos = start_pos;
    sp.history_len = *history_len;
    sp.history_cap = history_cap;
    sp.history_next = (history_cap > 0) ? (*history_len % history_cap) : 0;
    sp.temperature = temperature;
    sp.penalty = penalty;
    LPP_HIP(hipMemcpyAsync(m->step, &sp, sizeof sp, hipMemcpyHostToDevice, s));
    if (*history_len > 0)
        LPP_HIP(hipMemcpyAsync(m->history, history, static_cast<size_t>(*history_len) * sizeof(int),
                               hipMemcpyHostToDevice, s));
    if (uniforms)
        LPP_HIP(hipMemcpyAsync(m->gen_uniforms, uniforms, static_cast<size_t>(n_steps) * sizeof(float),
                               hipMemcpyHostToDevice, s));
    else
        LPP_TRY(lpp_memset(m->gen_uniforms, 0, static_cast<size_t>(n_steps) * sizeof(float)));
    hipGraphExec_t exec = nullptr;
    LPP_TRY(token_graph(m, true, &exec));
    LPP_HIP(hipStreamSynchronize(s));

    // main.cpp:196-223: one forward per token.  Token i+1 is launched before the
    // host waits for the 4 bytes of token i, so the device never idles on the host.
    LPP_HIP(hipEventRecord(m->ev_a, s));
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < n_steps; ++i) {
        LPP_HIP(hipGraphLaunch(exec, s));
        LPP_HIP(hipMemcpyAsync(m->pinned_tokens + i, m->gen_tokens + i, sizeof(int), hipMemcpyDeviceToHost, s));
        LPP_HIP(hipEventRecord(m->ev_tok[i & 1], s));
        if (i > 0) {
            LPP_HIP(hipEventSynchronize(m->ev_tok[(i - 1) & 1]));
            out_tokens[i - 1] = m->pinned_tokens[i - 1];
        }
    }
    LPP_HIP(hipEventSynchronize(m->ev_tok[(n_steps - 1) & 1]));
    out_tokens[n_steps - 1] = m->pinned_tokens[n_steps - 1];
    const auto t1 = std::chrono::steady_clock::now();
    LPP_HIP(hipEventRecord(m->ev_b, s));
    LPP_HIP(hipEventSynchronize(m->ev_b));

    // Hand the penalty window back in the reference's order (oldest first).
    LPP_HIP(hipMemcpy(&sp, m->step, sizeof sp, hipMemcpyDeviceToHost));
    if (sp.error != 0) return fail(LPP_ERR_HIP, "decode kernel reported error %d", sp.error);
    if (history_cap > 0) {
        std::vector<int> ring(static_cast<size_t>(history_cap));
        LPP_HIP(hipMemcpy(ring.data(), m->history, ring.size() * sizeof(int), hipMemcpyDeviceToHost));
        const int len = sp.history_len;
        const int oldest = (len < history_cap) ? 0 : sp.history_next;
        for (int i = 0; i < len; ++i) history[i] = ring[static_cast<size_t>((oldest + i) % history_cap)];
        *history_len = len;
    }
    if (stats) {
        float ms = 0.0f;
        LPP_HIP(hipEventElapsedTime(&ms, m->ev_a, m->ev_b));
        stats->wall_seconds = std::chrono::duration<double>(t1 - t0).count();
        stats->device_ms = ms;
        stats->tokens = n_steps;
    }
    return LPP_OK;
}

}  // namespace lpp
