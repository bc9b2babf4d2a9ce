// fused_decode.hip -- the two fast schedules of forward() (reference
// src/model.cpp:342-371) built from the phases of decode_phases.hpp:
//
//   LPP_PATH_FUSED       one launch per phase (5 per layer + classifier + sampler
//                        steps), recorded once into a HIP graph, replayed per token;
//   LPP_PATH_PERSISTENT  one kernel per token (dataflow_decode.hip); this file
//                        holds its host side: launch, generation loop, timing.
//
// All per-token scalars (token, position, penalty window, uniform draw) live in
// device memory, so the graph is not patched between tokens (the persistent
// kernel takes everything but the token id as launch arguments); the sampled id
// is fed back on the device and written straight into pinned host memory, 4
// bytes per token.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <vector>

#include "decode_phases.hpp"

// (defined with the timeline code at the end of the file)
static lpp_status calibrate_gateup(lpp_model* m);

namespace lpp {
namespace {

using namespace ph;

constexpr int kThreads = 256;            // graph path
constexpr int kWavesPerWg = kThreads / dev::kWave;
constexpr int kNoToken = -1;             // sentinel in the pinned token array

struct NoWait {
    __device__ __forceinline__ void operator()() const {}
};

// ---------------------------------------------------------------------------
// One launch per phase
// ---------------------------------------------------------------------------

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_qkv(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    phase_qkv<kF16, 2, false>(a, layer, blockIdx.x, gridDim.x, lds, NoWait{});
}

__global__ __launch_bounds__(kThreads) void k_attention(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    phase_attention<false>(a, layer, blockIdx.x, gridDim.x, lds, NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_oproj(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    const int wbytes = kF16 ? 2 : 4;
    const char* w = a.wo + static_cast<size_t>(layer) * a.dim * a.dim * wbytes;
    phase_proj_residual<kF16, 2, false>(w, a.dim, a.dim, a.xb, layer_input(a, layer), a.x, blockIdx.x, gridDim.x, lds,
                                 NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_gateup(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    phase_gateup<kF16, 2, false>(a, layer, blockIdx.x, gridDim.x, lds, NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_down(DecodeArgs a, int layer) {
    extern __shared__ __align__(16) float lds[];
    const int wbytes = kF16 ? 2 : 4;
    const char* w = a.w2 + static_cast<size_t>(layer) * a.dim * a.hidden * wbytes;
    phase_proj_residual<kF16, 1, false, 8>(w, a.dim, a.hidden, a.hb, a.x, a.x, blockIdx.x, gridDim.x, lds, NoWait{});
}

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_lmhead(DecodeArgs a) {
    extern __shared__ __align__(16) float lds[];
    phase_lmhead<kF16, 4, false>(a, blockIdx.x, gridDim.x, lds, NoWait{});
}

// Sampler steps; chunk c of the vocabulary is handled by workgroup c.
__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_scale(DecodeArgs a, int chunk) {
    sample_step_scale<false>(a, chunk, blockIdx.x);
}
__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_exp(DecodeArgs a, int chunk, int nchunks) {
    sample_step_exp<false>(a, chunk, nchunks, blockIdx.x);
}
__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_norm(DecodeArgs a, int chunk, int nchunks) {
    sample_step_norm<false>(a, chunk, nchunks, blockIdx.x);
}
__global__ __launch_bounds__(smp::kSampleThreads) void k_sample_search(DecodeArgs a, int chunk) {
    sample_step_search<false>(a, chunk, blockIdx.x);
}
__global__ void k_finish(DecodeArgs a) {
    if (threadIdx.x == 0 && blockIdx.x == 0) finish_token(a, a.sampled[0], 0u);
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

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
    a.out_tokens = with_arrays ? m->pinned_tokens_dev : nullptr;
    a.sampled = m->sampled_token;
    float* sc = m->sample_scratch;
    a.sample_scratch = smp::SampleScratch{sc, reinterpret_cast<int*>(sc + smp::kMaxChunks),
                                          sc + 2 * smp::kMaxChunks, sc + 3 * smp::kMaxChunks};
    a.trace = nullptr;
    return a;
}

int blocks_for_tiles(int ntiles) {
    int blocks = (ntiles + kWavesPerWg - 1) / kWavesPerWg;
    constexpr int per_cu = 8;
    const int cap = compute_units() * per_cu;
    if (blocks > cap) blocks = cap;
    return blocks < 1 ? 1 : blocks;
}

struct Launch {
    size_t lds_dim, lds_hidden, lds_att;
    int qkv_blocks, o_blocks, gu_blocks, down_blocks, lm_blocks, att_blocks, chunk, nchunks;
};

Launch launch_plan(const lpp_model* m) {
    const lpp_config& c = m->cfg;
    Launch p;
    p.lds_dim = static_cast<size_t>((c.dim + 7) & ~7) * 4;
    p.lds_hidden = static_cast<size_t>((c.hidden_dim + 7) & ~7) * 4;
    p.lds_att = static_cast<size_t>(attention_lds_floats(m->gqa, m->head_size, kThreads)) * 4;
    p.qkv_blocks = blocks_for_tiles((c.dim + 2 * m->kv_dim + 1) / 2);
    p.o_blocks = blocks_for_tiles((c.dim + 1) / 2);
    p.gu_blocks = blocks_for_tiles((c.hidden_dim + 1) / 2);
    p.down_blocks = blocks_for_tiles(c.dim);
    p.lm_blocks = blocks_for_tiles((c.vocab_size + 3) / 4);
    p.att_blocks = c.n_kv_heads * m->max_splits;
    p.chunk = smp::chunk_size_for(c.vocab_size);
    p.nchunks = (c.vocab_size + p.chunk - 1) / p.chunk;
    return p;
}

// Enqueue every launch of one token on `s` (graph path).
template <bool kF16>
lpp_status enqueue_token(const lpp_model* m, const DecodeArgs& a, hipStream_t s) {
    const Launch p = launch_plan(m);
    for (int layer = 0; layer < m->cfg.n_layers; ++layer) {
        hipLaunchKernelGGL((k_qkv<kF16>), dim3(p.qkv_blocks), dim3(kThreads), p.lds_dim, s, a, layer);
        hipLaunchKernelGGL(k_attention, dim3(p.att_blocks), dim3(kThreads), p.lds_att, s, a, layer);
        hipLaunchKernelGGL((k_oproj<kF16>), dim3(p.o_blocks), dim3(kThreads), p.lds_dim, s, a, layer);
        hipLaunchKernelGGL((k_gateup<kF16>), dim3(p.gu_blocks), dim3(kThreads), p.lds_dim, s, a, layer);
        hipLaunchKernelGGL((k_down<kF16>), dim3(p.down_blocks), dim3(kThreads), p.lds_hidden, s, a, layer);
    }
    hipLaunchKernelGGL((k_lmhead<kF16>), dim3(p.lm_blocks), dim3(kThreads), p.lds_dim, s, a);
    hipLaunchKernelGGL(k_sample_scale, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk);
    hipLaunchKernelGGL(k_sample_exp, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk, p.nchunks);
    hipLaunchKernelGGL(k_sample_norm, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk, p.nchunks);
    hipLaunchKernelGGL(k_sample_search, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk);
    hipLaunchKernelGGL(k_finish, dim3(1), dim3(64), 0, s, a);
    LPP_CHECK_LAUNCH("fused token");
    return LPP_OK;
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
        lpp_status st = m->cfg.weight_precision == LPP_WEIGHT_FP16 ? enqueue_token<true>(m, a, s)
                                                                     : enqueue_token<false>(m, a, s);
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

// One token on the model's current path.
lpp_status launch_token(lpp_model* m, bool with_arrays, hipStream_t s) {
    if (m->path == LPP_PATH_PERSISTENT) {
        return dataflow_launch(m, make_args(m, with_arrays), s);
    }
    hipGraphExec_t exec = nullptr;
    LPP_TRY(token_graph(m, with_arrays, &exec));
    LPP_HIP(hipGraphLaunch(exec, s));
    return LPP_OK;
}

lpp_status require_fused(const lpp_model* m) {
    if (!m->fused_ok) return fail(LPP_ERR_UNSUPPORTED, "fused decode path unavailable for this shape: %s", m->fused_why);
    return LPP_OK;
}

lpp_status ensure_gen_capacity(lpp_model* m, int n_steps) {
    if (n_steps <= m->gen_cap) return LPP_OK;
    int want = m->gen_cap > 0 ? m->gen_cap : 1024;
    while (want < n_steps) want *= 2;
    LPP_HIP(hipStreamSynchronize(stream()));
    drop_graphs(m);  // the recorded kernels hold the old array addresses
    lpp_free(m->gen_uniforms);
    m->gen_uniforms = nullptr;
    if (m->pinned_tokens) (void)hipHostFree(m->pinned_tokens);
    m->pinned_tokens = nullptr;
    m->pinned_tokens_dev = nullptr;
    m->gen_cap = 0;
    void* p = nullptr;
    LPP_TRY(lpp_malloc(&p, static_cast<size_t>(want) * sizeof(float)));
    m->gen_uniforms = static_cast<float*>(p);
    if (hipHostMalloc(reinterpret_cast<void**>(&m->pinned_tokens), static_cast<size_t>(want) * sizeof(int),
                      hipHostMallocMapped) != hipSuccess)
        return fail(LPP_ERR_OOM, "pinned token buffer allocation failed");
    LPP_HIP(hipHostGetDevicePointer(reinterpret_cast<void**>(&m->pinned_tokens_dev), m->pinned_tokens, 0));
    m->gen_cap = want;
    return LPP_OK;
}

// Wait until the kernels have delivered token i to pinned host memory.
lpp_status await_token(lpp_model* m, int i, hipStream_t s) {
    volatile int* slot = m->pinned_tokens + i;
    unsigned polls = 0;
    bool timing = false;
    std::chrono::steady_clock::time_point since;
    while (*slot == kNoToken) {
        if ((++polls & 0xfffu) != 0u) continue;
        // Nothing arrived for a while.  Once that while is far beyond a token's time, make sure the stream is still
        // making progress -- but not before: a query of a busy stream puts a marker of its own into the queue, behind
        // the launch that is already waiting there (in a kernel trace the launch after it starts 5.6 us late; two
        // queries a token cost 0.4-0.7 % of the tokens per second).
        const auto now = std::chrono::steady_clock::now();
        if (!timing) {
            timing = true;
            since = now;
            continue;
        }
        if (now - since < std::chrono::milliseconds(20)) continue;
        since = now;
        const hipError_t q = hipStreamQuery(s);
        if (q == hipSuccess) {
            if (*slot != kNoToken) break;
            return fail(LPP_ERR_HIP, "decode finished without delivering token %d", i);
        }
        if (q != hipErrorNotReady) return fail(LPP_ERR_HIP, "stream failed: %s", hipGetErrorString(q));
    }
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

    // About 256 positions per split once the context is long; at most 32 splits.
    int splits = c.seq_len / 256;
    if (splits < 1) splits = 1;
    if (splits > 32) splits = 32;
    m->max_splits = splits;
    m->spin_limit = 1u << 20;

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
    // words 0..63: attention split counters per KV head; 64: unused; 65: abort flag of the persistent kernel
    LPP_REQUIRE(c.n_kv_heads <= 64 || !m->fused_ok, "more than 64 KV heads");
    LPP_TRY(lpp_malloc(&p, 128 * sizeof(unsigned)));
    m->sync_words = static_cast<unsigned*>(p);
    LPP_TRY(lpp_memset(m->sync_words, 0, 128 * sizeof(unsigned)));
    LPP_TRY(lpp_malloc(&p, 4 * smp::kMaxChunks * sizeof(float)));
    m->sample_scratch = static_cast<float*>(p);
    LPP_TRY(lpp_malloc(&p, dataflow_tagged_bytes(m)));
    m->tagged = p;
    LPP_TRY(lpp_memset(m->tagged, 0, dataflow_tagged_bytes(m)));
    m->df_base = 0;
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
    lpp_free(m->tagged);
    for (int i = 0; i < 3; ++i) {
        lpp_free(m->df_rows[i]);
        lpp_free(m->df_gu_first[i]);
    }
    lpp_free(m->gen_uniforms);
    return LPP_OK;
}

// Bring the device-side step record (and the persistent kernel's abort flag)
// to a known start.
static lpp_status begin_run(lpp_model* m, const StepParams& init, hipStream_t s) {
    StepParams& sp = *m->step_host;
    sp = init;
    sp.epoch = 0;
    sp.error = 0;
    m->df_pos = sp.pos;
    m->df_history_len = sp.history_len;
    m->df_history_cap = sp.history_cap;
    m->df_step_index = sp.step_index;
    m->df_freeze = sp.freeze;
    m->df_temperature = sp.temperature;
    m->df_penalty = sp.penalty;
    m->df_r = sp.r;
    m->df_uniforms_host = nullptr;
    LPP_HIP(hipMemcpyAsync(m->step, &sp, sizeof sp, hipMemcpyHostToDevice, s));
    if (m->path == LPP_PATH_PERSISTENT) LPP_TRY(lpp_memset(m->sync_words + 64, 0, 2 * sizeof(unsigned)));
    return LPP_OK;
}

lpp_status fused_forward(lpp_model* m, int token, int pos, float temperature, float penalty, const int* history,
                         int history_len, float r, int* next_token) {
    LPP_TRY(require_fused(m));
    LPP_TRY(calibrate_gateup(m));
    hipStream_t s = stream();
    const bool use_history = penalty > 1.0f && history != nullptr && history_len > 0;
    if (use_history)
        LPP_REQUIRE(history_len <= m->cfg.seq_len, "lpp_forward: history_len %d exceeds seq_len %d", history_len,
                    m->cfg.seq_len);
    StepParams sp{};
    sp.token = token;
    sp.pos = pos;
    sp.history_len = use_history ? history_len : 0;
    sp.history_cap = 0;  // the caller owns the window (model.cpp:361-363 uploads it per call)
    sp.temperature = temperature;
    sp.penalty = penalty;
    sp.r = r;
    for (int attempt = 0;; ++attempt) {
        LPP_TRY(begin_run(m, sp, s));
        if (use_history)
            LPP_HIP(hipMemcpyAsync(m->history, history, static_cast<size_t>(history_len) * sizeof(int),
                                   hipMemcpyHostToDevice, s));
        LPP_TRY(launch_token(m, false, s));
        LPP_HIP(hipMemcpyAsync(next_token, m->sampled_token, sizeof(int), hipMemcpyDeviceToHost, s));
        LPP_HIP(hipStreamSynchronize(s));
        if (m->path != LPP_PATH_PERSISTENT) break;
        LPP_HIP(hipMemcpy(m->step_host, m->step, sizeof(StepParams), hipMemcpyDeviceToHost));
        if (m->step_host->error == 0) break;
        // The persistent kernel drained without a token.  Where the cause is the per-XCD numbering, that is
        // switched off and the same token launched once more (values carry sequence numbers that never repeat).
        bool relaunch = false;
        LPP_TRY(dataflow_after_error(m, m->step_host->error, &relaunch));
        if (!relaunch || attempt > 0) return fail(LPP_ERR_HIP, "decode kernel: workgroups unevenly spread over the XCDs");
    }
    return LPP_OK;
}

lpp_status fused_generate(lpp_model* m, int first_token, int start_pos, int n_steps, float temperature,
                          float penalty, int* history, int* history_len, int history_cap, const float* uniforms,
                          int* out_tokens, lpp_gen_stats* stats) {
    LPP_TRY(require_fused(m));
    if (n_steps == 0) return LPP_OK;
    LPP_TRY(calibrate_gateup(m));
    hipStream_t s = stream();
    LPP_TRY(ensure_gen_capacity(m, n_steps));
    StepParams sp{};
    sp.token = first_token;
    sp.pos = start_pos;
    sp.history_len = *history_len;
    sp.history_cap = history_cap;
    sp.history_next = (history_cap > 0) ? (*history_len % history_cap) : 0;
    sp.temperature = temperature;
    sp.penalty = penalty;
    LPP_TRY(begin_run(m, sp, s));
    if (*history_len > 0)
        LPP_HIP(hipMemcpyAsync(m->history, history, static_cast<size_t>(*history_len) * sizeof(int),
                               hipMemcpyHostToDevice, s));
    if (uniforms)
        LPP_HIP(hipMemcpyAsync(m->gen_uniforms, uniforms, static_cast<size_t>(n_steps) * sizeof(float),
                               hipMemcpyHostToDevice, s));
    else
        LPP_TRY(lpp_memset(m->gen_uniforms, 0, static_cast<size_t>(n_steps) * sizeof(float)));
    for (int i = 0; i < n_steps; ++i) m->pinned_tokens[i] = kNoToken;
    m->df_uniforms_host = uniforms;
    if (m->path != LPP_PATH_PERSISTENT) {
        hipGraphExec_t exec = nullptr;
        LPP_TRY(token_graph(m, true, &exec));  // record outside the timed loop
    }
    LPP_HIP(hipStreamSynchronize(s));

    // main.cpp:196-223: one forward per token.  The device feeds each sampled id
    // back by itself and writes it to pinned host memory; token i+1 is launched
    // before the host waits for the 4 bytes of token i, so the device never idles
    // on the host.
    LPP_HIP(hipEventRecord(m->ev_a, s));
    const auto t0 = std::chrono::steady_clock::now();
    int launched = 0;
    bool relaunched = false;
    for (int i = 0; i < n_steps; ++i) {
        while (launched < n_steps && launched <= i + 1) {
            LPP_TRY(launch_token(m, true, s));
            ++launched;
        }
        if (await_token(m, i, s) != LPP_OK) {
            // The stream went idle without token i: a persistent launch drained with an error code.  Such a launch
            // leaves the device's step record as it found it, so the record says where to pick up.
            if (m->path != LPP_PATH_PERSISTENT) return LPP_ERR_HIP;
            StepParams rec{};
            LPP_HIP(hipMemcpy(&rec, m->step, sizeof rec, hipMemcpyDeviceToHost));
            if (rec.error == 0) return LPP_ERR_HIP;  // (await_token's own message stands)
            bool again = false;
            LPP_TRY(dataflow_after_error(m, rec.error, &again));
            if (!again || relaunched || rec.step_index != i)
                return fail(LPP_ERR_HIP, "decode kernel: workgroups unevenly spread over the XCDs");
            relaunched = true;
            m->df_pos = rec.pos;
            m->df_history_len = rec.history_len;
            m->df_step_index = rec.step_index;
            launched = i;
            --i;
            continue;
        }
        out_tokens[i] = m->pinned_tokens[i];
    }
    m->df_uniforms_host = nullptr;
    const auto t1 = std::chrono::steady_clock::now();
    LPP_HIP(hipEventRecord(m->ev_b, s));
    LPP_HIP(hipEventSynchronize(m->ev_b));

    // Hand the penalty window back in the reference's order (oldest first).
    StepParams done{};
    LPP_HIP(hipMemcpy(&done, m->step, sizeof done, hipMemcpyDeviceToHost));
    if (done.error != 0) {
        bool again = false;
        LPP_TRY(dataflow_after_error(m, done.error, &again));
        return fail(LPP_ERR_HIP, "decode kernel reported error %d after the last token", done.error);
    }
    if (history_cap > 0) {
        std::vector<int> ring(static_cast<size_t>(history_cap));
        LPP_HIP(hipMemcpy(ring.data(), m->history, ring.size() * sizeof(int), hipMemcpyDeviceToHost));
        const int len = done.history_len;
        const int oldest = (len < history_cap) ? 0 : done.history_next;
        for (int i = 0; i < len; ++i) history[i] = ring[static_cast<size_t>((oldest + i) % history_cap)];
        *history_len = len;
    }
    if (stats) {
        float ms = 0.0f;
        LPP_HIP(hipEventElapsedTime(&ms, m->ev_a, m->ev_b));
        stats->wall_seconds = std::chrono::duration<double>(t1 - t0).count();
        stats->device_ms = ms;
        stats->tokens = n_steps;
        stats->kernel_launches = (m->path == LPP_PATH_PERSISTENT) ? n_steps : 0;
    }
    return LPP_OK;
}

// ---------------------------------------------------------------------------
// Per-kernel timing (lpp_profile_kernels)
// ---------------------------------------------------------------------------
namespace {

template <class EnqueueFn>
lpp_status time_class(lpp_model* m, int launches_in_graph, int reps, EnqueueFn enqueue, double* avg_ms) {
    hipStream_t s = stream();
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    LPP_HIP(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    enqueue(s);
    hipError_t e = hipStreamEndCapture(s, &graph);
    if (e != hipSuccess) return fail(LPP_ERR_HIP, "profile capture failed: %s", hipGetErrorString(e));
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) return fail(LPP_ERR_HIP, "profile instantiate failed: %s", hipGetErrorString(e));
    LPP_HIP(hipGraphLaunch(exec, s));  // warm-up
    LPP_HIP(hipStreamSynchronize(s));
    LPP_HIP(hipEventRecord(m->ev_a, s));
    for (int r = 0; r < reps; ++r) LPP_HIP(hipGraphLaunch(exec, s));
    LPP_HIP(hipEventRecord(m->ev_b, s));
    LPP_HIP(hipEventSynchronize(m->ev_b));
    float ms = 0.0f;
    LPP_HIP(hipEventElapsedTime(&ms, m->ev_a, m->ev_b));
    (void)hipGraphExecDestroy(exec);
    *avg_ms = static_cast<double>(ms) / (static_cast<double>(reps) * launches_in_graph);
    return LPP_OK;
}

template <bool kF16>
lpp_status profile_impl(lpp_model* m, int pos, int reps, lpp_kernel_time* out, int capacity, int* count) {
    const lpp_config& c = m->cfg;
    const DecodeArgs a = make_args(m, false);
    const Launch p = launch_plan(m);
    const int L = c.n_layers;
    const double wb = kF16 ? 2.0 : 4.0;
    const double dim = c.dim, hidden = c.hidden_dim, kv = m->kv_dim, vocab = c.vocab_size;
    int n = 0;
    auto add = [&](const char* name, int per_token, double ms, double bytes) {
        if (n < capacity) {
            std::snprintf(out[n].name, sizeof out[n].name, "%s", name);
            out[n].launches_per_token = per_token;
            out[n].avg_ms = ms;
            out[n].bytes_per_launch = bytes;
        }
        ++n;
    };
    // Algorithmic bytes of one token at this position (what Shape.bytes_per_token counts).
    const double token_bytes = wb * (L * (2 * dim * dim + 2 * kv * dim + 3 * hidden * dim) + vocab * dim) +
                               4 * (2 * L + 1) * dim + 4 * dim + 4.0 * kv * L * (pos + 1) + 4.0 * kv * L;
    double ms = 0.0;
    if (m->path == LPP_PATH_PERSISTENT) {
        // The whole token is one launch; a fresh step record per replay keeps pos fixed.
        hipStream_t s = stream();
        LPP_HIP(hipEventRecord(m->ev_a, s));
        for (int r = 0; r < reps; ++r) {
            LPP_TRY(dataflow_launch(m, a, s));
        }
        LPP_HIP(hipEventRecord(m->ev_b, s));
        LPP_HIP(hipEventSynchronize(m->ev_b));
        float total = 0.0f;
        LPP_HIP(hipEventElapsedTime(&total, m->ev_a, m->ev_b));
        add("k_decode_dataflow", 1, static_cast<double>(total) / reps, token_bytes);
        *count = n < capacity ? n : capacity;
        return LPP_OK;
    }
    LPP_TRY(time_class(m, L, reps, [&](hipStream_t s) {
        for (int l = 0; l < L; ++l)
            hipLaunchKernelGGL((k_qkv<kF16>), dim3(p.qkv_blocks), dim3(kThreads), p.lds_dim, s, a, l);
    }, &ms));
    add("k_qkv", L, ms, (dim + 2 * kv) * dim * wb + 8 * dim + 4 * kv);
    LPP_TRY(time_class(m, L, reps, [&](hipStream_t s) {
        for (int l = 0; l < L; ++l)
            hipLaunchKernelGGL(k_attention, dim3(p.att_blocks), dim3(kThreads), p.lds_att, s, a, l);
    }, &ms));
    add("k_attention", L, ms, 4.0 * kv * (pos + 1));
    LPP_TRY(time_class(m, L, reps, [&](hipStream_t s) {
        for (int l = 0; l < L; ++l)
            hipLaunchKernelGGL((k_oproj<kF16>), dim3(p.o_blocks), dim3(kThreads), p.lds_dim, s, a, l);
    }, &ms));
    add("k_oproj", L, ms, dim * dim * wb);
    LPP_TRY(time_class(m, L, reps, [&](hipStream_t s) {
        for (int l = 0; l < L; ++l)
            hipLaunchKernelGGL((k_gateup<kF16>), dim3(p.gu_blocks), dim3(kThreads), p.lds_dim, s, a, l);
    }, &ms));
    add("k_gateup", L, ms, 2 * hidden * dim * wb);
    LPP_TRY(time_class(m, L, reps, [&](hipStream_t s) {
        for (int l = 0; l < L; ++l)
            hipLaunchKernelGGL((k_down<kF16>), dim3(p.down_blocks), dim3(kThreads), p.lds_hidden, s, a, l);
    }, &ms));
    add("k_down", L, ms, dim * hidden * wb);
    LPP_TRY(time_class(m, 1, reps, [&](hipStream_t s) {
        hipLaunchKernelGGL((k_lmhead<kF16>), dim3(p.lm_blocks), dim3(kThreads), p.lds_dim, s, a);
    }, &ms));
    add("k_lmhead", 1, ms, vocab * dim * wb);
    LPP_TRY(time_class(m, 4, reps, [&](hipStream_t s) {
        hipLaunchKernelGGL(k_sample_scale, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk);
        hipLaunchKernelGGL(k_sample_exp, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk, p.nchunks);
        hipLaunchKernelGGL(k_sample_norm, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk, p.nchunks);
        hipLaunchKernelGGL(k_sample_search, dim3(p.nchunks), dim3(smp::kSampleThreads), 0, s, a, p.chunk);
    }, &ms));
    add("k_sample_*", 4, ms, 0.0);
    *count = n < capacity ? n : capacity;
    return LPP_OK;
}

}  // namespace
}  // namespace lpp

extern "C" lpp_status lpp_profile_kernels(lpp_model* m, int pos, int reps, lpp_kernel_time* out, int capacity,
                                          int* count) {
    using namespace lpp;
    LPP_REQUIRE(m && out && count && capacity > 0 && reps > 0, "lpp_profile_kernels: bad argument");
    LPP_REQUIRE(pos >= 0 && pos < m->cfg.seq_len, "lpp_profile_kernels: pos %d outside [0, %d)", pos, m->cfg.seq_len);
    for (int t = 0; t < LPP_T_COUNT; ++t)
        if (!m->w_loaded[t]) return fail(LPP_ERR_STATE, "weight tensor %d has not been uploaded", t);
    if (m->path == LPP_PATH_OPS) return ops_profile(m, pos, reps, out, capacity, count);
    if (!m->fused_ok) return fail(LPP_ERR_UNSUPPORTED, "fused path unavailable: %s", m->fused_why);
    LPP_TRY(calibrate_gateup(m));
    StepParams sp{};
    sp.pos = pos;
    sp.temperature = 0.8f;
    sp.penalty = 1.0f;
    sp.r = 0.5f;
    sp.freeze = 1;  // replays must not advance the position
    LPP_TRY(begin_run(m, sp, stream()));
    LPP_HIP(hipStreamSynchronize(stream()));
    return m->cfg.weight_precision == LPP_WEIGHT_FP16 ? profile_impl<true>(m, pos, reps, out, capacity, count)
                                                      : profile_impl<false>(m, pos, reps, out, capacity, count);
}

// Timeline of one token on the persistent path: for phase i, mark k is
// out[marks * i + k], in 10 ns ticks from workgroup 0's first instruction (0 where a
// mark does not apply).  The last of three replays is reported.  With all_workgroups
// the same block follows for every workgroup, one after the other.
static lpp_status trace_impl(lpp_model* m, int pos, unsigned long long* out, int capacity, int* count, int* marks_per_phase,
                             int* workgroups, bool all_workgroups) {
    using namespace lpp;
    LPP_REQUIRE(m && out && count && marks_per_phase, "lpp_trace_token: null argument");
    LPP_REQUIRE(pos >= 0 && pos < m->cfg.seq_len, "lpp_trace_token: pos %d outside [0, %d)", pos, m->cfg.seq_len);
    if (!m->fused_ok) return fail(LPP_ERR_UNSUPPORTED, "fused path unavailable: %s", m->fused_why);
    for (int t = 0; t < LPP_T_COUNT; ++t)
        if (!m->w_loaded[t]) return fail(LPP_ERR_STATE, "weight tensor %d has not been uploaded", t);
    const int marks = static_cast<int>(dataflow_trace_marks());
    const int n = marks * static_cast<int>(dataflow_phases_per_token(m->cfg.n_layers));
    const int nwg = all_workgroups ? compute_units() : 1;
    const size_t block = static_cast<size_t>(n) + 1;  // the last word of a block is the workgroup's start time
    LPP_REQUIRE(static_cast<size_t>(capacity) >= static_cast<size_t>(n) * nwg, "lpp_trace_token: capacity %d < %zu", capacity,
                static_cast<size_t>(n) * nwg);
    const int saved_path = m->path;
    m->path = LPP_PATH_PERSISTENT;
    void* p = nullptr;
    LPP_TRY(lpp_malloc(&p, block * nwg * sizeof(unsigned long long)));
    unsigned long long* d_trace = static_cast<unsigned long long*>(p);
    StepParams sp{};
    sp.pos = pos;
    sp.temperature = 0.8f;
    sp.penalty = 1.0f;
    sp.r = 0.5f;
    sp.freeze = 1;
    hipStream_t s = stream();
    lpp_status st = begin_run(m, sp, s);
    if (st == LPP_OK) st = lpp_memset(d_trace, 0, block * nwg * sizeof(unsigned long long));
    m->df_trace_stride = all_workgroups ? static_cast<int>(block) : 0;
    for (int rep = 0; rep < 3 && st == LPP_OK; ++rep) {
        DecodeArgs a = make_args(m, false);
        a.trace = d_trace;
        st = dataflow_launch(m, a, s);
    }
    m->df_trace_stride = 0;
    std::vector<unsigned long long> host(block * nwg);
    if (st == LPP_OK && hipStreamSynchronize(s) != hipSuccess) st = fail(LPP_ERR_HIP, "trace run failed");
    if (st == LPP_OK && hipMemcpy(host.data(), d_trace, host.size() * sizeof(unsigned long long),
                                  hipMemcpyDeviceToHost) != hipSuccess)
        st = fail(LPP_ERR_HIP, "trace copy failed");
    lpp_free(d_trace);
    m->path = saved_path;
    if (st != LPP_OK) return st;
    const unsigned long long t0 = host[static_cast<size_t>(n)];
    for (int w = 0; w < nwg; ++w)
        for (int i = 0; i < n; ++i) {
            const unsigned long long v = host[w * block + static_cast<size_t>(i)];
            out[static_cast<size_t>(w) * n + i] = v >= t0 ? v - t0 : 0ull;
        }
    *count = n;
    *marks_per_phase = marks;
    if (workgroups) *workgroups = nwg;
    return LPP_OK;
}

// The gate/up phase moves two thirds of a layer's bytes and ends when its slowest workgroup publishes.  How fast
// a workgroup gets through it depends on the XCD it runs on (the same XCDs finish late layer after layer, up to 2 us
// of a 31 us phase at the 8B shape) and on whether it holds an attention item.  Before a model's first token on the
// persistent path, two tokens are therefore traced at position 256 (a few hundred positions of context, whatever
// the cache holds there: what a short run sees on average) and the hidden units dealt out anew: a class of
// workgroups (those of one XCD that hold no attention item) that published d later than the median of a phase that
// took T gets 1 - d / T of its share, and so does the rest of its XCD.  Results do not change (a hidden unit's value does not depend on who forms it); the cache rows the
// traced tokens write at that position are put back.
static lpp_status calibrate_gateup(lpp_model* m) {
    using namespace lpp;
    if (m->path != LPP_PATH_PERSISTENT) return LPP_OK;
    LPP_TRY(dataflow_take_options(m, stream()));  // (a changed test option drops the calibration with the plans)
    if (m->df_calibrated) return LPP_OK;
    m->df_calibrated = true;
    if (test_option(LPP_OPT_DECODE_CALIBRATE) == 0) return LPP_OK;
    for (int t = 0; t < LPP_T_COUNT; ++t)
        if (!m->w_loaded[t]) return LPP_OK;
    const lpp_config& c = m->cfg;
    const int L = c.n_layers, hs = m->head_size, rows = L * c.n_kv_heads;
    if (L < 2) return LPP_OK;
    hipStream_t s = stream();
    // the traced position's row of every layer and KV head, as it is now
    const int at_pos = c.seq_len > 256 ? 256 : c.seq_len - 1;
    const size_t row_bytes = static_cast<size_t>(hs) * sizeof(uint16_t), pitch = static_cast<size_t>(c.seq_len) * row_bytes;
    uint16_t* k_rows = m->key_cache + static_cast<size_t>(at_pos) * hs;
    uint16_t* v_rows = m->value_cache + static_cast<size_t>(at_pos) * hs;
    std::vector<uint16_t> keep_k(static_cast<size_t>(rows) * hs), keep_v(keep_k.size());
    LPP_HIP(hipStreamSynchronize(s));
    LPP_HIP(hipMemcpy2D(keep_k.data(), row_bytes, k_rows, pitch, row_bytes, rows, hipMemcpyDeviceToHost));
    LPP_HIP(hipMemcpy2D(keep_v.data(), row_bytes, v_rows, pitch, row_bytes, rows, hipMemcpyDeviceToHost));
    const int nwg = compute_units();
    const int marks = static_cast<int>(dataflow_trace_marks());
    const int n = marks * static_cast<int>(dataflow_phases_per_token(L));
    std::vector<unsigned long long> t(static_cast<size_t>(n) * nwg);
    lpp_status st = LPP_OK;
    for (int pass = 0; pass < 2 && st == LPP_OK; ++pass) {
        int count = 0, per_phase = 0, workgroups = 0;
        st = trace_impl(m, at_pos, t.data(), static_cast<int>(t.size()), &count, &per_phase, &workgroups, true);
        if (st != LPP_OK || workgroups != nwg) break;
        int item_wgs = 0, n_xcc = 1;
        dataflow_partition_classes(m, &item_wgs, &n_xcc);
        if (n_xcc <= 1) break;  // (workgroups not numbered by XCD: nothing to tell them apart by)
        if (m->df_gu_weight.size() != static_cast<size_t>(nwg)) m->df_gu_weight.assign(nwg, 1.0f);
        const int classes = 2 * n_xcc;
        std::vector<double> late(classes, 0.0);
        std::vector<int> members(classes, 0);
        double phase_time = 0.0;
        int phases = 0;
        std::vector<double> pub(nwg), len(nwg), sorted(nwg);
        auto median = [&](const std::vector<double>& v) {
            sorted = v;
            std::nth_element(sorted.begin(), sorted.begin() + nwg / 2, sorted.end());
            return sorted[nwg / 2];
        };
        bool complete = true;
        for (int layer = 1; layer < L; ++layer) {
            const size_t at = static_cast<size_t>(marks) * (5 * layer + 3);  // the gate/up phase of the layer
            for (int w = 0; w < nwg; ++w) {
                const unsigned long long staged = t[static_cast<size_t>(w) * n + at + 2], published = t[static_cast<size_t>(w) * n + at + 4];
                complete = complete && staged != 0 && published >= staged;
                pub[w] = static_cast<double>(published);
                len[w] = static_cast<double>(published) - static_cast<double>(staged);
            }
            const double mid = median(pub);
            phase_time += median(len);
            ++phases;
            for (int w = 0; w < nwg; ++w) {
                const int cls = (w % n_xcc) + (w < item_wgs ? n_xcc : 0);
                late[cls] += pub[w] - mid;
                if (layer == 1) members[cls] += 1;
            }
        }
        if (!complete || phases == 0 || phase_time <= 0.0) break;
        phase_time /= phases;
        // class means; the classes of the item holders are folded into one factor on top of their XCD's
        std::vector<double> factor(classes, 1.0);
        for (int k = 0; k < classes; ++k)
            if (members[k] > 0) {
                const double d = late[k] / (static_cast<double>(members[k]) * phases);
                double f = 1.0 - d / phase_time;
                f = f < 0.85 ? 0.85 : (f > 1.15 ? 1.15 : f);
                factor[k] = f;
            }
        // (The workgroups that hold a short context's attention items publish early or late as a class too -- 1.6 us
        // early at the TinyLlama shape -- but shifting units to or from them made every shape tried slower: their
        // lead is spent on the next layer's items.  Only the XCDs' factors are applied.)
        if (n_xcc > 1)
            for (int w = 0; w < nwg; ++w) m->df_gu_weight[w] *= static_cast<float>(factor[w % n_xcc]);
        st = dataflow_forget_lists(m, s);
    }
    LPP_HIP(hipStreamSynchronize(s));
    LPP_HIP(hipMemcpy2D(k_rows, pitch, keep_k.data(), row_bytes, row_bytes, rows, hipMemcpyHostToDevice));
    LPP_HIP(hipMemcpy2D(v_rows, pitch, keep_v.data(), row_bytes, row_bytes, rows, hipMemcpyHostToDevice));
    return st;
}

extern "C" lpp_status lpp_trace_token(lpp_model* m, int pos, unsigned long long* out, int capacity, int* count,
                                      int* marks_per_phase) {
    if (m != nullptr && m->fused_ok) {  // (the timeline is that of the partition the decode loop runs with)
        const int saved_path = m->path;
        m->path = LPP_PATH_PERSISTENT;
        const lpp_status st = calibrate_gateup(m);
        m->path = saved_path;
        LPP_TRY(st);
    }
    return trace_impl(m, pos, out, capacity, count, marks_per_phase, nullptr, false);
}

extern "C" lpp_status lpp_trace_token_all(lpp_model* m, int pos, unsigned long long* out, int capacity, int* count,
                                          int* marks_per_phase, int* workgroups) {
    LPP_REQUIRE(workgroups != nullptr, "lpp_trace_token_all: null argument");
    if (m != nullptr && m->fused_ok) {
        const int saved_path = m->path;
        m->path = LPP_PATH_PERSISTENT;
        const lpp_status st = calibrate_gateup(m);
        m->path = saved_path;
        LPP_TRY(st);
    }
    return trace_impl(m, pos, out, capacity, count, marks_per_phase, workgroups, true);
}
