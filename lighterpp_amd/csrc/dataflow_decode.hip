// dataflow_decode.hip -- LPP_PATH_PERSISTENT: one kernel per token, no grid
// barrier.  The phases of forward() (reference src/model.cpp:342-371; see
// decode_phases.hpp for the split) are chained by the data itself: every value
// one phase hands to the next is published as ONE 8-byte device-scope store
// holding the fp32 value and a 32-bit sequence number, and a consumer simply
// polls the values it needs until their sequence number is the one it expects.
//
// Why: on this part a counter barrier across 256 workgroups costs ~3.7 us and
// the staging read behind it another memory round trip, five times per layer;
// with tagged values the hand-over is one round trip (the poll that sees the
// tag has the data in hand), and nothing waits for workgroups it does not
// depend on.  Weights never depend on activations: each phase requests its
// first weight tiles before it starts polling.
//
// Sequence numbers grow monotonically for the life of a model (the host hands
// every launch its base and advances it by the number of phases), so a stale
// value, even one left by a launch that gave up, is never taken for a fresh one.  Buffer reuse is safe without further synchronisation:
// every buffer is consumed one phase after it is produced and rewritten no
// sooner than two phases later, and each phase's inputs transitively require
// every workgroup to have finished reading the phase before the previous one.
// Polls are bounded: a workgroup that gives up raises a shared abort flag that
// ends every other poll, so the grid always drains.
#include <cstring>

#include "decode_phases.hpp"

namespace lpp {
namespace df {

using namespace ph;
using namespace dev;

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
constexpr int kPollBatch = 16;  // tagged values one thread requests before checking any

typedef unsigned long long u64;

__device__ __forceinline__ u64 pack(float v, unsigned tag) {
    return (static_cast<u64>(tag) << 32) | static_cast<u64>(__float_as_uint(v));
}
__device__ __forceinline__ float value_of(u64 u) { return __uint_as_float(static_cast<unsigned>(u)); }
__device__ __forceinline__ unsigned tag_of(u64 u) { return static_cast<unsigned>(u >> 32); }
__device__ __forceinline__ void publish(u64* slot, float v, unsigned tag) {
    __hip_atomic_store(slot, pack(v, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 peek(const u64* slot) {
    return __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Tagged vectors of one model, all in one device allocation.
struct Tagged {
    u64* x;      // [dim]     residual stream, written by the O and down projections
    u64* q;      // [dim]
    u64* k;      // [kv_dim]
    u64* v;      // [kv_dim]
    u64* xb;     // [dim]     attention output
    u64* hb;     // [hidden]  SwiGLU output
    u64* part;   // [n_heads][max_splits][head_size + 2] attention split partials
    u64* stats;  // [nwg][4]  per-workgroup sampler statistics (max, sum, argmax)
    unsigned base;    // sequence-number base of this launch, advanced by the host once per token
    unsigned* abort;  // raised by a workgroup whose poll ran out of patience
    unsigned spin_limit;
};

struct Ctx {
    const DecodeArgs& a;
    const Tagged& t;
    unsigned base;  // sequence-number base of this token
    unsigned long long* trace;
    unsigned phase_index;
    // Step parameters as they stood when the kernel started.  The workgroup that
    // finishes the token rewrites them while slower workgroups are still in the
    // sampler, so nothing reads them from memory after the first phase began.
    int token, pos, history_len;
    float temperature, penalty, r;

    __device__ __forceinline__ unsigned seq(int layer, int phase) const {
        return base + 1u + 5u * static_cast<unsigned>(layer) + static_cast<unsigned>(phase);
    }
    __device__ __forceinline__ unsigned seq_stats() const { return base + 1u + 5u * static_cast<unsigned>(a.n_layers); }
    __device__ __forceinline__ void mark(int which) {
        if (trace && threadIdx.x == 0) trace[2u * phase_index + which] = wall_clock64();
    }
};

__host__ __device__ inline unsigned phases_per_token(int n_layers) { return 5u * n_layers + 2u; }
enum { kQkv = 0, kAtt = 1, kOproj = 2, kGateUp = 3, kDown = 4 };

// Fetch n tagged values carrying sequence number `want` and hand each to
// sink(i, value).  A thread requests up to kPollBatch values, then re-requests
// only those that were not there yet.
template <class Sink>
__device__ __forceinline__ void poll_values(const u64* src, int n, unsigned want, const Ctx& c, Sink sink) {
    const int nthreads = static_cast<int>(blockDim.x);
    for (int first = static_cast<int>(threadIdx.x); first < n; first += nthreads * kPollBatch) {
        u64 got[kPollBatch];
        unsigned pending = 0u;
#pragma unroll
        for (int j = 0; j < kPollBatch; ++j) {
            const int i = first + j * nthreads;
            if (i < n) {
                got[j] = peek(src + i);
                pending |= 1u << j;
            }
        }
        unsigned spins = 0;
        while (true) {
#pragma unroll
            for (int j = 0; j < kPollBatch; ++j)
                if ((pending >> j) & 1u)
                    if (tag_of(got[j]) == want) pending &= ~(1u << j);
            if (pending == 0u) break;
            if ((spins & 63u) == 63u && __hip_atomic_load(c.t.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) break;
            if (++spins > c.t.spin_limit) {
                __hip_atomic_store(c.t.abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                c.a.step->error = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
#pragma unroll
            for (int j = 0; j < kPollBatch; ++j)
                if ((pending >> j) & 1u) got[j] = peek(src + first + j * nthreads);
        }
#pragma unroll
        for (int j = 0; j < kPollBatch; ++j) {
            const int i = first + j * nthreads;
            if (i < n) sink(i, value_of(got[j]));
        }
    }
}

// xs = the tagged vector itself, zero padded to a multiple of 8.  The leading
// block barrier keeps xs intact until every wavefront has left the phase that
// was reading it.
__device__ __forceinline__ void stage_tagged(float* xs, const u64* src, int n, unsigned want, const Ctx& c) {
    const int n_pad = (n + 7) & ~7;
    __syncthreads();
    for (int i = n + threadIdx.x; i < n_pad; i += blockDim.x) xs[i] = 0.0f;
    poll_values(src, n, want, c, [&](int i, float v) { xs[i] = v; });
    __syncthreads();
}

// xraw = the input vector (tagged x, or the embedding row for layer 0);
// xs = rmsnorm(xraw) * gain, ops.cpp:20-32.
__device__ __forceinline__ void stage_norm(float* xraw, float* xs, const u64* tagged_x, const float* plain_x, int n,
                                           unsigned want, const float* gain, const Ctx& c) {
#pragma clang fp contract(off)
    __shared__ float scratch[16];
    if (plain_x != nullptr) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) xraw[i] = plain_x[i];
    } else {
        poll_values(tagged_x, n, want, c, [&](int i, float v) { xraw[i] = v; });
    }
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {  // same index set this thread wrote
        const float v = xraw[i];
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    ss /= static_cast<float>(n);
    ss += 1e-5f;
    const float scale = 1.0f / sqrtf(ss);
    const int n_pad = (n + 7) & ~7;
    for (int i = threadIdx.x; i < n_pad; i += blockDim.x) xs[i] = (i < n) ? xraw[i] * scale * gain[i] : 0.0f;
    __syncthreads();
}

struct Lds {
    float* xraw;    // [dim_pad]   residual stream as last received
    float* xs;      // [max(dim, hidden)_pad]  staged GEMV input; attention scratch overlays it
    float* local;   // [rows per workgroup of the classifier, padded]
};

// ---------------------------------------------------------------------------
// GEMV phases
// ---------------------------------------------------------------------------

template <bool kF16>
__device__ __forceinline__ void df_qkv(Ctx& c, const Lds& l, int layer, int wg, int nwg) {
#pragma clang fp contract(off)
    constexpr int kRows = 2;
    const DecodeArgs& a = c.a;
    const int wbytes = kF16 ? 2 : 4;
    const int dim = a.dim, kv_dim = a.kv_dim, total_rows = a.dim + 2 * a.kv_dim;
    const int ntiles = (total_rows + kRows - 1) / kRows;
    auto row_ptr = [&](int tile, int r) -> const char* {
        const int g = tile * kRows + r;
        if (g < dim) return row_at(a.wq, dim, layer, g, dim, wbytes);
        if (g < dim + kv_dim) return row_at(a.wk, kv_dim, layer, g - dim, dim, wbytes);
        const int gv = (g < total_rows ? g : total_rows - 1) - dim - kv_dim;
        return row_at(a.wv, kv_dim, layer, gv, dim, wbytes);
    };
    auto pre = [&]() {
        const float* emb_row = (layer == 0) ? a.emb + static_cast<size_t>(c.token) * dim : nullptr;
        stage_norm(l.xraw, l.xs, c.t.x, emb_row, dim, layer == 0 ? 0u : c.seq(layer - 1, kDown),
                   a.rms_att + static_cast<size_t>(layer) * dim, c);
        c.mark(0);
    };
    const int pos = c.pos;
    const int hs = a.head_size;
    const float2* cs_row = a.rope + static_cast<size_t>(pos) * (hs / 2);
    const unsigned tag = c.seq(layer, kQkv);
    auto emit = [&](int tile, int r, float mine, float neighbour) {
        const int g = tile * kRows + r;
        if (g >= total_rows) return;
        float out = mine;
        if (g < dim + kv_dim) {  // ops.cpp:36-52 on the pair (i, i+1)
            const int gi = (g < dim) ? g : g - dim;
            const float2 cs = cs_row[((gi & ~1) % hs) >> 1];
            out = (gi & 1) ? neighbour * cs.y + mine * cs.x : mine * cs.x - neighbour * cs.y;
        }
        if (g < dim) {
            publish(c.t.q + g, out, tag);
            a.q[g] = out;
        } else {  // model.cpp:171-176 / scatter_kv.cu:15-18
            const bool is_k = g < dim + kv_dim;
            const int i = is_k ? g - dim : g - dim - kv_dim;
            const int head = i / hs, within = i - head * hs;
            const size_t dst = static_cast<size_t>(layer) * kv_dim * a.seq_len +
                               static_cast<size_t>(head) * a.seq_len * hs + static_cast<size_t>(pos) * hs + within;
            publish((is_k ? c.t.k : c.t.v) + i, out, tag);
            (is_k ? a.k : a.v)[i] = out;
            (is_k ? a.key_cache : a.value_cache)[dst] = f32_to_f16_bits(out);
        }
    };
    gemv_phase<kF16, kRows, 4>(ntiles, dim, l.xs, wg * kWaves + wave_index(), nwg * kWaves, row_ptr, emit, pre);
    c.mark(1);
    ++c.phase_index;
}

// out = W . src + xraw (model.cpp:160,218 and :225-226); the result is the new x.
template <bool kF16, int kRows, int kUnroll>
__device__ __forceinline__ void df_proj(Ctx& c, const Lds& l, const char* w_layer, int n, int d, const u64* src,
                                        unsigned src_tag, unsigned out_tag, int wg, int nwg) {
    const int wbytes = kF16 ? 2 : 4;
    const int ntiles = (n + kRows - 1) / kRows;
    auto row_ptr = [&](int tile, int r) -> const char* {
        const int g = tile * kRows + r;
        return w_layer + static_cast<size_t>(g < n ? g : n - 1) * d * wbytes;
    };
    auto pre = [&]() {
        stage_tagged(l.xs, src, d, src_tag, c);
        c.mark(0);
    };
    auto emit = [&](int tile, int r, float mine, float) {
        const int g = tile * kRows + r;
        if (g < n) publish(c.t.x + g, l.xraw[g] + mine, out_tag);
    };
    gemv_phase<kF16, kRows, kUnroll>(ntiles, d, l.xs, wg * kWaves + wave_index(), nwg * kWaves, row_ptr, emit, pre);
    c.mark(1);
    ++c.phase_index;
}

template <bool kF16>
__device__ __forceinline__ void df_gateup(Ctx& c, const Lds& l, int layer, int wg, int nwg) {
#pragma clang fp contract(off)
    constexpr int kRows = 2;  // row 0 = gate row j, row 1 = up row j
    const DecodeArgs& a = c.a;
    const int wbytes = kF16 ? 2 : 4;
    const int hidden = a.hidden, dim = a.dim;
    auto row_ptr = [&](int tile, int r) -> const char* {
        return row_at(r ? a.w3 : a.w1, hidden, layer, tile < hidden ? tile : hidden - 1, dim, wbytes);
    };
    auto pre = [&]() {
        stage_norm(l.xraw, l.xs, c.t.x, nullptr, dim, c.seq(layer, kOproj), a.rms_ffn + static_cast<size_t>(layer) * dim, c);
        c.mark(0);
    };
    const unsigned tag = c.seq(layer, kGateUp);
    auto emit = [&](int tile, int r, float gate, float up) {
        if (r != 0 || tile >= hidden) return;
        const float sigma = 1.0f / (1.0f + expf(-gate));  // ops.cpp:80-85
        publish(c.t.hb + tile, (gate * sigma) * up, tag);
    };
    gemv_phase<kF16, kRows, 4>(hidden, dim, l.xs, wg * kWaves + wave_index(), nwg * kWaves, row_ptr, emit, pre);
    c.mark(1);
    ++c.phase_index;
}

// ---------------------------------------------------------------------------
// Attention
// ---------------------------------------------------------------------------

// One work item (KV head, context split); same arithmetic as ph::attention_item.
// K rows of positions before the current one are requested before q is polled;
// the current position's k and v arrive tagged and are rounded to binary16
// exactly as the cache store rounds them.
template <int kGroup>
__device__ __forceinline__ void df_attention_item(Ctx& c, int layer, int kvh, int split, int nsplits, int npos,
                                                  float* lds) {
    const DecodeArgs& a = c.a;
    const int hs = a.head_size, gqa = a.gqa;
    constexpr int hs_pad = kGroup * 8;
    const int nthreads = static_cast<int>(blockDim.x);
    const int nwaves = nthreads / kWave;
    const int ngroups = nthreads / kGroup;
    const int tid = static_cast<int>(threadIdx.x);
    const int sub = tid % kGroup, grp = tid / kGroup;
    const int wave = tid / kWave;
    const bool lane_live = sub * 8 < hs;

    float* qs = lds;                          // [gqa][hs_pad]
    float* sc = qs + gqa * hs_pad;            // [gqa][kAttBlock]
    float* run_max = sc + gqa * kAttBlock;    // [gqa]
    float* run_sum = run_max + gqa;           // [gqa]
    float* corr = run_sum + gqa;              // [gqa]
    float* red = corr + gqa;                  // [nwaves][gqa][hs_pad]
    float* kv_now = red + nwaves * gqa * hs_pad;  // [2][hs_pad] current position's k and v

    const int chunk = (npos + nsplits - 1) / nsplits;
    const int t_begin = split * chunk;
    const int t_end = min(npos, t_begin + chunk);
    const int current = npos - 1;
    const bool has_current = current >= t_begin && current < t_end;
    const size_t head_base = (static_cast<size_t>(layer) * a.n_kv_heads + kvh) * a.seq_len * hs;
    const uint16_t* kbase = a.key_cache + head_base;
    const uint16_t* vbase = a.value_cache + head_base;

    constexpr int kMaxPerGroup = 8;
    int per_group = kAttBlock / ngroups;
    if (per_group > kMaxPerGroup) per_group = kMaxPerGroup;
    if (per_group < 1) per_group = 1;
    const int sub_block = per_group * ngroups;

    // first sub-block's K rows: independent of this token except the current position
    uintx4 rows8[kMaxPerGroup];
#pragma unroll
    for (int j = 0; j < kMaxPerGroup; ++j) {
        const int t = t_begin + grp + j * ngroups;
        rows8[j] = uintx4{0u, 0u, 0u, 0u};
        if (j < per_group && t < min(t_end, t_begin + sub_block) && t != current && lane_live)
            rows8[j] = load16(kbase + static_cast<size_t>(t) * hs + sub * 8);
    }

    // inputs of this token (the block barrier: no wavefront still reads this LDS
    // area as the activation vector of the previous phase)
    const unsigned tag_in = c.seq(layer, kQkv);
    __syncthreads();
    if (hs == hs_pad) {
        poll_values(c.t.q + static_cast<size_t>(kvh) * gqa * hs, gqa * hs, tag_in, c, [&](int i, float v) { qs[i] = v; });
    } else {
        for (int i = tid; i < gqa * hs_pad; i += nthreads) qs[i] = 0.0f;
        __syncthreads();
        poll_values(c.t.q + static_cast<size_t>(kvh) * gqa * hs, gqa * hs, tag_in, c,
                    [&](int i, float v) { qs[(i / hs) * hs_pad + (i % hs)] = v; });
    }
    if (has_current) {
        for (int i = tid; i < 2 * hs_pad; i += nthreads) kv_now[i] = 0.0f;
        __syncthreads();
        poll_values(c.t.k + static_cast<size_t>(kvh) * hs, hs, tag_in, c,
                    [&](int i, float v) { kv_now[i] = f16_bits_to_f32(f32_to_f16_bits(v)); });
        poll_values(c.t.v + static_cast<size_t>(kvh) * hs, hs, tag_in, c,
                    [&](int i, float v) { kv_now[hs_pad + i] = f16_bits_to_f32(f32_to_f16_bits(v)); });
    }
    if (tid < gqa) {
        run_max[tid] = -INFINITY;
        run_sum[tid] = 0.0f;
    }
    __syncthreads();
    c.mark(0);

    // a cache row as 8 fp32 values per lane; the current position comes from LDS
    auto row_values = [&](uintx4 bits, const float* now, bool is_current, float (&out)[8]) {
        const half8_t h = as_half8(bits);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = is_current ? now[sub * 8 + e] : static_cast<float>(h[e]);
    };

    const float scale = 1.0f / sqrtf(static_cast<float>(hs));  // model.cpp:188
    float acc[kMaxGqa][8];
#pragma unroll
    for (int qh = 0; qh < kMaxGqa; ++qh)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[qh][e] = 0.0f;

    for (int b0 = t_begin; b0 < t_end; b0 += sub_block) {
        const int b1 = min(t_end, b0 + sub_block);
        if (b0 != t_begin) {
#pragma unroll
            for (int j = 0; j < kMaxPerGroup; ++j) {
                const int t = b0 + grp + j * ngroups;
                rows8[j] = uintx4{0u, 0u, 0u, 0u};
                if (j < per_group && t < b1 && t != current && lane_live)
                    rows8[j] = load16(kbase + static_cast<size_t>(t) * hs + sub * 8);
            }
        }
#pragma unroll
        for (int j = 0; j < kMaxPerGroup; ++j) {
            const int t = b0 + grp + j * ngroups;
            float kf[8];
            row_values(rows8[j], kv_now, t == current, kf);
#pragma unroll
            for (int qh = 0; qh < kMaxGqa; ++qh) {
                if (qh < gqa) {
                    const float* qv = qs + qh * hs_pad + sub * 8;
                    float s = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) s = fmaf(kf[e], qv[e], s);
                    s = group_sum<kGroup>(s);
                    if (j < per_group && t < b1 && sub == 0) sc[qh * kAttBlock + (t - b0)] = s * scale;
                }
            }
        }
        // V rows travel while the softmax is formed
#pragma unroll
        for (int j = 0; j < kMaxPerGroup; ++j) {
            const int t = b0 + grp + j * ngroups;
            rows8[j] = uintx4{0u, 0u, 0u, 0u};
            if (j < per_group && t < b1 && t != current && lane_live)
                rows8[j] = load16(vbase + static_cast<size_t>(t) * hs + sub * 8);
        }
        __syncthreads();
        for (int qh = wave; qh < gqa; qh += nwaves) {
            float* row = sc + qh * kAttBlock;
            const int n = b1 - b0;
            float m = -INFINITY;
            for (int i = lane_id(); i < n; i += kWave) m = fmaxf(m, row[i]);
            m = wave_max(m);
            const float m_old = run_max[qh];
            const float m_new = fmaxf(m_old, m);
            float lsum = 0.0f;
            for (int i = lane_id(); i < n; i += kWave) {
                const float p = expf(row[i] - m_new);
                row[i] = p;
                lsum += p;
            }
            lsum = wave_sum(lsum);
            if (lane_id() == 0) {
                const float cf = (m_old == -INFINITY) ? 0.0f : expf(m_old - m_new);
                corr[qh] = cf;
                run_sum[qh] = run_sum[qh] * cf + lsum;
                run_max[qh] = m_new;
            }
        }
        __syncthreads();
#pragma unroll
        for (int qh = 0; qh < kMaxGqa; ++qh) {
            if (qh < gqa) {
                const float cf = corr[qh];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[qh][e] *= cf;
            }
        }
#pragma unroll
        for (int j = 0; j < kMaxPerGroup; ++j) {
            const int t = b0 + grp + j * ngroups;
            if (j < per_group && t < b1 && lane_live) {
                float vf[8];
                row_values(rows8[j], kv_now + hs_pad, t == current, vf);
#pragma unroll
                for (int qh = 0; qh < kMaxGqa; ++qh) {
                    if (qh < gqa) {
                        const float p = sc[qh * kAttBlock + (t - b0)];
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc[qh][e] = fmaf(vf[e], p, acc[qh][e]);
                    }
                }
            }
        }
        __syncthreads();
    }

    // per-group partial outputs -> wavefront (lane exchange) -> workgroup (LDS, wave order)
#pragma unroll
    for (int qh = 0; qh < kMaxGqa; ++qh) {
        if (qh < gqa) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float v = acc[qh][e];
#pragma unroll
                for (int off = kGroup; off < kWave; off <<= 1) v += __shfl_xor(v, off);
                acc[qh][e] = v;
            }
            if (lane_id() < kGroup) {
#pragma unroll
                for (int e = 0; e < 8; ++e) red[(wave * gqa + qh) * hs_pad + sub * 8 + e] = acc[qh][e];
            }
        }
    }
    __syncthreads();
    const unsigned tag_out = c.seq(layer, kAtt);
    const int stride = hs + 2;
    if (nsplits == 1) {
        for (int i = tid; i < gqa * hs; i += nthreads) {
            const int qh = i / hs, e = i - qh * hs;
            float o = 0.0f;
            for (int w = 0; w < nwaves; ++w) o += red[(w * gqa + qh) * hs_pad + e];
            publish(c.t.xb + static_cast<size_t>(kvh * gqa + qh) * hs + e, o / run_sum[qh], tag_out);
        }
        return;
    }
    for (int i = tid; i < gqa * hs; i += nthreads) {
        const int qh = i / hs, e = i - qh * hs;
        float o = 0.0f;
        for (int w = 0; w < nwaves; ++w) o += red[(w * gqa + qh) * hs_pad + e];
        u64* part = c.t.part + (static_cast<size_t>(kvh * gqa + qh) * a.max_splits + split) * stride;
        publish(part + e, o, tag_out);
        if (e == 0) {
            publish(part + hs, run_max[qh], tag_out);
            publish(part + hs + 1, run_sum[qh], tag_out);
        }
    }
}

// Combine the context splits of one KV head: collect every split's (output,
// max, sum), rescale to the common maximum and normalise.  Runs after the
// workgroup has published all of its own partials, so a workgroup waiting here
// never holds back a partial another combiner needs.
__device__ __forceinline__ void df_attention_combine(Ctx& c, int layer, int kvh, int nsplits, float* gathered) {
    const DecodeArgs& a = c.a;
    const int hs = a.head_size, gqa = a.gqa;
    const int stride = hs + 2;
    const int tid = static_cast<int>(threadIdx.x), nthreads = static_cast<int>(blockDim.x);
    const unsigned tag_out = c.seq(layer, kAtt);
    __syncthreads();
    for (int qh = 0; qh < gqa; ++qh) {  // gathered: [gqa][max_splits][stride]
        const size_t first = static_cast<size_t>(kvh * gqa + qh) * a.max_splits * stride;
        float* dst = gathered + static_cast<size_t>(qh) * a.max_splits * stride;
        poll_values(c.t.part + first, nsplits * stride, tag_out, c, [&](int i, float v) { dst[i] = v; });
    }
    __syncthreads();
    for (int i = tid; i < gqa * hs; i += nthreads) {
        const int qh = i / hs, e = i - qh * hs;
        const float* basep = gathered + static_cast<size_t>(qh) * a.max_splits * stride;
        float top = -INFINITY;
        for (int s = 0; s < nsplits; ++s) top = fmaxf(top, basep[s * stride + hs]);
        float o = 0.0f, lsum = 0.0f;
        for (int s = 0; s < nsplits; ++s) {
            const float ms = basep[s * stride + hs];
            const float wgt = (ms == -INFINITY) ? 0.0f : expf(ms - top);
            o += basep[s * stride + e] * wgt;
            lsum += basep[s * stride + hs + 1] * wgt;
        }
        publish(c.t.xb + static_cast<size_t>(kvh * gqa + qh) * hs + e, o / lsum, tag_out);
    }
}

__device__ __forceinline__ void df_attention(Ctx& c, const Lds& l, int layer, int wg, int nwg) {
    const DecodeArgs& a = c.a;
    const int npos = c.pos + 1;
    const int nsplits = active_splits(npos, a.max_splits);
    const int items = a.n_kv_heads * nsplits;
    const int hs = a.head_size;
    bool marked = false;
    for (int item = wg; item < items; item += nwg) {
        const int kvh = item / nsplits, split = item - kvh * nsplits;
        if (hs <= 8) df_attention_item<1>(c, layer, kvh, split, nsplits, npos, l.xs);
        else if (hs <= 16) df_attention_item<2>(c, layer, kvh, split, nsplits, npos, l.xs);
        else if (hs <= 32) df_attention_item<4>(c, layer, kvh, split, nsplits, npos, l.xs);
        else if (hs <= 64) df_attention_item<8>(c, layer, kvh, split, nsplits, npos, l.xs);
        else df_attention_item<16>(c, layer, kvh, split, nsplits, npos, l.xs);
        __syncthreads();
        marked = true;
    }
    if (nsplits > 1) {
        for (int item = wg; item < items; item += nwg) {
            const int kvh = item / nsplits, split = item - kvh * nsplits;
            if (split == 0) df_attention_combine(c, layer, kvh, nsplits, l.xs);
        }
    }
    if (!marked) c.mark(0);
    c.mark(1);
    ++c.phase_index;
}

// ---------------------------------------------------------------------------
// Classifier + sampler
// ---------------------------------------------------------------------------

// Workgroup w owns the contiguous vocabulary rows [w*rows_per_wg, ...): their
// logits stay in LDS, the sampler's per-row work happens there, and only three
// numbers per workgroup (maximum, its lowest index, sum of exponentials) are
// exchanged.  The workgroup whose slice of the CDF contains the draw (or that
// holds the first maximum, for temperature 0) finishes the token
// (model.cpp:256-303, main.cpp:200-208).
template <bool kF16>
__device__ __forceinline__ void df_classify_sample(Ctx& c, const Lds& l, int wg, int nwg, int rows_per_wg) {
    constexpr int kRows = 2;
    const DecodeArgs& a = c.a;
    const int wbytes = kF16 ? 2 : 4;
    const int vocab = a.vocab, dim = a.dim;
    const int r0 = min(vocab, wg * rows_per_wg), r1 = min(vocab, r0 + rows_per_wg);
    const int n = r1 - r0;
    const int ntiles = (n + kRows - 1) / kRows;
    const int tid = static_cast<int>(threadIdx.x), nthreads = static_cast<int>(blockDim.x);
    float* lg = l.local;
    auto row_ptr = [&](int tile, int r) -> const char* {
        int g = r0 + tile * kRows + r;
        if (g >= vocab) g = vocab - 1;
        return a.wcls + static_cast<size_t>(g) * dim * wbytes;
    };
    auto pre = [&]() {
        stage_norm(l.xraw, l.xs, c.t.x, nullptr, dim, c.seq(a.n_layers - 1, kDown), a.rms_final, c);
        c.mark(0);
    };
    auto emit = [&](int tile, int r, float mine, float) {
        const int i = tile * kRows + r;
        if (i < n) {
            lg[i] = mine;
            a.logits[r0 + i] = mine;  // raw logits stay readable after the token
        }
    };
    gemv_phase<kF16, kRows, 4>(ntiles, dim, l.xs, wave_index(), kWaves, row_ptr, emit, pre);
    __syncthreads();
    c.mark(1);
    ++c.phase_index;

    // ---- sampler on the local rows ----
    __shared__ float s_val[16];
    __shared__ int s_idx[16];
    __shared__ float s_scratch[16];
    __shared__ int s_target, s_token;
    const float temperature = c.temperature, penalty = c.penalty;
    const int history_len = c.history_len;
    if (penalty > 1.0f && history_len > 0) {  // model.cpp:258-270, once per occurrence
        for (int i = tid; i < history_len; i += nthreads) {
            const int tok = a.history[i];
            if (tok < r0 || tok >= r1) continue;
            const int count = smp::owned_count(a.history, history_len, i);
            if (count > 0) lg[tok - r0] = smp::penalise(lg[tok - r0], penalty, count);
        }
        __syncthreads();
    }
    ArgMax best{-INFINITY, 0x7fffffff};
    for (int i = tid; i < n; i += nthreads) {
        float v = lg[i];
        if (temperature != 0.0f) v = v / temperature;  // model.cpp:286-288
        lg[i] = v;
        best = argmax_better(best, ArgMax{v, r0 + i});
    }
    best = wave_argmax(best);
    if (lane_id() == 0) {
        s_val[tid / kWave] = best.v;
        s_idx[tid / kWave] = best.i;
    }
    __syncthreads();
    ArgMax mine{s_val[0], s_idx[0]};
    for (int w = 1; w < kWaves; ++w) mine = argmax_better(mine, ArgMax{s_val[w], s_idx[w]});
    float local_sum = 0.0f;
    if (temperature != 0.0f) {
        float part = 0.0f;
        for (int i = tid; i < n; i += nthreads) {
            const float e = expf(lg[i] - mine.v);  // ops.cpp:65, against the local maximum
            lg[i] = e;
            part += e;
        }
        local_sum = block_sum(part, s_scratch);
    }
    const unsigned tag = c.seq_stats();
    if (tid == 0) {
        publish(c.t.stats + wg * 4 + 0, mine.v, tag);
        publish(c.t.stats + wg * 4 + 1, local_sum, tag);
        publish(c.t.stats + wg * 4 + 2, __int_as_float(mine.i), tag);
        publish(c.t.stats + wg * 4 + 3, 0.0f, tag);
    }
    // every workgroup reads all statistics and reaches the same decision
    float* st_max = l.xs;            // [nwg]
    float* st_sum = l.xs + nwg;      // [nwg]
    float* st_arg = l.xs + 2 * nwg;  // [nwg] (int bits)
    float* st_cum = l.xs + 3 * nwg;  // [nwg] inclusive mass
    __syncthreads();
    poll_values(c.t.stats, nwg * 4, tag, c, [&](int i, float v) {
        const int w = i >> 2, f = i & 3;
        if (f == 0) st_max[w] = v;
        else if (f == 1) st_sum[w] = v;
        else if (f == 2) st_arg[w] = v;
    });
    __syncthreads();
    c.mark(0);
    if (temperature == 0.0f) {  // model.cpp:272-283: first maximum wins
        if (tid == 0) {
            ArgMax g{-INFINITY, 0x7fffffff};
            int target = 0;
            for (int w = 0; w < nwg; ++w) {
                const ArgMax cand{st_max[w], __float_as_int(st_arg[w])};
                if (cand.v > g.v || (cand.v == g.v && cand.i < g.i)) {
                    g = cand;
                    target = w;
                }
            }
            s_target = target;
            s_token = (g.i == 0x7fffffff) ? 0 : g.i;
        }
        __syncthreads();
    } else {
        float top = -INFINITY;
        for (int w = tid; w < nwg; w += nthreads) top = fmaxf(top, st_max[w]);
        top = block_max(top, s_scratch);
        float mass = 0.0f;
        for (int w = tid; w < nwg; w += nthreads) {
            const float m = (st_max[w] == -INFINITY) ? 0.0f : st_sum[w] * expf(st_max[w] - top);
            st_cum[w] = m;
            mass += m;
        }
        const float total = block_sum(mass, s_scratch);
        const float r = c.r;
        if (tid == 0) {
            // sequential in workgroup order = index order of the CDF (model.cpp:294-301)
            float cum = 0.0f;
            int target = -1;
            for (int w = 0; w < nwg; ++w) {
                const float before = cum;
                cum += st_cum[w] / total;
                st_cum[w] = before;
                if (target < 0 && r < cum) target = w;
            }
            s_target = target;
            s_token = vocab - 1;  // model.cpp:302 when no bucket is reached
        }
        __syncthreads();
        if (s_target == wg) {
            // inside the target workgroup: p_i = e_i * exp(m_w - top) / total, running sum in index order
            const float f = expf(mine.v - top) / total;
            const float before = st_cum[wg];
            const int per_thread = (n + nthreads - 1) / nthreads;
            const int begin = tid * per_thread, end = min(n, begin + per_thread);
            float chunk_sum = 0.0f;
            for (int i = begin; i < end; ++i) chunk_sum += lg[i] * f;
            const float incl = wave_inclusive_scan(chunk_sum);
            __shared__ float wave_tot[16];
            if (lane_id() == kWave - 1) wave_tot[tid / kWave] = incl;
            __syncthreads();
            float offset = before;
            for (int w = 0; w < tid / kWave; ++w) offset += wave_tot[w];
            offset += incl - chunk_sum;
            float run = 0.0f;
            int found = 0x7fffffff;
            for (int i = begin; i < end; ++i) {
                run += lg[i] * f;
                if (found == 0x7fffffff && r < offset + run) found = r0 + i;
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) found = min(found, __shfl_xor(found, off));
            __shared__ int wave_found[16];
            if (lane_id() == 0) wave_found[tid / kWave] = found;
            __syncthreads();
            if (tid == 0) {
                int f0 = wave_found[0];
                for (int w = 1; w < kWaves; ++w) f0 = min(f0, wave_found[w]);
                s_token = (f0 == 0x7fffffff) ? r1 - 1 : f0;  // rounding left the bucket short: its last row
            }
            __syncthreads();
        }
    }
    // Exactly one workgroup finishes the token: the target, or (no bucket reached) the last one.
    const bool finisher = (s_target == wg) || (s_target < 0 && wg == nwg - 1);
    if (finisher && tid == 0) {
        finish_token(a, s_token, 0u);
    }
    c.mark(1);
    ++c.phase_index;
}

// ---------------------------------------------------------------------------
// The kernel
// ---------------------------------------------------------------------------

template <bool kF16>
__global__ __launch_bounds__(kThreads) void k_decode_dataflow(DecodeArgs a, Tagged t, int rows_per_wg,
                                                              int lds_xs_floats) {
    extern __shared__ __align__(16) float lds[];
    const int wg = blockIdx.x, nwg = gridDim.x;
    const int dim_pad = (a.dim + 7) & ~7;
    Lds l{lds, lds + dim_pad, lds + dim_pad + lds_xs_floats};
    const StepParams* sp = a.step;
    Ctx c{a, t, t.base, (wg == 0) ? a.trace : nullptr, 0u,
          sp->token, sp->pos, sp->history_len, sp->temperature, sp->penalty, step_uniform(a)};
    if (c.trace && threadIdx.x == 0) c.trace[2u * phases_per_token(a.n_layers)] = wall_clock64();
    const int wbytes = kF16 ? 2 : 4;
    for (int layer = 0; layer < a.n_layers; ++layer) {
        df_qkv<kF16>(c, l, layer, wg, nwg);
        df_attention(c, l, layer, wg, nwg);
        df_proj<kF16, 2, 4>(c, l, a.wo + static_cast<size_t>(layer) * a.dim * a.dim * wbytes, a.dim, a.dim, t.xb,
                            c.seq(layer, kAtt), c.seq(layer, kOproj), wg, nwg);
        df_gateup<kF16>(c, l, layer, wg, nwg);
        df_proj<kF16, 1, 8>(c, l, a.w2 + static_cast<size_t>(layer) * a.dim * a.hidden * wbytes, a.dim, a.hidden, t.hb,
                            c.seq(layer, kGateUp), c.seq(layer, kDown), wg, nwg);
    }
    df_classify_sample<kF16>(c, l, wg, nwg, rows_per_wg);
}

}  // namespace df

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

namespace {

struct Plan {
    int grid;
    int rows_per_wg;
    int xs_floats;
    size_t lds_bytes;
};

Plan plan_for(const lpp_model* m) {
    const lpp_config& c = m->cfg;
    Plan p;
    p.grid = compute_units();
    const int per = (c.vocab_size + p.grid - 1) / p.grid;
    p.rows_per_wg = (per + 1) & ~1;
    const int dim_pad = (c.dim + 7) & ~7;
    int xs = (c.hidden_dim + 7) & ~7;
    if (dim_pad > xs) xs = dim_pad;
    int hs_pad = 8;  // lanes per position * 8, as df_attention_item rounds it
    while (hs_pad < m->head_size) hs_pad *= 2;
    const int nwaves = df::kThreads / dev::kWave;
    const int att = m->gqa * hs_pad + m->gqa * ph::kAttBlock + 3 * m->gqa + nwaves * m->gqa * hs_pad  // q, scores, reduce
                    + 2 * hs_pad                                                                   // current k, v
                    + m->gqa * m->max_splits * (m->head_size + 2);                                 // split gather
    if (att > xs) xs = att;
    if (4 * p.grid > xs) xs = 4 * p.grid;
    p.xs_floats = xs;
    p.lds_bytes = static_cast<size_t>(dim_pad + xs + ((p.rows_per_wg + 7) & ~7)) * sizeof(float);
    return p;
}

df::Tagged tagged_of(const lpp_model* m) {
    const lpp_config& c = m->cfg;
    df::Tagged t;
    df::u64* p = static_cast<df::u64*>(m->tagged);
    t.x = p;            p += c.dim;
    t.q = p;            p += c.dim;
    t.k = p;            p += m->kv_dim;
    t.v = p;            p += m->kv_dim;
    t.xb = p;           p += c.dim;
    t.hb = p;           p += c.hidden_dim;
    t.part = p;         p += static_cast<size_t>(c.n_heads) * m->max_splits * (m->head_size + 2);
    t.stats = p;
    t.base = m->df_base;
    t.abort = m->sync_words + 65;
    t.spin_limit = m->spin_limit;
    return t;
}

}  // namespace

size_t dataflow_tagged_bytes(const lpp_model* m) {
    const lpp_config& c = m->cfg;
    const size_t n = static_cast<size_t>(c.dim) * 3 + static_cast<size_t>(m->kv_dim) * 2 + c.hidden_dim +
                     static_cast<size_t>(c.n_heads) * m->max_splits * (m->head_size + 2) + 4u * 1024u;
    return n * sizeof(df::u64);
}

template <bool kF16>
static lpp_status launch_impl(lpp_model* m, const ph::DecodeArgs& a, hipStream_t s) {
    const Plan p = plan_for(m);
    if (m->persist_grid == 0) {
        LPP_REQUIRE(p.grid <= 1024, "persistent decode: %d compute units exceed the statistics table", p.grid);
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&df::k_decode_dataflow<kF16>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(p.lds_bytes)) != hipSuccess)
            return fail(LPP_ERR_UNSUPPORTED, "persistent decode needs %zu bytes of LDS per workgroup", p.lds_bytes);
        int per_cu = 0;
        LPP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, df::k_decode_dataflow<kF16>, df::kThreads,
                                                              p.lds_bytes));
        if (per_cu < 1)
            return fail(LPP_ERR_UNSUPPORTED, "persistent decode kernel does not fit a compute unit (LDS %zu bytes)",
                        p.lds_bytes);
        m->persist_grid = p.grid;
    }
    hipLaunchKernelGGL((df::k_decode_dataflow<kF16>), dim3(m->persist_grid), dim3(df::kThreads), p.lds_bytes, s, a,
                       tagged_of(m), p.rows_per_wg, p.xs_floats);
    LPP_CHECK_LAUNCH("k_decode_dataflow");
    m->df_base += df::phases_per_token(m->cfg.n_layers);
    return LPP_OK;
}

lpp_status dataflow_launch(lpp_model* m, const ph::DecodeArgs& a, hipStream_t s) {
    return m->cfg.weight_precision == LPP_WEIGHT_FP16 ? launch_impl<true>(m, a, s) : launch_impl<false>(m, a, s);
}

unsigned dataflow_phases_per_token(int n_layers) { return df::phases_per_token(n_layers); }

}  // namespace lpp
