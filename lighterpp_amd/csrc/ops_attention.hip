// ops_attention.hip -- lpp_multihead_gemv, lpp_scale_multihead,
// lpp_softmax_multihead, lpp_aggregation_multihead.
//
// Replace cuda_multihead_gemv (reference src/multihead_gemv.cu:6-68),
// cuda_scale_multihead (src/scale.cu:6-21), cuda_softmax_multihead
// (src/softmax.cu:5-125) and cuda_aggregation_multihead
// (src/aggregation.cu:6-31).  The CPU statement of the same steps is
// src/model.cpp:178-199 with softmax from src/ops.cpp:56-75.
//
// K and V rows are head_size binary16 values; a group of kGroup lanes covers
// one cache position with one 16-byte load per lane, so a wavefront load
// spans 64/kGroup consecutive positions of one KV head (contiguous in the
// [layer][kv_head][pos][head_size] cache).  Query heads that share a KV head
// are served from the same loaded K.
#include "lpp_device.hpp"
#include "lpp_internal.hpp"

namespace lpp {
namespace {

using namespace dev;

constexpr int kAttThreads = 256;

// Sum over a group of kGroup adjacent lanes (kGroup a power of two <= 16).
template <int kGroup>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (kGroup >= 2) v += dpp_move<kDppXor1>(v);
    if constexpr (kGroup >= 4) v += dpp_move<kDppXor2>(v);
    if constexpr (kGroup >= 8) v += dpp_move<kDppHalfMirror>(v);
    if constexpr (kGroup >= 16) v += dpp_move<kDppMirror>(v);
    return v;
}

// scores: grid (position tiles, kv heads).
template <int kGroup>
__global__ __launch_bounds__(kAttThreads) void scores_kernel(float* __restrict__ out,
                                                             const float* __restrict__ q,
                                                             const uint16_t* __restrict__ k_layer,
                                                             int npos, int gqa, int head_size,
                                                             int seq_len) {
    extern __shared__ __align__(16) float qs[];  // [gqa][hs_pad]
    const int kvh = blockIdx.y;
    const int hs_pad = kGroup * 8;
    for (int i = threadIdx.x; i < gqa * hs_pad; i += kAttThreads) {
        const int qh = i / hs_pad, e = i - qh * hs_pad;
        qs[i] = (e < head_size) ? q[static_cast<size_t>(kvh * gqa + qh) * head_size + e] : 0.0f;
    }
    __syncthreads();

    constexpr int kPosPerBlock = kAttThreads / kGroup;
    const int sub = static_cast<int>(threadIdx.x) % kGroup;
    const int t = static_cast<int>(blockIdx.x) * kPosPerBlock + static_cast<int>(threadIdx.x) / kGroup;
    const bool live = (t < npos) && (sub * 8 < head_size);
    uintx4 kb = uintx4{0u, 0u, 0u, 0u};
    if (live) {
        const uint16_t* kp = k_layer + (static_cast<size_t>(kvh) * seq_len + t) * head_size + sub * 8;
        kb = load16(kp);
    }
    for (int qh = 0; qh < gqa; ++qh) {
        const float* qv = qs + qh * hs_pad + sub * 8;
        floatx4 xa = *reinterpret_cast<const floatx4*>(qv);
        floatx4 xb = *reinterpret_cast<const floatx4*>(qv + 4);
        float s = group_sum<kGroup>(dot8(kb, xa, xb, 0.0f));
        if (sub == 0 && t < npos) out[static_cast<size_t>(kvh * gqa + qh) * seq_len + t] = s;
    }
}

// Any head_size: one thread per (head, position).
__global__ __launch_bounds__(kAttThreads) void scores_generic_kernel(float* __restrict__ out,
                                                                     const float* __restrict__ q,
                                                                     const uint16_t* __restrict__ k_layer,
                                                                     int npos, int gqa, int head_size,
                                                                     int seq_len) {
    const int h = blockIdx.y;
    const int t = static_cast<int>(blockIdx.x) * kAttThreads + static_cast<int>(threadIdx.x);
    if (t >= npos) return;
    const uint16_t* kp = k_layer + (static_cast<size_t>(h / gqa) * seq_len + t) * head_size;
    const float* qv = q + static_cast<size_t>(h) * head_size;
    float s = 0.0f;
    for (int e = 0; e < head_size; ++e) s = fmaf(f16_bits_to_f32(kp[e]), qv[e], s);
    out[static_cast<size_t>(h) * seq_len + t] = s;
}

__global__ __launch_bounds__(kAttThreads) void scale_kernel(float* att, float scale, int npos,
                                                            int att_stride) {
    const int t = static_cast<int>(blockIdx.x) * kAttThreads + static_cast<int>(threadIdx.x);
    if (t < npos) att[static_cast<size_t>(blockIdx.y) * att_stride + t] *= scale;
}

// ops.cpp:56-75 per head: max, expf(x - max) with a tree sum, true division.
constexpr int kSoftmaxThreads = 1024;
// kSoftmaxKept: values a thread keeps in registers (1, 4 or 16: rows of up to 16384 positions, the context cap of
// loader.cpp:310); 0: any length, the row re-read from memory in every pass.
template <int kSoftmaxKept>
__global__ __launch_bounds__(kSoftmaxThreads) void softmax_kernel(float* out, const float* x,
                                                                  int npos, int att_stride) {
    __shared__ float scratch[16];
    const float* row = x + static_cast<size_t>(blockIdx.x) * att_stride;
    float* orow = out + static_cast<size_t>(blockIdx.x) * att_stride;
    if constexpr (kSoftmaxKept > 0) {
        // The row stays in registers between the three passes (one read, one write; the same values meet the same
        // reductions in the same order as below, so the result is the same bit for bit).
        float v[kSoftmaxKept > 0 ? kSoftmaxKept : 1];
        float top = -INFINITY;
#pragma unroll
        for (int k = 0; k < kSoftmaxKept; ++k) {
            const int t = static_cast<int>(threadIdx.x) + k * kSoftmaxThreads;
            v[k] = t < npos ? row[t] : -INFINITY;
        }
#pragma unroll
        for (int k = 0; k < kSoftmaxKept; ++k) top = fmaxf(top, v[k]);
        top = block_max(top, scratch);
        float total = 0.0f;
#pragma unroll
        for (int k = 0; k < kSoftmaxKept; ++k) {
            const int t = static_cast<int>(threadIdx.x) + k * kSoftmaxThreads;
            if (t < npos) {
                v[k] = expf(v[k] - top);
                total += v[k];
            }
        }
        total = block_sum(total, scratch);
#pragma unroll
        for (int k = 0; k < kSoftmaxKept; ++k) {
            const int t = static_cast<int>(threadIdx.x) + k * kSoftmaxThreads;
            if (t < npos) orow[t] = v[k] / total;
        }
        return;
    }
    float top = -INFINITY;
    for (int t = threadIdx.x; t < npos; t += kSoftmaxThreads) top = fmaxf(top, row[t]);
    top = block_max(top, scratch);
    float total = 0.0f;
    for (int t = threadIdx.x; t < npos; t += kSoftmaxThreads) {
        const float e = expf(row[t] - top);
        orow[t] = e;
        total += e;
    }
    total = block_sum(total, scratch);
    for (int t = threadIdx.x; t < npos; t += kSoftmaxThreads) orow[t] = orow[t] / total;
}

// aggregation: one workgroup per query head.  Lane groups stride over the
// positions, each lane keeping 8 output columns; the per-group partial sums
// are combined through LDS in a fixed order.
constexpr int kAggThreads = 1024;
template <int kGroup>
__global__ __launch_bounds__(kAggThreads) void aggregate_kernel(float* __restrict__ out,
                                                                const uint16_t* __restrict__ v_layer,
                                                                const float* __restrict__ att,
                                                                int npos, int head_size, int gqa,
                                                                int att_stride) {
    extern __shared__ __align__(16) float part[];  // [ngroups][hs_pad]
    constexpr int kGroups = kAggThreads / kGroup;
    const int hs_pad = kGroup * 8;
    const int h = blockIdx.x;
    const int sub = static_cast<int>(threadIdx.x) % kGroup;
    const int grp = static_cast<int>(threadIdx.x) / kGroup;
    const uint16_t* vh = v_layer + static_cast<size_t>(h / gqa) * att_stride * head_size;
    const float* ah = att + static_cast<size_t>(h) * att_stride;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (sub * 8 < head_size) {
        for (int t = grp; t < npos; t += kGroups) {
            const float a = ah[t];
            half8_t vv = as_half8(load16(vh + static_cast<size_t>(t) * head_size + sub * 8));
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = fmaf(static_cast<float>(vv[e]), a, acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[grp * hs_pad + sub * 8 + e] = acc[e];
    __syncthreads();
    // Tree over groups: halve until one row is left.
    for (int width = kGroups / 2; width >= 1; width >>= 1) {
        for (int i = threadIdx.x; i < width * hs_pad; i += kAggThreads)
            part[i] += part[i + width * hs_pad];
        __syncthreads();
    }
    for (int e = threadIdx.x; e < head_size; e += kAggThreads)
        out[static_cast<size_t>(h) * head_size + e] = part[e];
}

// Long contexts: several workgroups per query head, each over a contiguous run of positions, so that the launch has
// work for every compute unit (one workgroup per head leaves most of them idle and takes 29 us for 8193 positions
// of the 1B shape).  A workgroup leaves its partial sums in a scratch area that lives in the library's device image
// (the operator allocates nothing and takes no workspace argument); the workgroup of a head that finishes last adds
// the partials up, always in split order, so the result does not depend on who finished when.  Calls on different
// streams would share the scratch: like the reference's operators, these are for one stream.
constexpr int kAggSplitThreads = 512;
constexpr int kAggMaxHeads = 256, kAggMaxSplits = 8, kAggPad = 128;
static __device__ float agg_partials[kAggMaxHeads * kAggMaxSplits * kAggPad];
static __device__ unsigned agg_tickets[kAggMaxHeads];  // back at zero after every launch

template <int kGroup>
__global__ __launch_bounds__(kAggSplitThreads) void aggregate_split_kernel(float* __restrict__ out,
                                                                           const uint16_t* __restrict__ v_layer,
                                                                           const float* __restrict__ att, int npos,
                                                                           int head_size, int gqa, int att_stride,
                                                                           float* partials, unsigned* tickets) {
    constexpr int kWaves = kAggSplitThreads / kWave;
    __shared__ float part[kWaves][kAggPad];  // a wavefront's sums, one row each
    __shared__ int is_last;
    constexpr int kGroups = kAggSplitThreads / kGroup;
    const int h = blockIdx.x, split = blockIdx.y, nsplits = gridDim.y;
    const int sub = static_cast<int>(threadIdx.x) % kGroup;
    const int grp = static_cast<int>(threadIdx.x) / kGroup;
    const int chunk = (npos + nsplits - 1) / nsplits;
    const int t_begin = split * chunk, t_end = min(npos, t_begin + chunk);
    const uint16_t* vh = v_layer + static_cast<size_t>(h / gqa) * att_stride * head_size + sub * 8;
    const float* ah = att + static_cast<size_t>(h) * att_stride;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (sub * 8 < head_size) {
        constexpr int kUnroll = 8;  // rows requested before the first is used: 512 positions a trip (heads of 64)
        for (int t0 = t_begin + grp; t0 < t_end; t0 += kUnroll * kGroups) {
            uintx4 rows[kUnroll];
            float w[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int t = t0 + u * kGroups;
                const bool live = t < t_end;
                rows[u] = load16(vh + static_cast<size_t>(live ? t : t_begin) * head_size);
                w[u] = live ? ah[t] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const half8_t vv = as_half8(rows[u]);
                // (a weight of zero must not meet whatever the clamped row holds)
                if (w[u] != 0.0f) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) acc[e] = fmaf(static_cast<float>(vv[e]), w[u], acc[e]);
                }
            }
        }
    }
    // The groups of a wavefront meet by lane exchange (group g with g ^ 1, then ^ 2, ...), the wavefronts through LDS,
    // added in wavefront order: always the same order, so a call repeats bit for bit.
#pragma unroll
    for (int off = kGroup; off < kWave; off <<= 1)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], off);
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    if (lane_id() < kGroup) {
#pragma unroll
        for (int e = 0; e < 8; ++e) part[wave][sub * 8 + e] = acc[e];
    }
    __syncthreads();
    float* mine = partials + (static_cast<size_t>(h) * kAggMaxSplits + split) * kAggPad;
    for (int e = threadIdx.x; e < head_size; e += kAggSplitThreads) {
        float s = part[0][e];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) s += part[w][e];
        Mem<true>::st(mine + e, s);
    }
    // (the barrier waits for this workgroup's stores; the ticket is drawn after it)
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned ticket = __hip_atomic_fetch_add(&tickets[h], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = ticket == static_cast<unsigned>(nsplits - 1) ? 1 : 0;
        if (is_last) __hip_atomic_store(&tickets[h], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return;
    // the last range to arrive adds the ranges' sums in range order, eight of them requested at a time
    const float* all = partials + static_cast<size_t>(h) * kAggMaxSplits * kAggPad;
    for (int e = threadIdx.x; e < head_size; e += kAggSplitThreads) {
        float s = 0.0f;
        for (int k0 = 0; k0 < nsplits; k0 += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = k0 + u < nsplits ? Mem<true>::ld(all + (k0 + u) * kAggPad + e) : 0.0f;
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (k0 + u < nsplits) s = (k0 + u == 0) ? v[u] : s + v[u];
        }
        out[static_cast<size_t>(h) * head_size + e] = s;
    }
}

// Device addresses of the scratch above, per device (the arrays' names are host-side handles only).
constexpr int kMaxDevices = 64;
float* g_agg_partials[kMaxDevices] = {};
unsigned* g_agg_tickets[kMaxDevices] = {};
lpp_status agg_scratch(float** partials, unsigned** tickets) {
    int device = -1;
    LPP_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(LPP_ERR_UNSUPPORTED, "device ordinal %d beyond %d", device, kMaxDevices - 1);
    if (g_agg_partials[device] == nullptr) {
        void* p = nullptr;
        void* t = nullptr;
        LPP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(agg_partials)));
        LPP_HIP(hipGetSymbolAddress(&t, HIP_SYMBOL(agg_tickets)));
        g_agg_partials[device] = static_cast<float*>(p);
        g_agg_tickets[device] = static_cast<unsigned*>(t);
    }
    *partials = g_agg_partials[device];
    *tickets = g_agg_tickets[device];
    return LPP_OK;
}

__global__ __launch_bounds__(kAttThreads) void aggregate_generic_kernel(float* __restrict__ out,
                                                                        const uint16_t* __restrict__ v_layer,
                                                                        const float* __restrict__ att,
                                                                        int npos, int head_size,
                                                                        int gqa, int att_stride) {
    const int h = blockIdx.x;
    const uint16_t* vh = v_layer + static_cast<size_t>(h / gqa) * att_stride * head_size;
    const float* ah = att + static_cast<size_t>(h) * att_stride;
    for (int e = threadIdx.x; e < head_size; e += kAttThreads) {
        float s = 0.0f;
        for (int t = 0; t < npos; ++t) s = fmaf(f16_bits_to_f32(vh[static_cast<size_t>(t) * head_size + e]), ah[t], s);
        out[static_cast<size_t>(h) * head_size + e] = s;
    }
}

int group_for(int head_size) {
    if (head_size % 8 != 0 || head_size > 128) return 0;
    int g = 1;
    while (g * 8 < head_size) g *= 2;
    return g;
}

}  // namespace
}  // namespace lpp

extern "C" {

lpp_status lpp_multihead_gemv(float* d_out, const float* d_q, const lpp_half* d_k_cache, int layer,
                              int pos, int n_heads, int n_kv_heads, int head_size, int seq_len) {
    using namespace lpp;
    LPP_REQUIRE(d_out && d_q && d_k_cache, "lpp_multihead_gemv: null pointer");
    LPP_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
                "lpp_multihead_gemv: n_heads = %d must be a positive multiple of n_kv_heads = %d",
                n_heads, n_kv_heads);
    LPP_REQUIRE(head_size > 0 && seq_len > 0 && layer >= 0, "lpp_multihead_gemv: head_size = %d, seq_len = %d, layer = %d",
                head_size, seq_len, layer);
    LPP_REQUIRE(pos >= 0 && pos < seq_len, "lpp_multihead_gemv: pos = %d outside [0, %d)", pos, seq_len);
    const int gqa = n_heads / n_kv_heads;
    const int npos = pos + 1;
    // multihead_gemv.cu:27-30: the layer offset is applied here, in 64 bits.
    const uint16_t* k_layer = d_k_cache + static_cast<size_t>(layer) * n_kv_heads * seq_len * head_size;
    const int g = group_for(head_size);
    const bool aligned = reinterpret_cast<uintptr_t>(k_layer) % 16 == 0;
    if (g == 0 || !aligned) {
        hipLaunchKernelGGL(scores_generic_kernel, dim3((npos + kAttThreads - 1) / kAttThreads, n_heads),
                           dim3(kAttThreads), 0, stream(), d_out, d_q, k_layer, npos, gqa, head_size, seq_len);
        LPP_CHECK_LAUNCH("scores_generic_kernel");
        return LPP_OK;
    }
    const int per_block = kAttThreads / g;
    const dim3 grid((npos + per_block - 1) / per_block, n_kv_heads);
    const size_t lds = static_cast<size_t>(gqa) * g * 8 * sizeof(float);
    LPP_REQUIRE(lds <= 65536, "lpp_multihead_gemv: %d query heads per KV head do not fit in LDS", gqa);
#define LPP_SCORES(G)                                                                              \
    hipLaunchKernelGGL((scores_kernel<G>), grid, dim3(kAttThreads), lds, stream(), d_out, d_q,     \
                       k_layer, npos, gqa, head_size, seq_len)
    switch (g) {
        case 1: LPP_SCORES(1); break;
        case 2: LPP_SCORES(2); break;
        case 4: LPP_SCORES(4); break;
        case 8: LPP_SCORES(8); break;
        default: LPP_SCORES(16); break;
    }
#undef LPP_SCORES
    LPP_CHECK_LAUNCH("scores_kernel");
    return LPP_OK;
}

lpp_status lpp_scale_multihead(float* d_att, float scale, int n_heads, int seq_len, int att_stride) {
    using namespace lpp;
    LPP_REQUIRE(d_att != nullptr, "lpp_scale_multihead: null pointer");
    LPP_REQUIRE(n_heads > 0 && seq_len >= 0 && att_stride >= seq_len,
                "lpp_scale_multihead: n_heads = %d, seq_len = %d, att_stride = %d", n_heads, seq_len, att_stride);
    if (seq_len == 0) return LPP_OK;
    hipLaunchKernelGGL(scale_kernel, dim3((seq_len + kAttThreads - 1) / kAttThreads, n_heads),
                       dim3(kAttThreads), 0, stream(), d_att, scale, seq_len, att_stride);
    LPP_CHECK_LAUNCH("scale_kernel");
    return LPP_OK;
}

lpp_status lpp_softmax_multihead(float* d_out, const float* d_x, int n_heads, int seq_len, int att_stride) {
    using namespace lpp;
    LPP_REQUIRE(d_out && d_x, "lpp_softmax_multihead: null pointer");
    LPP_REQUIRE(n_heads > 0 && seq_len > 0 && att_stride >= seq_len,
                "lpp_softmax_multihead: n_heads = %d, seq_len = %d, att_stride = %d", n_heads, seq_len, att_stride);
#define LPP_SOFTMAX(KEPT)                                                                                    \
    hipLaunchKernelGGL((softmax_kernel<KEPT>), dim3(n_heads), dim3(kSoftmaxThreads), 0, stream(), d_out, d_x, \
                       seq_len, att_stride)
    if (seq_len <= kSoftmaxThreads) LPP_SOFTMAX(1);
    else if (seq_len <= 4 * kSoftmaxThreads) LPP_SOFTMAX(4);
    else if (seq_len <= 16 * kSoftmaxThreads) LPP_SOFTMAX(16);
    else LPP_SOFTMAX(0);
#undef LPP_SOFTMAX
    LPP_CHECK_LAUNCH("softmax_kernel");
    return LPP_OK;
}

lpp_status lpp_aggregation_multihead(float* d_out, const lpp_half* d_v, const float* d_att, int n_heads,
                                     int seq_len, int head_size, int gqa_factor, int att_stride) {
    using namespace lpp;
    LPP_REQUIRE(d_out && d_v && d_att, "lpp_aggregation_multihead: null pointer");
    LPP_REQUIRE(n_heads > 0 && head_size > 0 && gqa_factor > 0 && seq_len > 0 && att_stride >= seq_len,
                "lpp_aggregation_multihead: n_heads = %d, head_size = %d, gqa_factor = %d, seq_len = %d, att_stride = %d",
                n_heads, head_size, gqa_factor, seq_len, att_stride);
    const int g = group_for(head_size);
    const bool aligned = reinterpret_cast<uintptr_t>(d_v) % 16 == 0;
    if (g == 0 || !aligned) {
        hipLaunchKernelGGL(aggregate_generic_kernel, dim3(n_heads), dim3(kAttThreads), 0, stream(), d_out,
                           d_v, d_att, seq_len, head_size, gqa_factor, att_stride);
        LPP_CHECK_LAUNCH("aggregate_generic_kernel");
        return LPP_OK;
    }
    // Work for every compute unit once a head's context is long: a workgroup per head and range of a few hundred
    // positions.  No more than eight ranges: the ranges of a head meet at one counter, and read-modify-writes of one
    // address at device scope are served one at a time, 0.1 us each (8193 positions, 32 heads: 13.2 us with 32 ranges,
    // 10.3 with 16, 9.6 with 8, of which an empty launch of the same grid takes 3.9).
    int splits = (compute_units() + n_heads - 1) / n_heads;
    if (splits > kAggMaxSplits) splits = kAggMaxSplits;
    if (splits > seq_len / 256) splits = seq_len / 256;
    if (splits > 1 && n_heads <= kAggMaxHeads && g >= 1) {
        float* partials = nullptr;
        unsigned* tickets = nullptr;
        LPP_TRY(agg_scratch(&partials, &tickets));
        const size_t lds_split = 0;
#define LPP_AGG_SPLIT(G)                                                                                              \
    hipLaunchKernelGGL((aggregate_split_kernel<G>), dim3(n_heads, splits), dim3(kAggSplitThreads), lds_split, stream(), \
                       d_out, d_v, d_att, seq_len, head_size, gqa_factor, att_stride, partials, tickets)
        switch (g) {
            case 1: LPP_AGG_SPLIT(1); break;
            case 2: LPP_AGG_SPLIT(2); break;
            case 4: LPP_AGG_SPLIT(4); break;
            case 8: LPP_AGG_SPLIT(8); break;
            default: LPP_AGG_SPLIT(16); break;
        }
#undef LPP_AGG_SPLIT
        LPP_CHECK_LAUNCH("aggregate_split_kernel");
        return LPP_OK;
    }
    const size_t lds = static_cast<size_t>(kAggThreads) * 8 * sizeof(float);  // 32 KiB
#define LPP_AGG(G)                                                                                  \
    hipLaunchKernelGGL((aggregate_kernel<G>), dim3(n_heads), dim3(kAggThreads), lds, stream(), d_out, \
                       d_v, d_att, seq_len, head_size, gqa_factor, att_stride)
    switch (g) {
        case 1: LPP_AGG(1); break;
        case 2: LPP_AGG(2); break;
        case 4: LPP_AGG(4); break;
        case 8: LPP_AGG(8); break;
        default: LPP_AGG(16); break;
    }
#undef LPP_AGG
    LPP_CHECK_LAUNCH("aggregate_kernel");
    return LPP_OK;
}

}  // extern "C"
