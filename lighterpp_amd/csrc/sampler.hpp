// sampler.hpp -- device-side steps of the sampler, shared by the lpp_sample
// operator (one launch per step) and the fused decode paths.
//
// Semantics are those of the CPU sampler (reference src/model.cpp:256-303):
//   1. repetition penalty, once per occurrence in the history window;
//   2. temperature 0: lowest index of the maximum;
//   3. otherwise x / temperature, softmax, and the smallest index i with
//      r < p_0 + ... + p_i, or vocab-1 when there is none.
// The vocabulary is cut into chunks of `chunk` entries, one workgroup per chunk;
// the per-chunk results the next step needs are kept in a SampleScratch the
// caller provides.  kCoh selects device-coherent accesses for everything another
// workgroup wrote earlier in the SAME kernel (see dev::Mem); between separate
// launches ordinary accesses do.
#pragma once

#include "lpp_device.hpp"

namespace lpp {
namespace smp {

using namespace dev;

constexpr int kSampleThreads = 256;
constexpr int kMaxChunks = 1024;

struct SampleScratch {
    float* chunk_max;   // [kMaxChunks]
    int* chunk_arg;     // [kMaxChunks]
    float* chunk_sum;   // [kMaxChunks]
    float* chunk_prob;  // [kMaxChunks]
};

// Entries per chunk so that at most kMaxChunks chunks cover the vocabulary; a
// multiple of 1024 so that any workgroup size up to 1024 divides it.
__host__ __device__ inline int chunk_size_for(int vocab) {
    int per_thread = 4;
    while (static_cast<long>(per_thread) * kSampleThreads * kMaxChunks < vocab) per_thread *= 2;
    return per_thread * kSampleThreads;
}

// Penalised value of one logit seen `count` times in the window
// (model.cpp:262-267 applied `count` times in a row).
__device__ __forceinline__ float penalise(float v, float penalty, int count) {
    for (int c = 0; c < count; ++c) {
        if (v > 0) v /= penalty;
        else v *= penalty;
    }
    return v;
}

// Occurrences of history[i] in the window if i is its first occurrence, else 0.
__device__ __forceinline__ int owned_count(const int* __restrict__ history, int history_len, int i) {
    const int tok = history[i];
    for (int j = 0; j < i; ++j)
        if (history[j] == tok) return 0;
    int count = 1;
    for (int j = i + 1; j < history_len; ++j) count += (history[j] == tok) ? 1 : 0;
    return count;
}

// Step 0 (one workgroup): penalty over the whole window, in place.  The thread
// holding a token's first occurrence replays all of that token's occurrences,
// so duplicates never race.
__device__ __forceinline__ void penalty_all(float* logits, int vocab, float penalty,
                                            const int* __restrict__ history, int history_len) {
    for (int i = threadIdx.x; i < history_len; i += blockDim.x) {
        const int tok = history[i];
        if (tok < 0 || tok >= vocab) continue;
        const int count = owned_count(history, history_len, i);
        if (count > 0) logits[tok] = penalise(logits[tok], penalty, count);
    }
}

// Step 1 (chunk c): src -> dst with the optional penalty (tokens that fall into
// this chunk only) and division by the temperature; records the chunk maximum
// and its lowest index.  src may equal dst.  A null history applies no penalty.
// dst[chunk c] is only ever touched again by the workgroup that owns chunk c.
template <bool kCoh>
__device__ __forceinline__ void scale_max_chunk(const float* src, float* dst, int vocab, int chunk,
                                                int c, float temperature, float penalty,
                                                const int* __restrict__ history, int history_len,
                                                SampleScratch sc) {
    __shared__ float sv[16];
    __shared__ int si[16];
    const int begin = c * chunk;
    const int end = min(begin + chunk, vocab);
    const int nthreads = static_cast<int>(blockDim.x);
    const bool penalise_here = history != nullptr && penalty > 1.0f && history_len > 0;
    if (penalise_here) {
        for (int i = begin + threadIdx.x; i < end; i += nthreads) dst[i] = Mem<kCoh>::ld(src + i);
        __syncthreads();
        for (int i = threadIdx.x; i < history_len; i += nthreads) {
            const int tok = history[i];
            if (tok < begin || tok >= end) continue;
            const int count = owned_count(history, history_len, i);
            if (count > 0) dst[tok] = penalise(dst[tok], penalty, count);
        }
        __syncthreads();
    }
    ArgMax best{-INFINITY, 0x7fffffff};
    for (int i = begin + threadIdx.x; i < end; i += nthreads) {
        float v = penalise_here ? dst[i] : Mem<kCoh>::ld(src + i);
        if (temperature != 0.0f) v = v / temperature;
        dst[i] = v;
        best = argmax_better(best, ArgMax{v, i});
    }
    best = wave_argmax(best);
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    const int nwaves = (nthreads + kWave - 1) / kWave;
    __syncthreads();
    if (lane_id() == 0) {
        sv[wave] = best.v;
        si[wave] = best.i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        ArgMax m{sv[0], si[0]};
        for (int w = 1; w < nwaves; ++w) m = argmax_better(m, ArgMax{sv[w], si[w]});
        Mem<kCoh>::st(sc.chunk_max + c, m.v);
        Mem<kCoh>::sti(sc.chunk_arg + c, m.i);
    }
}

// Temperature 0 (one workgroup): model.cpp:272-283, first maximum wins.
// Returns the answer in every thread.
template <bool kCoh>
__device__ __forceinline__ int argmax_over_chunks(int nchunks, SampleScratch sc) {
    __shared__ float sv[16];
    __shared__ int si[16];
    __shared__ int answer;
    ArgMax best{-INFINITY, 0x7fffffff};
    for (int c = threadIdx.x; c < nchunks; c += blockDim.x)
        best = argmax_better(best, ArgMax{Mem<kCoh>::ld(sc.chunk_max + c), Mem<kCoh>::ldi(sc.chunk_arg + c)});
    best = wave_argmax(best);
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    const int nwaves = (static_cast<int>(blockDim.x) + kWave - 1) / kWave;
    __syncthreads();
    if (lane_id() == 0) {
        sv[wave] = best.v;
        si[wave] = best.i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        ArgMax m{sv[0], si[0]};
        for (int w = 1; w < nwaves; ++w) m = argmax_better(m, ArgMax{sv[w], si[w]});
        // All-NaN logits leave the sentinel; the CPU loop would answer 0.
        answer = (m.i == 0x7fffffff) ? 0 : m.i;
    }
    __syncthreads();
    return answer;
}

// Every workgroup derives the same global value from a chunk table in the same
// order, so all of them agree to the bit.
template <bool kCoh>
__device__ __forceinline__ float table_max(const float* table, int n, float* scratch) {
    float v = -INFINITY;
    for (int c = threadIdx.x; c < n; c += blockDim.x) v = fmaxf(v, Mem<kCoh>::ld(table + c));
    return block_max(v, scratch);
}
template <bool kCoh>
__device__ __forceinline__ float table_sum(const float* table, int n, float* scratch) {
    float v = 0.0f;
    for (int c = threadIdx.x; c < n; c += blockDim.x) v += Mem<kCoh>::ld(table + c);
    return block_sum(v, scratch);
}

// Step 2 (chunk c): e = expf(x - max) in place; per-chunk sum.
template <bool kCoh>
__device__ __forceinline__ void exp_sum_chunk(float* vals, int vocab, int chunk, int nchunks, int c,
                                              SampleScratch sc) {
    __shared__ float scratch[16];
    const float top = table_max<kCoh>(sc.chunk_max, nchunks, scratch);
    const int begin = c * chunk;
    const int end = min(begin + chunk, vocab);
    float total = 0.0f;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const float e = expf(vals[i] - top);
        vals[i] = e;
        total += e;
    }
    total = block_sum(total, scratch);
    if (threadIdx.x == 0) Mem<kCoh>::st(sc.chunk_sum + c, total);
}

// Step 3 (chunk c): p = e / sum in place (the CPU leaves probabilities in the
// buffer too); per-chunk probability mass.
template <bool kCoh>
__device__ __forceinline__ void normalise_chunk(float* vals, int vocab, int chunk, int nchunks, int c,
                                                SampleScratch sc) {
    __shared__ float scratch[16];
    const float total = table_sum<kCoh>(sc.chunk_sum, nchunks, scratch);
    const int begin = c * chunk;
    const int end = min(begin + chunk, vocab);
    float mass = 0.0f;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const float p = vals[i] / total;
        vals[i] = p;
        mass += p;
    }
    mass = block_sum(mass, scratch);
    if (threadIdx.x == 0) Mem<kCoh>::st(sc.chunk_prob + c, mass);
}

// Step 4 (chunk c): cdf_i = (mass of earlier chunks) + (running sum inside the
// chunk); lowers *result to the smallest i of this chunk with r < cdf_i
// (model.cpp:296-301).  *result must hold vocab-1 (the :302 fallback) before any
// chunk runs this step.  Each thread owns chunk/blockDim consecutive entries and
// adds them in index order.
template <bool kCoh>
__device__ __forceinline__ void cdf_search_chunk(const float* probs, int vocab, int chunk, int c, float r,
                                                 SampleScratch sc, int* result) {
    __shared__ float scratch[16];
    __shared__ float wave_tot[16];
    float before = 0.0f;
    for (int k = threadIdx.x; k < c; k += blockDim.x) before += Mem<kCoh>::ld(sc.chunk_prob + k);
    before = block_sum(before, scratch);

    const int per_thread = chunk / static_cast<int>(blockDim.x);
    const int begin = c * chunk + static_cast<int>(threadIdx.x) * per_thread;
    const int end = min(begin + per_thread, vocab);
    float mine = 0.0f;
    for (int i = begin; i < end; ++i) mine += probs[i];
    const float incl = wave_inclusive_scan(mine);
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    __syncthreads();
    if (lane_id() == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    float offset = before;
    for (int w = 0; w < wave; ++w) offset += wave_tot[w];
    offset += incl - mine;

    float run = 0.0f;
    int found = 0x7fffffff;
    for (int i = begin; i < end; ++i) {
        run += probs[i];
        if (found == 0x7fffffff && r < offset + run) found = i;
    }
    // One atomic per workgroup: about half of all threads hold a candidate (every
    // entry past the crossing qualifies), and that many device-scope atomics on
    // one word would serialise for hundreds of microseconds.
    __shared__ int wave_found[16];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) found = min(found, __shfl_xor(found, off));
    __syncthreads();
    if (lane_id() == 0) wave_found[wave] = found;
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nwaves = (static_cast<int>(blockDim.x) + kWave - 1) / kWave;
        int best = wave_found[0];
        for (int w = 1; w < nwaves; ++w) best = min(best, wave_found[w]);
        if (best != 0x7fffffff) atomicMin(result, best);
    }
}

}  // namespace smp
}  // namespace lpp
