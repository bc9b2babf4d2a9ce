// prefill.hip -- batched prefill: the key/value cache entries of a run of prompt
// tokens in one pass over the weights.
//
// The reference has no such path: it prefills by decoding the prompt one token at
// a time and dropping what the sampler returns (src/main.cpp:163-180), which reads
// every weight once per prompt token.  Here the prompt's tokens go through each
// layer together, so the matrix products are GEMMs on the matrix cores
// (v_mfma_f32_32x32x16_f16) and every weight is read once per chunk of up to 512
// tokens.  What a prefill leaves behind is exactly what the decode loop reads
// later: K and V of the prompt positions, rounded to binary16 as the cache store
// rounds them (model.cpp:171-176, kernels.cuh:34).  The classifier and the sampler
// are not run: the ids they would produce are the ones main.cpp drops.
//
// Arithmetic: weights binary16 as stored; activations fp32, split for the matrix
// cores into a binary16 head and a binary16 remainder (x = hi + lo to about 2^-22),
// both multiplied into the same fp32 accumulators; everything between the GEMMs
// (RMSNorm, RoPE, softmax, SwiGLU, residual) in fp32 with the operators' own
// operation order (ops.cpp:20-87).
#include <cmath>
#include <cstdlib>

#include "lpp_device.hpp"
#include "lpp_internal.hpp"
#include "lpp_model.hpp"

namespace lpp {
namespace pf {

using namespace dev;

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTileTokens = 128;    // token rows of a workgroup's output tile
constexpr int kTileFeatures = 128;  // weight rows of it
constexpr int kChunk = 512;         // prompt tokens per pass over the weights
constexpr int kMaxGqa = 8;          // query heads per KV head the attention kernel keeps in registers

// ---------------------------------------------------------------------------
// Small per-token kernels
// ---------------------------------------------------------------------------

// x[t][:] = embedding row of tokens[t] (model.cpp:346-348).
__global__ __launch_bounds__(256) void k_embed(const float* __restrict__ emb, const int* __restrict__ tokens,
                                               float* __restrict__ x, int dim) {
    const int t = blockIdx.x;
    const float* src = emb + static_cast<size_t>(tokens[t]) * dim;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) x[static_cast<size_t>(t) * dim + i] = src[i];
}

__device__ __forceinline__ float block_sum256(float v, float* scratch) {
    v = wave_sum(v);
    if (lane_id() == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    const float total = (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
    __syncthreads();
    return total;
}

__device__ __forceinline__ void split_store(half_t* hi, half_t* lo, size_t at, float v) {
    const half_t h = static_cast<half_t>(v);
    hi[at] = h;
    lo[at] = static_cast<half_t>(v - static_cast<float>(h));
}

// (hi, lo)[t][:] = RMSNorm(x[t][:]) * gain (ops.cpp:20-32); rows t >= n_tokens are zero.
// With `splits` > 0 the residual update that precedes the norm is done here: x[t][:] += p[0][t][:] +
// p[1][t][:] + ... in that order, the partial products of a GEMM whose K was split (p[z] starts at
// partials + z * split_stride), written back to x.
__global__ __launch_bounds__(256) void k_norm_split(float* __restrict__ x, const float* __restrict__ gain,
                                                    half_t* __restrict__ hi, half_t* __restrict__ lo, int dim,
                                                    int n_tokens, const float* __restrict__ partials, int splits,
                                                    size_t split_stride) {
#pragma clang fp contract(off)
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const size_t row = static_cast<size_t>(t) * dim;
    if (t >= n_tokens) {
        for (int i = threadIdx.x; i < dim; i += blockDim.x) {
            hi[row + i] = static_cast<half_t>(0.0f);
            lo[row + i] = static_cast<half_t>(0.0f);
        }
        return;
    }
    float ss = 0.0f;
    for (int i = 4 * threadIdx.x; i < dim; i += 4 * blockDim.x) {
        floatx4 v = *reinterpret_cast<const floatx4*>(x + row + i);
        if (splits > 0) {
            for (int z = 0; z < splits; ++z) {
                const floatx4 a = *reinterpret_cast<const floatx4*>(partials + z * split_stride + row + i);
                v = floatx4{v[0] + a[0], v[1] + a[1], v[2] + a[2], v[3] + a[3]};
            }
            *reinterpret_cast<floatx4*>(x + row + i) = v;
        }
        ss += v[0] * v[0];
        ss += v[1] * v[1];
        ss += v[2] * v[2];
        ss += v[3] * v[3];
    }
    ss = block_sum256(ss, scratch);
    ss /= static_cast<float>(dim);
    ss += 1e-5f;
    const float scale = 1.0f / sqrtf(ss);
    for (int i = 4 * threadIdx.x; i < dim; i += 4 * blockDim.x) {
        const floatx4 v = *reinterpret_cast<const floatx4*>(x + row + i);
        const floatx4 gn = *reinterpret_cast<const floatx4*>(gain + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) split_store(hi, lo, row + i + e, v[e] * scale * gn[e]);
    }
}

// The same with a workgroup per row (dim = 1024 kPer) and the number of partial products known to
// the compiler: a thread's kPer x (1 + kSplits) loads are all requested before the first is used, so
// a row costs one round trip to memory and is read once.  Residual sum in the same order; the sum
// of squares runs over a thread's elements in order, across the lanes, then over the four
// wavefronts as (0 + 1) + (2 + 3).
template <int kPer, int kSplits>
__global__ __launch_bounds__(256) void k_norm_split_wide(float* __restrict__ x, const float* __restrict__ gain,
                                                         half_t* __restrict__ hi, half_t* __restrict__ lo, int n_tokens,
                                                         const float* __restrict__ partials, size_t split_stride) {
#pragma clang fp contract(off)
    constexpr int kDim = 1024 * kPer;
    __shared__ float scratch[4];
    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
    const int t = blockIdx.x;
    const size_t row = static_cast<size_t>(t) * kDim;
    const int first = 4 * threadIdx.x;
    if (t >= n_tokens) {
        const half4_t zero = {static_cast<half_t>(0.0f), static_cast<half_t>(0.0f), static_cast<half_t>(0.0f), static_cast<half_t>(0.0f)};
#pragma unroll
        for (int c = 0; c < kPer; ++c) {
            *reinterpret_cast<half4_t*>(hi + row + 1024 * c + first) = zero;
            if (lo != nullptr) *reinterpret_cast<half4_t*>(lo + row + 1024 * c + first) = zero;
        }
        return;
    }
    floatx4 v[kPer], a[kSplits > 0 ? kSplits : 1][kPer], gn[kPer];
#pragma unroll
    for (int c = 0; c < kPer; ++c) v[c] = *reinterpret_cast<const floatx4*>(x + row + 1024 * c + first);
#pragma unroll
    for (int z = 0; z < kSplits; ++z)
#pragma unroll
        for (int c = 0; c < kPer; ++c) a[z][c] = *reinterpret_cast<const floatx4*>(partials + z * split_stride + row + 1024 * c + first);
#pragma unroll
    for (int c = 0; c < kPer; ++c) gn[c] = *reinterpret_cast<const floatx4*>(gain + 1024 * c + first);
    if (kSplits > 0) {
#pragma unroll
        for (int c = 0; c < kPer; ++c) {
#pragma unroll
            for (int z = 0; z < kSplits; ++z)
                v[c] = floatx4{v[c][0] + a[z][c][0], v[c][1] + a[z][c][1], v[c][2] + a[z][c][2], v[c][3] + a[z][c][3]};
            *reinterpret_cast<floatx4*>(x + row + 1024 * c + first) = v[c];
        }
    }
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < kPer; ++c) {
        ss += v[c][0] * v[c][0];
        ss += v[c][1] * v[c][1];
        ss += v[c][2] * v[c][2];
        ss += v[c][3] * v[c][3];
    }
    ss = block_sum256(ss, scratch);
    ss /= static_cast<float>(kDim);
    ss += 1e-5f;
    const float scale = 1.0f / sqrtf(ss);
#pragma unroll
    for (int c = 0; c < kPer; ++c) {
        half4_t h, l;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float y = v[c][e] * scale * gn[c][e];
            h[e] = static_cast<half_t>(y);
            l[e] = static_cast<half_t>(y - static_cast<float>(h[e]));
        }
        *reinterpret_cast<half4_t*>(hi + row + 1024 * c + first) = h;
        if (lo != nullptr) *reinterpret_cast<half4_t*>(lo + row + 1024 * c + first) = l;  // (null: nobody reads the remainders)
    }
}

// RoPE on q and k of token t (ops.cpp:34-54), q kept in fp32, k and v written to the
// caches as binary16 at position pos0 + t (model.cpp:171-176).  With `splits` > 1, qs/ks/vs are the
// first of that many partial products, split_stride floats apart, and are summed in order here;
// q receives the rotated sum either way.
__global__ __launch_bounds__(256) void k_rope_scatter(float* __restrict__ q, const float* __restrict__ qs,
                                                      const float* __restrict__ ks, const float* __restrict__ vs,
                                                      const float2* __restrict__ rope, uint16_t* __restrict__ key_cache,
                                                      uint16_t* __restrict__ value_cache, int layer, int pos0, int dim,
                                                      int kv_dim, int hs, int seq_len, int splits, size_t split_stride) {
#pragma clang fp contract(off)
    const int t = blockIdx.x;
    const int pos = pos0 + t;
    const float2* cs_row = rope + static_cast<size_t>(pos) * (hs / 2);
    // (two pairs per thread: 16-byte loads and stores; dim, kv_dim and the head size are multiples of 4)
    auto summed = [&](const float* first, size_t at) {
        floatx4 v = *reinterpret_cast<const floatx4*>(first + at);
        for (int z = 1; z < splits; ++z) {
            const floatx4 a = *reinterpret_cast<const floatx4*>(first + z * split_stride + at);
            v = floatx4{v[0] + a[0], v[1] + a[1], v[2] + a[2], v[3] + a[3]};
        }
        return v;
    };
    for (int i = 4 * threadIdx.x; i < dim; i += 4 * blockDim.x) {
        const size_t at = static_cast<size_t>(t) * dim + i;
        const floatx4 cs = *reinterpret_cast<const floatx4*>(cs_row + ((i % hs) >> 1));  // (cos, sin) of two pairs
        const floatx4 v = summed(qs, at);
        *reinterpret_cast<floatx4*>(q + at) =
            floatx4{v[0] * cs[0] - v[1] * cs[1], v[0] * cs[1] + v[1] * cs[0], v[2] * cs[2] - v[3] * cs[3], v[2] * cs[3] + v[3] * cs[2]};
    }
    for (int i = 4 * threadIdx.x; i < kv_dim; i += 4 * blockDim.x) {
        const size_t at = static_cast<size_t>(t) * kv_dim + i;
        const floatx4 kk = summed(ks, at), vv = summed(vs, at);
        const floatx4 cs = *reinterpret_cast<const floatx4*>(cs_row + ((i % hs) >> 1));
        const int head = i / hs, within = i - head * hs;
        const size_t dst = static_cast<size_t>(layer) * kv_dim * seq_len + static_cast<size_t>(head) * seq_len * hs +
                           static_cast<size_t>(pos) * hs + within;
        typedef uint16_t ushort4_t __attribute__((ext_vector_type(4)));
        *reinterpret_cast<ushort4_t*>(key_cache + dst) =
            ushort4_t{f32_to_f16_bits(kk[0] * cs[0] - kk[1] * cs[1]), f32_to_f16_bits(kk[0] * cs[1] + kk[1] * cs[0]),
                      f32_to_f16_bits(kk[2] * cs[2] - kk[3] * cs[3]), f32_to_f16_bits(kk[2] * cs[3] + kk[3] * cs[2])};
        *reinterpret_cast<ushort4_t*>(value_cache + dst) =
            ushort4_t{f32_to_f16_bits(vv[0]), f32_to_f16_bits(vv[1]), f32_to_f16_bits(vv[2]), f32_to_f16_bits(vv[3])};
    }
}

// (hi, lo)[t][u] = (g * sigmoid(g)) * up (ops.cpp:78-87); rows t >= n_tokens are zero.
__global__ __launch_bounds__(256) void k_swiglu_split(const float* __restrict__ gate, const float* __restrict__ up,
                                                      half_t* __restrict__ hi, half_t* __restrict__ lo, int hidden,
                                                      int n_tokens) {
#pragma clang fp contract(off)
    const int t = blockIdx.y;
    const int u = blockIdx.x * blockDim.x + threadIdx.x;
    if (u >= hidden) return;
    const size_t at = static_cast<size_t>(t) * hidden + u;
    float out = 0.0f;
    if (t < n_tokens) {
        const float g = gate[at];
        const float sigma = 1.0f / (1.0f + expf(-g));
        out = (g * sigma) * up[at];
    }
    split_store(hi, lo, at, out);
}

// ---------------------------------------------------------------------------
// GEMM on the matrix cores: Y[t][f] (+)= sum_k W[f][k] * (Xh[t][k] + Xl[t][k])
// ---------------------------------------------------------------------------
//
// W is [n][K] binary16 row-major (a weight matrix as stored), Xh/Xl are [T][K]
// binary16 row-major, Y is [T][ldy] fp32.  n % 128 == 0, T % 128 == 0, K % 32 == 0.
// A workgroup of four wavefronts owns a square tile of 128 x 128 (kSub = 2: each wavefront
// a 64 x 64 quarter = 2 x 2 MFMA tiles of 32 x 32) or of 64 x 64 (kSub = 1) features x tokens;
// the smaller tile is used when the larger one would leave compute units without a workgroup.  Both operands have k as their
// contiguous dimension, so a lane reads its 8 k-values of a fragment row as one
// 16-byte load (the two halves of the wavefront take the two halves of a 16-wide
// k-step); the weight fragment is the A operand, the activations the B operand, and
// a lane ends up holding, for ONE token, 4 runs of 4 consecutive features per tile.
template <bool kAccumulate, int kSub>
__global__ __launch_bounds__(256) void k_gemm(const half_t* __restrict__ w, const half_t* __restrict__ xh,
                                              const half_t* __restrict__ xl, float* __restrict__ y, int K, int ldy) {
    const int lane = lane_id();
    const int wave = wave_index();
    constexpr int kWaveTile = 32 * kSub;  // a wavefront's square of the workgroup's (2 * kWaveTile)^2 tile
    const int f0 = blockIdx.x * (2 * kWaveTile) + (wave & 1) * kWaveTile;
    const int t0 = blockIdx.y * (2 * kWaveTile) + (wave >> 1) * kWaveTile;
    const int r = lane & 31, g = lane >> 5;
    const half_t* wrow[kSub];
    const half_t* hrow[kSub];
    const half_t* lrow[kSub];
#pragma unroll
    for (int i = 0; i < kSub; ++i) {
        wrow[i] = w + static_cast<size_t>(f0 + 32 * i + r) * K + 8 * g;
        hrow[i] = xh + static_cast<size_t>(t0 + 32 * i + r) * K + 8 * g;
        lrow[i] = xl + static_cast<size_t>(t0 + 32 * i + r) * K + 8 * g;
    }
    floatx16 acc[kSub][kSub];
#pragma unroll
    for (int i = 0; i < kSub; ++i)
#pragma unroll
        for (int j = 0; j < kSub; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // Two k-steps (32 columns) per trip: a lane's two 16-byte pieces of a row are 32 bytes apart, and a
    // row's 128-byte line is used up in two trips while it is still in the cache.  The fragments of the
    // next trip are requested before this trip's products are issued.
    struct Frags {
        half8_t a[2][kSub], bh[2][kSub], bl[2][kSub];
    };
    auto fetch = [&](Frags& f, int k0) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < kSub; ++i) {
                f.a[s][i] = *reinterpret_cast<const half8_t*>(wrow[i] + k0 + 16 * s);
                f.bh[s][i] = *reinterpret_cast<const half8_t*>(hrow[i] + k0 + 16 * s);
                f.bl[s][i] = *reinterpret_cast<const half8_t*>(lrow[i] + k0 + 16 * s);
            }
    };
    auto multiply = [&](const Frags& f) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < kSub; ++i)
#pragma unroll
                for (int j = 0; j < kSub; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[s][i], f.bh[s][j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[s][i], f.bl[s][j], acc[i][j], 0, 0, 0);
                }
    };
    Frags cur, nxt;
    fetch(cur, 0);
    for (int k0 = 32; k0 < K; k0 += 32) {
        fetch(nxt, k0);
        multiply(cur);
        cur = nxt;
    }
    multiply(cur);
    // D[m][n]: lane holds column n = lane % 32 (a token) and rows m = 8 * (e / 4) + 4 * (lane / 32) + e % 4 (features)
#pragma unroll
    for (int i = 0; i < kSub; ++i)
#pragma unroll
        for (int j = 0; j < kSub; ++j) {
            float* row = y + static_cast<size_t>(t0 + 32 * j + r) * ldy + f0 + 32 * i + 4 * g;
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                floatx4* dst = reinterpret_cast<floatx4*>(row + 8 * e4);
                floatx4 v = floatx4{acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]};
                if constexpr (kAccumulate) {
                    const floatx4 old = *dst;
                    v = floatx4{old[0] + v[0], old[1] + v[1], old[2] + v[2], old[3] + v[3]};
                }
                *dst = v;
            }
        }
}

// The same product as a pipeline of LDS stages filled by the memory system itself.
//
// A workgroup is eight wavefronts: four that multiply and four that only request data.  A request
// instruction holds its wavefront until the compute unit's memory pipeline has taken it (64 bytes
// a cycle: a trip's 64 KiB are 1000 cycles of that), and a wavefront that issues MFMAs cannot
// issue them while it is held, so the requests go out from wavefronts with nothing else to do;
// a SIMD runs one of each kind.
//
// The four multiplying wavefronts (2 x 2) own a tile of 64 kFi features x 64 kTj tokens; a wavefront
// owns 32 kFi x 32 kTj of it (kFi x kTj MFMA tiles: the weight side is the longer one, because the
// activations come twice, as head and remainder, and every fragment is read from LDS once per
// wavefront that uses it).  A trip covers kTripK columns (64 = a whole cache line per row and
// trip, or 32 where 64 would leave room for two stages only): the rows of the three operand
// tiles lie one after the other in a stage of LDS, and a requesting wavefront fills 1 KiB of it
// with one global_load_lds_dwordx4 (lane i -> 16 bytes at M0 + 16 i): no registers are staged
// and nothing waits for the data but the s_waitcnt ahead of the trip that multiplies it.  As
// many stages as 160 KiB hold, five at most.
//
// LDS banks: a fragment read takes 16 bytes per lane from 32 consecutive rows; with rows of 128
// (64) bytes every second (fourth) row starts in the same bank, so the 16-byte pieces of row r
// are stored in the order piece ^ ((r >> 1) & 7) (piece ^ ((r >> 2) & 3)): 16 consecutive lanes then
// cover all 64 banks once.  The permutation is applied on the way in, by the address each lane
// requests.
//
// The requests are inline assembly: written with the builtin, every LDS read of the loop would
// wait for all outstanding requests (they may alias), which is the pipeline's whole depth.
//
// kMode 0 stores the tile, 1 adds it to y, 2 is the feed-forward pair: the tile's weight rows are
// 32 kFi features of W1 (the wavefront's first kFi / 2 MFMA tiles) and the same features of W3
// (its last kFi / 2), and what is stored is (g * sigmoid(g)) * up (ops.cpp:78-87), split into
// binary16 head and remainder as the next product wants it.
struct PipeJob {
    const half_t* w[3];
    float* y[3];
    int ldy[3];
    int first_tile[3];  // first feature tile of matrix i (first_tile[0] = 0); unused entries = INT_MAX
    const half_t* xh;
    const half_t* xl;
    int K;      // row length of w and x
    int k_len;  // columns a workgroup multiplies: split z covers [z * k_len, (z + 1) * k_len) and writes y + z * split_stride
    size_t split_stride;
    int feature_tiles, token_tiles, groups;  // groups = feature_tiles * splits
    half_t* out_hi;                          // kMode 2: [tokens][out_ld]
    half_t* out_lo;
    int out_ld;
};

constexpr int kPipeTripK = 64;  // columns per trip of the narrow tiles; K must be a multiple

// (kLo: the activations' remainder tile travels and is multiplied too; without it a stage is a third smaller)
template <int kFi, int kTj, int kTripK, bool kLo = true>
struct PipeShape {
    static constexpr int kRowBytes = 2 * kTripK;
    static constexpr int kRowsA = 64 * kFi, kRowsB = 64 * kTj, kRows = kRowsA + (kLo ? 2 : 1) * kRowsB;
    static constexpr int kStageBytes = kRows * kRowBytes;
    static constexpr int kStages = (160 * 1024) / kStageBytes > 5 ? 5 : (160 * 1024) / kStageBytes;
    static constexpr int kLoads = kStageBytes / 4096;  // requests of 1 KiB per wavefront and stage
    static constexpr int kLdsBytes = kStages * kStageBytes;
};

template <int kCount>
__device__ __forceinline__ void wait_requests() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kCount) : "memory");
}

typedef _Float16 half4_pf_t __attribute__((ext_vector_type(4)));

// (hi, lo) = SwiGLU of four (gate, up) pairs, ops.cpp:78-87
__device__ __forceinline__ void swiglu_split4(half4_pf_t& hi, half4_pf_t& lo, const float* g, const float* u) {
#pragma clang fp contract(off)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float sigma = 1.0f / (1.0f + expf(-g[e]));  // (hardware exp and reciprocal here: 0.4 % of a prefill)
        const float v = (g[e] * sigma) * u[e];
        hi[e] = static_cast<half_t>(v);
        lo[e] = static_cast<half_t>(v - static_cast<float>(hi[e]));
    }
}

template <int kFi, int kTj, int kMode, int kTripK, bool kLo>
__global__ __launch_bounds__(512) void k_gemm_pipe(PipeJob job) {
    typedef PipeShape<kFi, kTj, kTripK, kLo> Shape;
    constexpr int kRowsA = Shape::kRowsA, kRowsB = Shape::kRowsB, kStages = Shape::kStages, kLoads = Shape::kLoads;
    constexpr int kStageBytes = Shape::kStageBytes, kRowBytes = Shape::kRowBytes;
    constexpr int kSteps = kTripK / 16;      // k-steps per trip
    constexpr int kPieces = kTripK / 8;      // 16-byte pieces of a row
    constexpr int kSwizzleShift = kPieces == 8 ? 1 : 2;
    extern __shared__ __align__(1024) char pipe_lds[];
    const int lane = lane_id();
    const int wave_of_8 = __builtin_amdgcn_readfirstlane(wave_index());
    const bool requester = wave_of_8 >= 4;
    const int wave = wave_of_8 & 3;  // which quarter of the tile (multiplying) or of the requests (requesting)
    // Workgroups are handed to the eight dies in turn: those that share a weight tile (same features
    // and columns, other tokens) get numbers that are equal modulo 8, so the tile crosses one die's L2.
    const int id = static_cast<int>(blockIdx.x), die = id & 7, within = id >> 3;
    const int group = (within / job.token_tiles) * 8 + die;
    if (group >= job.groups) return;
    const int token_tile = within % job.token_tiles;
    const int tile_all = group % job.feature_tiles, split = group / job.feature_tiles;
    const int which = tile_all >= job.first_tile[2] ? 2 : (tile_all >= job.first_tile[1] ? 1 : 0);
    const int tile_x = tile_all - (which == 2 ? job.first_tile[2] : (which == 1 ? job.first_tile[1] : 0));
    const half_t* __restrict__ w = which == 2 ? job.w[2] : (which == 1 ? job.w[1] : job.w[0]);
    const int K = job.K, k_first = split * job.k_len;
    const int r = lane & 31, g = lane >> 5;
    const int wf = wave & 1, wt = wave >> 1;
    constexpr int kFeaturesPerTile = kMode == 2 ? 32 * kFi : 64 * kFi;
    const int f_base = tile_x * kFeaturesPerTile, t_base = token_tile * kRowsB;

    // what each lane requests: request q of this wavefront fills 1 KiB = rows (64 / kPieces) (wave + 4 q) .. of a stage
    const char* src[kLoads];
#pragma unroll
    for (int q = 0; q < kLoads; ++q) {
        const int row = (64 / kPieces) * (wave + 4 * q) + lane / kPieces;
        const int piece = (lane % kPieces) ^ ((row >> kSwizzleShift) & (kPieces - 1));
        const half_t* from;
        if (row < kRowsA) {
            if constexpr (kMode == 2) {
                const int wave_rows = 32 * kFi, half_rows = 16 * kFi;
                const int owner = row / wave_rows, rem = row % wave_rows;
                const half_t* matrix = rem >= half_rows ? job.w[1] : job.w[0];
                from = matrix + static_cast<size_t>(f_base + owner * half_rows + rem % half_rows) * K;
            } else {
                from = w + static_cast<size_t>(f_base + row) * K;
            }
        } else if (!kLo || row < kRowsA + kRowsB) {
            from = job.xh + static_cast<size_t>(t_base + row - kRowsA) * K;
        } else {
            from = job.xl + static_cast<size_t>(t_base + row - kRowsA - kRowsB) * K;
        }
        src[q] = reinterpret_cast<const char*>(from + k_first) + 16 * piece;
    }
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) char*)pipe_lds));
    const int trips = job.k_len / kTripK;
    auto request = [&](int trip) {
        const unsigned at = __builtin_amdgcn_readfirstlane(lds_base + (trip % kStages) * kStageBytes + wave * 1024);
        const int column = __builtin_amdgcn_readfirstlane(trip * kRowBytes);
#pragma unroll
        for (int q = 0; q < kLoads; ++q)
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off\n" ::"v"(src[q] + column), "s"(at + q * 4096)
                         : "memory");
    };
    // where each lane reads its fragments: row r of an MFMA tile, pieces 2 s + g of k-step s
    int a_off[kSteps], b_off[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
        const int piece = (2 * s + g) ^ ((r >> kSwizzleShift) & (kPieces - 1));
        a_off[s] = (wf * 32 * kFi + r) * kRowBytes + 16 * piece;
        b_off[s] = (kRowsA + wt * 32 * kTj + r) * kRowBytes + 16 * piece;
    }

    floatx16 acc[kFi][kTj];
#pragma unroll
    for (int i = 0; i < kFi; ++i)
#pragma unroll
        for (int j = 0; j < kTj; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    struct Frags {
        half8_t a[kFi], bh[kTj], bl[kTj];
    };
    auto read = [&](Frags& f, int trip, int s) {
        const char* stage = pipe_lds + (trip % kStages) * kStageBytes;
#pragma unroll
        for (int i = 0; i < kFi; ++i) f.a[i] = *reinterpret_cast<const half8_t*>(stage + a_off[s] + i * 32 * kRowBytes);
#pragma unroll
        for (int j = 0; j < kTj; ++j) {
            f.bh[j] = *reinterpret_cast<const half8_t*>(stage + b_off[s] + j * 32 * kRowBytes);
            if constexpr (kLo) f.bl[j] = *reinterpret_cast<const half8_t*>(stage + b_off[s] + (kRowsB + j * 32) * kRowBytes);
        }
    };
    // (one half of a k-step's MFMAs: the weight tiles [kFi / 2 * half, kFi / 2 * (half + 1)))
    auto multiply_half = [&](const Frags& f, int half) {
#pragma unroll
        for (int i = kFi / 2 * half; i < kFi / 2 * (half + 1); ++i)
#pragma unroll
            for (int j = 0; j < kTj; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[i], f.bh[j], acc[i][j], 0, 0, 0);
                if constexpr (kLo) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[i], f.bl[j], acc[i][j], 0, 0, 0);
            }
    };
    // (requesting wavefronts) wait until the requests of `trip` have landed: those of later trips, at
    // most kStages - 2 of them, may be in flight
    auto landed = [&](int trip, int trips) {
        const int later = trips - 1 - trip;
        if (kStages > 2 && later >= kStages - 2) wait_requests<(kStages - 2) * kLoads>();
        else wait_requests<0>();
    };
    // One barrier per trip, inside the last k-step of the trip before: the requesting wavefronts
    // arrive when the trip's data has landed, the multiplying ones when they hold the last
    // fragments of the trip before in registers, which frees that trip's stage for the requests of
    // trip t + kStages.
    if (requester) {
#pragma unroll
        for (int t = 0; t < kStages - 1; ++t)
            if (t < trips) request(t);
        landed(0, trips);
        __syncthreads();
        if (kStages - 1 < trips) request(kStages - 1);
        for (int t = 0; t < trips; ++t) {
            landed(t + 1, trips);
            __syncthreads();
            if (t + kStages < trips) request(t + kStages);
        }
        return;
    }
    Frags frags[2];
    __syncthreads();
    read(frags[0], 0, 0);
    // The fragments of a k-step are read from LDS behind the first half of the MFMAs of the k-step
    // before and are waited for by the k-step after: the wait the compiler places is for every
    // read in flight, so none may be in flight that has not had half a k-step to arrive.
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const Frags& cur = frags[s & 1];
            Frags& next = frags[(s + 1) & 1];
            const bool last = s == kSteps - 1;
            multiply_half(cur, 0);
            __builtin_amdgcn_sched_barrier(0);
            // (after the last trip this reads a stage nobody uses: one path through the loop)
            if (last) __syncthreads();
            read(next, last ? t + 1 : t, last ? 0 : s + 1);
            __builtin_amdgcn_sched_barrier(0);
            multiply_half(cur, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // D[m][n]: a lane holds column n = lane % 32 (a token) and rows m = 8 (e / 4) + 4 (lane / 32) + e % 4 (features):
    // stored from there, an instruction would write 16 or 32 bytes to each of 32 rows of the output.  Every 32 x 32
    // tile therefore passes through LDS, [token][feature], and leaves as whole 128-byte lines, eight lanes to a
    // token's row.  The room is the wavefront's quarter of a stage that neither the last trip nor the read past
    // it uses; a wavefront's LDS accesses are served in order, so no barrier is needed between a tile's writes, its
    // reads and the next tile's writes.
    static_assert(kStages >= 3 && kStageBytes / 4 >= 32 * 144, "room for a transposed tile per wavefront");
    char* room = pipe_lds + ((trips + 1) % kStages) * kStageBytes + wave * (kStageBytes / 4);
    const int row8 = lane >> 3, part8 = lane & 7;
    if constexpr (kMode == 2) {
        static_assert(kFi == 4, "a wavefront's gate and up tiles: two of each");
        typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
        constexpr int kPitch = 72;  // binary16 per token row of the transposed tile: 64 features + padding
        half_t* tile = reinterpret_cast<half_t*>(room);
#pragma unroll
        for (int j = 0; j < kTj; ++j) {
            half4_t h[2][4], l[2][4];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const float gate[4] = {acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]};
                    const float up[4] = {acc[i + 2][j][4 * e4], acc[i + 2][j][4 * e4 + 1], acc[i + 2][j][4 * e4 + 2],
                                         acc[i + 2][j][4 * e4 + 3]};
                    swiglu_split4(h[i][e4], l[i][e4], gate, up);
                }
            const size_t at = static_cast<size_t>(t_base + wt * 32 * kTj + 32 * j) * job.out_ld + f_base + wf * 64 + 8 * part8;
#pragma unroll
            for (int part = 0; part < (kLo ? 2 : 1); ++part) {  // (without kLo the next GEMM reads no remainders either)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4)
                        *reinterpret_cast<half4_t*>(tile + r * kPitch + 32 * i + 8 * e4 + 4 * g) = part == 0 ? h[i][e4] : l[i][e4];
                half_t* out = part == 0 ? job.out_hi : job.out_lo;
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
                    const int n = 8 * pass + row8;
                    *reinterpret_cast<half8_t*>(out + at + static_cast<size_t>(n) * job.out_ld) =
                        *reinterpret_cast<const half8_t*>(tile + n * kPitch + 8 * part8);
                }
            }
        }
    } else {
        constexpr int kPitch = 36;  // floats per token row of the transposed tile: 32 features + padding
        float* tile = reinterpret_cast<float*>(room);
        float* __restrict__ y = (which == 2 ? job.y[2] : (which == 1 ? job.y[1] : job.y[0])) + static_cast<size_t>(split) * job.split_stride;
        const int ldy = which == 2 ? job.ldy[2] : (which == 1 ? job.ldy[1] : job.ldy[0]);
#pragma unroll
        for (int i = 0; i < kFi; ++i)
#pragma unroll
            for (int j = 0; j < kTj; ++j) {
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4)
                    *reinterpret_cast<floatx4*>(tile + r * kPitch + 8 * e4 + 4 * g) =
                        floatx4{acc[i][j][4 * e4], acc[i][j][4 * e4 + 1], acc[i][j][4 * e4 + 2], acc[i][j][4 * e4 + 3]};
                float* first = y + static_cast<size_t>(t_base + wt * 32 * kTj + 32 * j) * ldy + f_base + wf * 32 * kFi + 32 * i + 4 * part8;
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) {
                    const int n = 8 * pass + row8;
                    floatx4* out = reinterpret_cast<floatx4*>(first + static_cast<size_t>(n) * ldy);
                    floatx4 v = *reinterpret_cast<const floatx4*>(tile + n * kPitch + 4 * part8);
                    if constexpr (kMode == 1) {
                        const floatx4 old = *out;
                        v = floatx4{old[0] + v[0], old[1] + v[1], old[2] + v[2], old[3] + v[3]};
                    }
                    *out = v;
                }
            }
    }
}

// ---------------------------------------------------------------------------
// Causal attention over the cache
// ---------------------------------------------------------------------------
//
// One wavefront per (token t, KV head), four tokens to a workgroup: its query heads (gqa of
// them) attend to cache positions 0 .. pos0 + t (model.cpp:178-198; every row of the cache for these
// positions is in place, this chunk's included).  kGroup lanes share a position,
// 8 binary16 each; every lane group keeps a running maximum, sum and weighted V sum
// per query head (rescaled when the maximum grows), and the groups are merged by the
// same rule at the end.  Output: the heads' outputs, split into
// (hi, lo) for the output projection's GEMM.
// Sum over the kGroup lanes that share a position, by DPP moves (no LDS round trip).
template <int kGroup>
__device__ __forceinline__ float lanes_sum(float v) {
    static_assert(kGroup == 8 || kGroup == 16, "lane groups of 8 or 16");
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    if constexpr (kGroup == 16) v += dpp_move<kDppMirror>(v);
    return v;
}

// exp(x) as one hardware exponential (about an ulp off expf; the weights it forms are normalised
// by their own sum).
__device__ __forceinline__ float exp_fast(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }

template <int kGroup>
__global__ __launch_bounds__(256) void k_attention(const float* __restrict__ q, const uint16_t* __restrict__ key_cache,
                                                   const uint16_t* __restrict__ value_cache, half_t* __restrict__ out_hi,
                                                   half_t* __restrict__ out_lo, int layer, int pos0, int dim, int kv_dim,
                                                   int hs, int gqa, int seq_len, int n_tokens) {
    constexpr int kGroups = kWave / kGroup;  // positions a wavefront covers per pass
    const int lane = lane_id(), wave = wave_index();
    const int t = static_cast<int>(blockIdx.x) * 4 + wave, kvh = blockIdx.y;
    if (t >= n_tokens) return;  // (wavefronts of a workgroup do not meet again)
    const int npos = pos0 + t + 1;
    const int sub = lane % kGroup, grp = lane / kGroup;
    const bool lane_live = sub * 8 < hs;
    const int off = lane_live ? sub * 8 : 0;
    const size_t head_base = static_cast<size_t>(layer) * kv_dim * seq_len + static_cast<size_t>(kvh) * seq_len * hs;
    const uint16_t* kbase = key_cache + head_base;
    const uint16_t* vbase = value_cache + head_base;
    const float scale = 1.0f / sqrtf(static_cast<float>(hs));  // model.cpp:188

    float qreg[kMaxGqa][8];
    float top[kMaxGqa], lsum[kMaxGqa], acc[kMaxGqa][8];
#pragma unroll
    for (int h = 0; h < kMaxGqa; ++h) {
        top[h] = -INFINITY;
        lsum[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[h][e] = 0.0f;
            qreg[h][e] = (h < gqa && lane_live) ? q[static_cast<size_t>(t) * dim + (kvh * gqa + h) * hs + off + e] : 0.0f;
        }
    }
    // (the rows of the position after this one are requested before this one's arithmetic; past the end
    // the last valid row is read again and dropped)
    const int first = grp;
    const int clamp = npos - 1;
    uintx4 k_next = load16(kbase + static_cast<size_t>(first < npos ? first : clamp) * hs + off);
    uintx4 v_next = load16(vbase + static_cast<size_t>(first < npos ? first : clamp) * hs + off);
    for (int p = first; p < npos; p += kGroups) {
        const half8_t kh = as_half8(k_next);
        const half8_t vh = as_half8(v_next);
        const int pn = p + kGroups;
        k_next = load16(kbase + static_cast<size_t>(pn < npos ? pn : clamp) * hs + off);
        v_next = load16(vbase + static_cast<size_t>(pn < npos ? pn : clamp) * hs + off);
#pragma unroll
        for (int h = 0; h < kMaxGqa; ++h) {
            if (h < gqa) {
                float s = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) s = fmaf(static_cast<float>(kh[e]), qreg[h][e], s);
                s = lane_live ? s : 0.0f;
                s = lanes_sum<kGroup>(s) * scale;
                const float grown = fmaxf(top[h], s);
                const float corr = (top[h] == -INFINITY) ? 0.0f : exp_fast(top[h] - grown);
                const float pw = exp_fast(s - grown);
                top[h] = grown;
                lsum[h] = lsum[h] * corr + pw;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(static_cast<float>(vh[e]), pw, acc[h][e] * corr);
            }
        }
    }
    // lane groups of a wavefront
#pragma unroll
    for (int h = 0; h < kMaxGqa; ++h) {
        if (h < gqa) {
            float all = top[h];
#pragma unroll
            for (int o = kGroup; o < kWave; o <<= 1) all = fmaxf(all, __shfl_xor(all, o));
            const float f = (top[h] == -INFINITY) ? 0.0f : exp_fast(top[h] - all);
            float ls = lsum[h] * f;
#pragma unroll
            for (int o = kGroup; o < kWave; o <<= 1) ls += __shfl_xor(ls, o);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float v = acc[h][e] * f;
#pragma unroll
                for (int o = kGroup; o < kWave; o <<= 1) v += __shfl_xor(v, o);
                acc[h][e] = v;
            }
            if (grp == 0 && lane_live) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    split_store(out_hi, out_lo, static_cast<size_t>(t) * dim + (kvh * gqa + h) * hs + off + e, acc[h][e] / ls);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// The same attention on the matrix cores
// ---------------------------------------------------------------------------
//
// A workgroup owns 32 query rows = (32 / gqa) consecutive tokens x the gqa query heads of one KV
// head; its four wavefronts share the cache's blocks of 32 positions among them (wavefront w takes
// blocks w, w + 4, ..: a row's work is a chain of dependent steps per block, so the longest rows
// set the kernel's time), each with its own running maximum, sum and output, merged through
// LDS at the end.  Per block:
//   S^T[pos][row] = sum_d K[pos][d] Q[row][d]     A = K block (a lane's 8 d-values: one 16-byte
//                                                 load from the cache row), B = Q (head + remainder)
//   online softmax: in the result a LANE holds one query row (its column) and 16 of the block's 32
//                   positions, the lane 32 further on the other 16 -- maximum, sum and rescaling are
//                   per lane, with one exchange between the two halves of the wavefront
//   O^T[d][row] += sum_pos V^T[d][pos] P^T[pos][row]   A = V transposed: the wavefront loads its block of
//                                                      V as the cache holds it (a position's row at a
//                                                      time, 16 bytes a lane), writes it into a tile of
//                                                      LDS of its own with positions contiguous, and
//                                                      reads its fragments from there,
//                                                      B = P straight from the lane's own registers
// A lane's 16 positions of a block are {8j + 4g .. 8j + 4g + 3 : j = 0..3} (g = lane / 32), so as
// B operand of the second product it supplies, per 16-position step, positions 4g..4g+3 and
// 8+4g..8+4g+3; the V^T fragment is read in the same order (two 8-byte reads).  Any such
// permutation of k is fine as long as both operands use it.
// Probabilities and queries are split into binary16 head + remainder like every other activation.

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

template <int kHs, bool kLo>
__global__ __launch_bounds__(256) void k_attention_mfma(const float* __restrict__ q, const uint16_t* __restrict__ key_cache,
                                                        const uint16_t* __restrict__ value_cache, half_t* __restrict__ out_hi,
                                                        half_t* __restrict__ out_lo, int layer, int pos0, int dim, int kv_dim,
                                                        int gqa, int seq_len, int n_tokens) {
    constexpr int kDTiles = kHs / 32, kKSteps = kHs / 16;
    const int lane = lane_id(), wave = wave_index();
    const int r = lane & 31, g = lane >> 5;
    const int tokens_per_tile = 32 / gqa;
    // (the tiles with the longest contexts are dispatched first: where not all workgroups are resident at once, the
    // short ones fill the gaps at the end instead of the long ones starting last)
    const int t0 = static_cast<int>(gridDim.x - 1 - blockIdx.x) * tokens_per_tile;
    if (t0 >= n_tokens) return;  // (the whole workgroup)
    const int kvh = blockIdx.y;
    const int my_tok = t0 + r / gqa, my_head = r % gqa;
    const bool valid = my_tok < n_tokens;
    const int tok_c = valid ? my_tok : n_tokens - 1;
    const int last_tok = (t0 + tokens_per_tile < n_tokens ? t0 + tokens_per_tile : n_tokens) - 1;
    const int limit = pos0 + last_tok + 1;    // positions the tile reads: [0, limit)
    const int my_limit = pos0 + tok_c + 1;    // positions this lane's row attends to: [0, my_limit)
    const uint16_t* kbase = key_cache + static_cast<size_t>(layer) * kv_dim * seq_len + static_cast<size_t>(kvh) * seq_len * kHs;
    const uint16_t* vbase = value_cache + static_cast<size_t>(layer) * kv_dim * seq_len + static_cast<size_t>(kvh) * seq_len * kHs;
    // this wavefront's tile of the block's V rows, as the cache holds them: [32 positions][kHs], rows 16 bytes
    // longer than a cache row, so that the rows four positions apart, which the two halves of the wavefront read
    // side by side, start 16 banks apart
    constexpr int kTileRow = kHs + 8;  // binary16 per row
    __shared__ __align__(16) uint16_t vt_tiles[4][32 * kTileRow];
    uint16_t* vt_tile = vt_tiles[wave];
    constexpr int kVChunks = kHs / 16;  // 16-byte pieces of the block's V rows per lane
    const float scale = 1.0f / sqrtf(static_cast<float>(kHs));  // model.cpp:188

    // The K rows and the V rows of a wavefront's next block are requested a block ahead (the first block's
    // before q is read), so that they travel while this block is worked on.  (Four blocks ahead measures
    // slower: a block's time is its ~400 vector instructions, and the registers cost more than the wait.)
    auto fetch_k = [&](half8_t (&kf)[kKSteps], int p0) {
        const int prow = (p0 + r < seq_len) ? p0 + r : seq_len - 1;  // (rows past the tile's limit are masked below)
        const uint16_t* krow = kbase + static_cast<size_t>(prow) * kHs + 8 * g;
#pragma unroll
        for (int s = 0; s < kKSteps; ++s) kf[s] = as_half8(load16(krow + 16 * s));
    };
    // a block's V rows: piece c of the block = 8 dimensions of one position (zero past the context)
    auto fetch_v = [&](uintx4 (&vr)[kVChunks], int p0) {
#pragma unroll
        for (int i = 0; i < kVChunks; ++i) {
            const int c = lane + 64 * i, p = c / (kHs / 8), d0 = (c % (kHs / 8)) * 8;
            const int pos = p0 + p;
            vr[i] = pos < limit ? load16(vbase + static_cast<size_t>(pos) * kHs + d0) : uintx4{0u, 0u, 0u, 0u};
        }
    };
    half8_t k_next[kKSteps];
    uintx4 v_next[kVChunks];
    fetch_k(k_next, 32 * wave);
    fetch_v(v_next, 32 * wave);

    half8_t qh[kKSteps], ql[kKSteps];
    {
        const float* qrow = q + static_cast<size_t>(tok_c) * dim + (kvh * gqa + my_head) * kHs + 8 * g;
#pragma unroll
        for (int s = 0; s < kKSteps; ++s)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float v = qrow[16 * s + e];
                const half_t h = static_cast<half_t>(v);
                qh[s][e] = h;
                ql[s][e] = static_cast<half_t>(v - static_cast<float>(h));
            }
    }
    floatx16 o[kDTiles];
#pragma unroll
    for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] = 0.0f;
    float top = -INFINITY, lsum = 0.0f;

    for (int p0 = 32 * wave; p0 < limit; p0 += 128) {
        floatx16 st;
#pragma unroll
        for (int e = 0; e < 16; ++e) st[e] = 0.0f;
        half8_t kf[kKSteps];
#pragma unroll
        for (int s = 0; s < kKSteps; ++s) kf[s] = k_next[s];
        uintx4 vrows[kVChunks];
#pragma unroll
        for (int i = 0; i < kVChunks; ++i) vrows[i] = v_next[i];
        if (p0 + 128 < limit) {
            fetch_k(k_next, p0 + 128);
            fetch_v(v_next, p0 + 128);
        }
#pragma unroll
        for (int s = 0; s < kKSteps; ++s) {
            st = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], qh[s], st, 0, 0, 0);
            if constexpr (kLo) st = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], ql[s], st, 0, 0, 0);
        }
        float sv[16];
        float block_top = -INFINITY;
        if (p0 + 32 <= pos0 + t0 + 1) {  // (uniform) every row of the tile attends to the whole block: nothing to mask
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                sv[e] = st[e] * scale;
                block_top = fmaxf(block_top, sv[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int pos = p0 + 8 * (e >> 2) + 4 * g + (e & 3);
                sv[e] = (pos < my_limit) ? st[e] * scale : -INFINITY;
                block_top = fmaxf(block_top, sv[e]);
            }
        }
        block_top = fmaxf(block_top, __shfl_xor(block_top, 32));
        // The reference the exponentials are taken against follows the row's maximum lazily: it moves only when a
        // block's maximum exceeds it by more than kSlack (weights then stay below e^kSlack, far inside binary16, and
        // any reference gives the same quotient in the end).  After a row's first blocks it hardly ever moves, and a
        // block in which no row's reference moved skips the rescaling of the running sums and outputs altogether.
        constexpr float kSlack = 4.0f;
        const bool moves = block_top > top + kSlack;  // (true for the first block: top is -inf; finite from then on: position 0 is in every row's range)
        const float grown = moves ? block_top : top;
        const float corr = (top == -INFINITY) ? 0.0f : (moves ? exp_fast(top - grown) : 1.0f);
        const bool rescale = __builtin_amdgcn_ballot_w64(moves && top != -INFINITY) != 0ull;  // (uniform; outputs are still zero before the first block)
        half8_t ph[2], pl[2];
        float block_sum = 0.0f;
        // (a row that has seen nothing but masked positions so far keeps -inf as its reference: its weights are
        // exp(-inf - 0) = 0 instead of exp(-inf + inf))
        const float against = (grown == -INFINITY) ? 0.0f : grown;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const float pw = exp_fast(sv[e] - against);
            block_sum += pw;
            const half_t h = static_cast<half_t>(pw);
            ph[e >> 3][e & 7] = h;
            pl[e >> 3][e & 7] = static_cast<half_t>(pw - static_cast<float>(h));
        }
        block_sum += __shfl_xor(block_sum, 32);
        lsum = lsum * corr + block_sum;
        top = grown;
        // V rows into the tile, 16 bytes a lane (no two lanes of a quarter wavefront on one bank); the LDS serves a
        // wavefront's accesses in order, so the fragment reads below see them (and the next block's writes come
        // after these reads)
#pragma unroll
        for (int i = 0; i < kVChunks; ++i) {
            const int c = lane + 64 * i, p = c / (kHs / 8), d0 = (c % (kHs / 8)) * 8;
            *reinterpret_cast<uintx4*>(vt_tile + p * kTileRow + d0) = vrows[i];
        }
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt) {
            if (rescale) {
#pragma unroll
                for (int e = 0; e < 16; ++e) o[dt][e] *= corr;
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                // the fragment: dimension 32 dt + r at the eight positions this lane supplies, one 2-byte read each
                // (32 lanes read 64 consecutive bytes: every bank once per half wavefront)
                const half_t* vcol = reinterpret_cast<const half_t*>(vt_tile) + (16 * s2 + 4 * g) * kTileRow + 32 * dt + r;
                half8_t vf;
#pragma unroll
                for (int j = 0; j < 8; ++j) vf[j] = vcol[((j & 3) + 8 * (j >> 2)) * kTileRow];
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, ph[s2], o[dt], 0, 0, 0);
                if constexpr (kLo) o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pl[s2], o[dt], 0, 0, 0);
            }
        }
    }
    // merge: wavefronts 1..3 hand their (maximum, sum, output) to wavefront 0, lane for lane
    __shared__ float merge_o[3][kDTiles * 16][64];
    __shared__ float merge_ms[3][2][64];
    if (wave > 0) {
        merge_ms[wave - 1][0][lane] = top;
        merge_ms[wave - 1][1][lane] = lsum;
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) merge_o[wave - 1][dt * 16 + e][lane] = o[dt][e];
    }
    __syncthreads();
    if (wave > 0) return;
    float all_top = top;  // finite: block 0 is wavefront 0's and position 0 is in every row's range
#pragma unroll
    for (int w = 0; w < 3; ++w) all_top = fmaxf(all_top, merge_ms[w][0][lane]);
    const float own = exp_fast(top - all_top);
    lsum *= own;
#pragma unroll
    for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[dt][e] *= own;
#pragma unroll
    for (int w = 0; w < 3; ++w) {
        const float their_top = merge_ms[w][0][lane];
        const float weight = (their_top == -INFINITY) ? 0.0f : exp_fast(their_top - all_top);
        lsum += merge_ms[w][1][lane] * weight;
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[dt][e] += merge_o[w][dt * 16 + e][lane] * weight;
    }
    if (valid) {
        const size_t base = static_cast<size_t>(my_tok) * dim + (kvh * gqa + my_head) * kHs;
        const float inv_sum = 1.0f / lsum;
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                half4_t h, l;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float v = o[dt][4 * e4 + u] * inv_sum;
                    h[u] = static_cast<half_t>(v);
                    l[u] = static_cast<half_t>(v - static_cast<float>(h[u]));
                }
                *reinterpret_cast<half4_t*>(out_hi + base + 32 * dt + 8 * e4 + 4 * g) = h;
                if constexpr (kLo) *reinterpret_cast<half4_t*>(out_lo + base + 32 * dt + 8 * e4 + 4 * g) = l;
            }
    }
}

// x[i] (+)= p[0][i] + p[1][i] + ... in that order: the partial products of a GEMM whose K was split.
template <bool kAccumulate>
__global__ __launch_bounds__(256) void k_add_partials(float* __restrict__ x, const float* __restrict__ p, int splits,
                                                      size_t stride, size_t count) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
    if (i >= count) return;
    floatx4 v = kAccumulate ? *reinterpret_cast<const floatx4*>(x + i) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = 0; s < splits; ++s) {
        const floatx4 a = *reinterpret_cast<const floatx4*>(p + s * stride + i);
        v = floatx4{v[0] + a[0], v[1] + a[1], v[2] + a[2], v[3] + a[3]};
    }
    *reinterpret_cast<floatx4*>(x + i) = v;
}

// (hi, lo) = x as it is (the GEMM entry point's own inputs).
__global__ __launch_bounds__(256) void k_split(const float* __restrict__ x, half_t* __restrict__ hi, half_t* __restrict__ lo,
                                               size_t count) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) split_store(hi, lo, i, x[i]);
}

}  // namespace pf

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

namespace {

// Buffers of a chunk of t_pad tokens, in lpp_model::pf_buf order.
enum { kBufTokens, kBufX, kBufQ, kBufK, kBufV, kBufGate, kBufUp, kBufHi, kBufLo, kBufHi2, kBufLo2, kBufCount };
static_assert(kBufCount <= static_cast<int>(sizeof(lpp_model::pf_buf) / sizeof(void*)), "lpp_model::pf_buf is too small");

const char* unsupported_reason(const lpp_model* m) {
    const lpp_config& c = m->cfg;
    if (c.weight_precision != LPP_WEIGHT_FP16) return "weights are not binary16";
    if (c.dim % pf::kTileFeatures != 0 || m->kv_dim % pf::kTileFeatures != 0 || c.hidden_dim % pf::kTileFeatures != 0)
        return "dim, kv_dim and hidden_dim must be multiples of 128";
    if (m->head_size != 64 && m->head_size != 128) return "head_size must be 64 or 128";
    if (m->gqa > pf::kMaxGqa) return "more than 8 query heads per KV head";
    return nullptr;
}

lpp_status ensure_scratch(lpp_model* m, int t_pad) {
    if (m->pf_cap >= t_pad) return LPP_OK;
    prefill_release(m);
    const lpp_config& c = m->cfg;
    const size_t t = static_cast<size_t>(t_pad);
    const size_t widest = static_cast<size_t>(c.hidden_dim > c.dim ? c.hidden_dim : c.dim);
    const size_t bytes[kBufCount] = {t * sizeof(int),
                                     t * c.dim * sizeof(float),
                                     t * c.dim * sizeof(float),
                                     t * m->kv_dim * sizeof(float),
                                     t * m->kv_dim * sizeof(float),
                                     t * c.hidden_dim * sizeof(float),
                                     t * c.hidden_dim * sizeof(float),
                                     t * widest * sizeof(pf::half_t),
                                     t * widest * sizeof(pf::half_t),
                                     // the feed-forward activations, written while hi/lo are still being read
                                     t * c.hidden_dim * sizeof(pf::half_t),
                                     t * c.hidden_dim * sizeof(pf::half_t)};
    for (int i = 0; i < kBufCount; ++i) {
        lpp_status st = lpp_malloc(&m->pf_buf[i], bytes[i]);
        if (st != LPP_OK) {
            prefill_release(m);
            return st;
        }
    }
    m->pf_cap = t_pad;
    return LPP_OK;
}

// Y_i[t][f] (+)= sum_k W_i[f][k] * x[t][k] for up to three matrices W_i of n_i rows that share x.
struct Product {
    const void* w;
    float* y;
    int n;
};

// The kernel's LDS need, told to the runtime once per device (the attribute belongs to the device's copy of the kernel).
template <int kFi, int kTj, int kMode, int kTripK, bool kLo = true>
lpp_status size_pipe() {
    static bool sized[64] = {};
    int device = 0;
    LPP_HIP(hipGetDevice(&device));
    if (device < 0 || device >= 64 || !sized[device]) {
        LPP_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(&pf::k_gemm_pipe<kFi, kTj, kMode, kTripK, kLo>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, pf::PipeShape<kFi, kTj, kTripK, kLo>::kLdsBytes));
        if (device >= 0 && device < 64) sized[device] = true;
    }
    return LPP_OK;
}

template <int kFi, int kTj, int kMode, int kTripK, bool kLo>
lpp_status launch_pipe_as(const pf::PipeJob& job, hipStream_t s) {
    typedef pf::PipeShape<kFi, kTj, kTripK, kLo> Shape;
    LPP_TRY((size_pipe<kFi, kTj, kMode, kTripK, kLo>()));
    const int per_die = (job.groups + 7) / 8;
    hipLaunchKernelGGL((pf::k_gemm_pipe<kFi, kTj, kMode, kTripK, kLo>), dim3(per_die * 8 * job.token_tiles), dim3(512), Shape::kLdsBytes, s, job);
    LPP_CHECK_LAUNCH("k_gemm_pipe");
    return LPP_OK;
}
// (a job without a remainder array takes the kernels that neither fetch nor multiply one)
template <int kFi, int kTj, int kMode, int kTripK = pf::kPipeTripK>
lpp_status launch_pipe(const pf::PipeJob& job, hipStream_t s) {
    return job.xl != nullptr ? launch_pipe_as<kFi, kTj, kMode, kTripK, true>(job, s) : launch_pipe_as<kFi, kTj, kMode, kTripK, false>(job, s);
}

// `partials` (optional, partial_floats long): room for the partial products of a split K.  A product
// with too few output tiles for the compute units is cut along K into ranges, each multiplied by
// its own workgroups into `partials`: range z of matrix i lies at partials + z * t_pad * (n_0 + n_1 +
// ..) + t_pad * (n_0 + .. + n_(i-1)), rows of n_i floats.  With `left_split` the caller adds the
// ranges itself (in order, in the kernel that reads the product next) and gets their number there;
// without it they are added to y here, in order.
lpp_status gemm(const Product* prods, int count, const pf::half_t* xh, const pf::half_t* xl, int K, int t_pad, bool accumulate,
                hipStream_t s, float* partials = nullptr, size_t partial_floats = 0, int* left_split = nullptr,
                bool remainder = true) {
    LPP_REQUIRE(count >= 1 && count <= 3 && t_pad % pf::kTileTokens == 0 && K % 32 == 0, "prefill GEMM: %d products, K %d, T %d",
                count, K, t_pad);
    if (left_split != nullptr) *left_split = 1;
    int total_n = 0;
    bool wide = true;  // every matrix a whole number of 256-row tiles
    for (int i = 0; i < count; ++i) {
        LPP_REQUIRE(prods[i].n > 0 && prods[i].n % pf::kTileFeatures == 0, "prefill GEMM: n %d", prods[i].n);
        total_n += prods[i].n;
        wide = wide && prods[i].n % 256 == 0;
    }
    const bool staged = K % pf::kPipeTripK == 0 && test_option(LPP_OPT_PREFILL_STAGED_GEMM) != 0;
    if (staged) {
        const int token_tiles = t_pad / pf::kTileTokens;
        wide = wide && (total_n / 256) * token_tiles >= compute_units() && test_option(LPP_OPT_PREFILL_WIDE_TILES) != 0;
        const int tile = wide ? 256 : 128;
        const int feature_tiles = total_n / tile;
        const size_t stride = static_cast<size_t>(t_pad) * total_n;
        int splits = 1;
        if (partials != nullptr && (count == 1 || left_split != nullptr)) {
            while (splits < 8 && feature_tiles * token_tiles * splits * 2 <= compute_units() &&
                   K % (2 * pf::kPipeTripK * splits) == 0 && K / (2 * splits) >= 512 && stride * 2 * splits <= partial_floats)
                splits *= 2;
        }
        pf::PipeJob job = {};
        int at = 0;
        size_t before = 0;
        for (int i = 0; i < 3; ++i) {
            const Product& p = prods[i < count ? i : count - 1];
            job.w[i] = static_cast<const pf::half_t*>(p.w);
            job.y[i] = splits > 1 ? partials + before : p.y;
            job.ldy[i] = p.n;
            job.first_tile[i] = i < count ? at : 0x7fffffff;
            if (i < count) {
                at += p.n / tile;
                before += static_cast<size_t>(t_pad) * p.n;
            }
        }
        job.xh = xh;
        job.xl = remainder ? xl : nullptr;  // (without: the kernels that neither fetch nor multiply the remainder)
        job.K = K;
        job.k_len = K / splits;
        job.split_stride = stride;
        job.feature_tiles = feature_tiles;
        job.token_tiles = token_tiles;
        job.groups = feature_tiles * splits;
        const bool add_in_kernel = accumulate && splits == 1;
        if (wide) {
            if (add_in_kernel) LPP_TRY((launch_pipe<4, 2, 1, 32>(job, s)));
            else LPP_TRY((launch_pipe<4, 2, 0, 32>(job, s)));
        } else {
            if (add_in_kernel) LPP_TRY((launch_pipe<2, 2, 1>(job, s)));
            else LPP_TRY((launch_pipe<2, 2, 0>(job, s)));
        }
        if (splits > 1 && left_split != nullptr) {
            *left_split = splits;
        } else if (splits > 1) {
            if (accumulate)
                hipLaunchKernelGGL(pf::k_add_partials<true>, dim3(static_cast<unsigned>((stride / 4 + 255) / 256)), dim3(256), 0, s,
                                   prods[0].y, partials, splits, stride, stride);
            else
                hipLaunchKernelGGL(pf::k_add_partials<false>, dim3(static_cast<unsigned>((stride / 4 + 255) / 256)), dim3(256), 0, s,
                                   prods[0].y, partials, splits, stride, stride);
            LPP_CHECK_LAUNCH("k_add_partials");
        }
        return LPP_OK;
    }
    const bool large_tiles = (total_n / pf::kTileFeatures) * (t_pad / pf::kTileTokens) >= compute_units();
    const int tile = large_tiles ? pf::kTileFeatures : 64;
    // fragments straight from memory: one launch per matrix
    for (int i = 0; i < count; ++i) {
        const pf::half_t* wh = static_cast<const pf::half_t*>(prods[i].w);
        const dim3 grid(prods[i].n / tile, t_pad / tile);
        float* y = prods[i].y;
        const int ldy = prods[i].n;
        if (large_tiles) {
            if (accumulate) hipLaunchKernelGGL((pf::k_gemm<true, 2>), grid, dim3(256), 0, s, wh, xh, xl, y, K, ldy);
            else hipLaunchKernelGGL((pf::k_gemm<false, 2>), grid, dim3(256), 0, s, wh, xh, xl, y, K, ldy);
        } else {
            if (accumulate) hipLaunchKernelGGL((pf::k_gemm<true, 1>), grid, dim3(256), 0, s, wh, xh, xl, y, K, ldy);
            else hipLaunchKernelGGL((pf::k_gemm<false, 1>), grid, dim3(256), 0, s, wh, xh, xl, y, K, ldy);
        }
        LPP_CHECK_LAUNCH("k_gemm");
    }
    return LPP_OK;
}

// (remainders false: nobody reads lo after this norm, and the wide kernel leaves it unwritten)
lpp_status norm_split(float* x, const float* gain, pf::half_t* hi, pf::half_t* lo, int dim, int n, int t_pad, const float* partials,
                      int splits, size_t split_stride, hipStream_t s, bool remainders = true) {
    pf::half_t* lo_wide = remainders ? lo : nullptr;
#define LPP_NORM_WIDE(PER, SPLITS) \
    hipLaunchKernelGGL((pf::k_norm_split_wide<PER, SPLITS>), dim3(t_pad), dim3(256), 0, s, x, gain, hi, lo_wide, n, partials, split_stride)
#define LPP_NORM_WIDE_DIM(PER)          \
    switch (splits) {                   \
        case 0: LPP_NORM_WIDE(PER, 0); break; \
        case 2: LPP_NORM_WIDE(PER, 2); break; \
        case 4: LPP_NORM_WIDE(PER, 4); break; \
        default: LPP_NORM_WIDE(PER, 8); break; \
    }
    // (gemm() cuts K into 1, 2, 4 or 8 ranges)
    const bool wide = (dim == 1024 || dim == 2048 || dim == 4096) && (splits == 0 || splits == 2 || splits == 4 || splits == 8);
    if (wide && dim == 1024) {
        LPP_NORM_WIDE_DIM(1)
    } else if (wide && dim == 2048) {
        LPP_NORM_WIDE_DIM(2)
    } else if (wide) {
        LPP_NORM_WIDE_DIM(4)
    } else {
        hipLaunchKernelGGL(pf::k_norm_split, dim3(t_pad), dim3(256), 0, s, x, gain, hi, lo, dim, n, partials, splits, split_stride);
    }
#undef LPP_NORM_WIDE_DIM
#undef LPP_NORM_WIDE
    LPP_CHECK_LAUNCH("k_norm_split");
    return LPP_OK;
}

// (hi, lo)[t][u] = SwiGLU(W1 x[t], W3 x[t])[u] in one launch: the gate and the up projection of a
// feature share a workgroup, and the activation is applied to the accumulators.
lpp_status gate_up_swiglu(const void* w1, const void* w3, int hidden, const pf::half_t* xh, const pf::half_t* xl, int K, int t_pad,
                          pf::half_t* out_hi, pf::half_t* out_lo, hipStream_t s, bool remainder) {
    pf::PipeJob job = {};
    job.w[0] = static_cast<const pf::half_t*>(w1);
    job.w[1] = static_cast<const pf::half_t*>(w3);
    job.w[2] = job.w[1];
    job.first_tile[0] = 0;
    job.first_tile[1] = job.first_tile[2] = 0x7fffffff;
    job.xh = xh;
    job.xl = remainder ? xl : nullptr;
    job.K = K;
    job.k_len = K;
    job.feature_tiles = hidden / 128;  // 128 features a tile: 128 rows of W1 and the same 128 of W3
    job.token_tiles = t_pad / pf::kTileTokens;
    job.groups = job.feature_tiles;
    job.out_hi = out_hi;
    job.out_lo = out_lo;
    job.out_ld = hidden;
    return launch_pipe<4, 2, 2, 32>(job, s);
}

// One chunk: tokens[0..n) at positions pos0 .. pos0 + n - 1; n <= kChunk.
lpp_status prefill_chunk(lpp_model* m, const int* tokens, int n, int pos0) {
    const lpp_config& c = m->cfg;
    const int dim = c.dim, kv = m->kv_dim, hidden = c.hidden_dim, hs = m->head_size;
    const int t_pad = (n + pf::kTileTokens - 1) / pf::kTileTokens * pf::kTileTokens;
    LPP_TRY(ensure_scratch(m, t_pad));
    hipStream_t s = stream();
    int* d_tokens = static_cast<int*>(m->pf_buf[kBufTokens]);
    float* x = static_cast<float*>(m->pf_buf[kBufX]);
    float* q = static_cast<float*>(m->pf_buf[kBufQ]);
    float* k = static_cast<float*>(m->pf_buf[kBufK]);
    float* v = static_cast<float*>(m->pf_buf[kBufV]);
    float* gate = static_cast<float*>(m->pf_buf[kBufGate]);
    float* up = static_cast<float*>(m->pf_buf[kBufUp]);
    pf::half_t* hi = static_cast<pf::half_t*>(m->pf_buf[kBufHi]);
    pf::half_t* lo = static_cast<pf::half_t*>(m->pf_buf[kBufLo]);
    LPP_HIP(hipMemcpyAsync(d_tokens, tokens, static_cast<size_t>(n) * sizeof(int), hipMemcpyHostToDevice, s));
    hipLaunchKernelGGL(pf::k_embed, dim3(n), dim3(256), 0, s, static_cast<const float*>(m->w[LPP_T_TOKEN_EMBEDDING]), d_tokens,
                       x, dim);
    LPP_CHECK_LAUNCH("k_embed");
    const size_t wb = sizeof(pf::half_t);
    auto layer_of = [&](int t, int l, size_t rows, size_t cols) {
        return static_cast<const char*>(m->w[t]) + static_cast<size_t>(l) * rows * cols * wb;
    };
    pf::half_t* hi2 = static_cast<pf::half_t*>(m->pf_buf[kBufHi2]);
    pf::half_t* lo2 = static_cast<pf::half_t*>(m->pf_buf[kBufLo2]);
    // The fp32 gate and up buffers double as room for the partial products of the GEMMs whose K is
    // split (each is t_pad * hidden floats): up for Wq/Wk/Wv, gate for Wo and then for W2.
    const size_t room = static_cast<size_t>(t_pad) * hidden;
    // LPP_PREFILL_EXACT: every product takes the activations as binary16 head + remainder.  LPP_PREFILL_FAST: the head
    // alone, in the staged kernels (what a GEMM sees of its input is then what the reference's own GPU GEMV sees,
    // matmul.cu:85-98; accumulation stays fp32).
    const bool exact = m->pf_mode != LPP_PREFILL_FAST;
    const bool fused_ffn = dim % pf::kPipeTripK == 0 && hidden % 128 == 0 && test_option(LPP_OPT_PREFILL_STAGED_GEMM) != 0 &&
                           test_option(LPP_OPT_PREFILL_FUSED_FFN) != 0;
    // Nobody reads a remainder when every GEMM of the chain is a staged one in the fast mode: the kernels that produce
    // activations then leave the remainders unwritten.  (The direct GEMM, taken for other shapes, always reads them.)
    const bool lean = !exact && fused_ffn;
    int pending = 0;  // ranges of the product before (W2's, then Wo's) still to be added to x
    for (int l = 0; l < c.n_layers; ++l) {
        // attention block, model.cpp:216-218
        LPP_TRY(norm_split(x, static_cast<const float*>(m->w[LPP_T_RMS_ATT]) + static_cast<size_t>(l) * dim, hi, lo, dim, n, t_pad, gate,
                           pending > 1 ? pending : 0, static_cast<size_t>(t_pad) * dim, s, !lean));
        // What a prefill leaves behind is the cache: the last layer needs its K and V rows only, and
        // nothing reads what the rest of that layer would compute.
        const bool last_layer = l == c.n_layers - 1;
        const Product qkv[3] = {{layer_of(LPP_T_WQ, l, dim, dim), q, dim}, {layer_of(LPP_T_WK, l, kv, dim), k, kv},
                                {layer_of(LPP_T_WV, l, kv, dim), v, kv}};
        const int q_dim = last_layer ? 0 : dim;
        int qkv_split = 1;
        LPP_TRY(gemm(qkv + (last_layer ? 1 : 0), last_layer ? 2 : 3, hi, lo, dim, t_pad, false, s, up, room, &qkv_split, exact));
        const size_t qkv_stride = static_cast<size_t>(t_pad) * (q_dim + 2 * kv);
        const float* qs = qkv_split > 1 ? up : q;
        const float* ks = qkv_split > 1 ? up + static_cast<size_t>(t_pad) * q_dim : k;
        const float* vs = qkv_split > 1 ? up + static_cast<size_t>(t_pad) * (q_dim + kv) : v;
        hipLaunchKernelGGL(pf::k_rope_scatter, dim3(n), dim3(256), 0, s, q, qs, ks, vs, m->rope, m->key_cache, m->value_cache, l,
                           pos0, q_dim, kv, hs, c.seq_len, qkv_split, qkv_stride);
        LPP_CHECK_LAUNCH("k_rope_scatter");
        if (last_layer) break;
        // (rows n .. t_pad of hi/lo are still the zeros k_norm_split wrote: the attention writes rows < n only)
        const bool matrix_cores = 32 % m->gqa == 0 && test_option(LPP_OPT_PREFILL_MFMA_ATTENTION) != 0;
        if (matrix_cores) {
            const int tiles = (n + 32 / m->gqa - 1) / (32 / m->gqa);
            const dim3 grid(tiles, c.n_kv_heads);
#define LPP_PF_ATTENTION(HS, LO)                                                                                          \
    hipLaunchKernelGGL((pf::k_attention_mfma<HS, LO>), grid, dim3(256), 0, s, q, m->key_cache, m->value_cache, hi, lo, l, pos0, \
                       dim, kv, m->gqa, c.seq_len, n)
            // (the fast mode rounds q and the softmax weights to binary16 as it rounds every GEMM input)
            if (hs == 64) {
                if (!lean) LPP_PF_ATTENTION(64, true);
                else LPP_PF_ATTENTION(64, false);
            } else {
                if (!lean) LPP_PF_ATTENTION(128, true);
                else LPP_PF_ATTENTION(128, false);
            }
#undef LPP_PF_ATTENTION
            LPP_CHECK_LAUNCH("k_attention_mfma");
        } else if (hs == 64)
            hipLaunchKernelGGL(pf::k_attention<8>, dim3((n + 3) / 4, c.n_kv_heads), dim3(256), 0, s, q, m->key_cache,
                               m->value_cache, hi, lo, l, pos0, dim, kv, hs, m->gqa, c.seq_len, n);
        else
            hipLaunchKernelGGL(pf::k_attention<16>, dim3((n + 3) / 4, c.n_kv_heads), dim3(256), 0, s, q, m->key_cache,
                               m->value_cache, hi, lo, l, pos0, dim, kv, hs, m->gqa, c.seq_len, n);
        LPP_CHECK_LAUNCH("k_attention");
        const Product wo = {layer_of(LPP_T_WO, l, dim, dim), x, dim};
        LPP_TRY(gemm(&wo, 1, hi, lo, dim, t_pad, true, s, gate, room, &pending, exact));
        // feed-forward block, model.cpp:221-226
        LPP_TRY(norm_split(x, static_cast<const float*>(m->w[LPP_T_RMS_FFN]) + static_cast<size_t>(l) * dim, hi, lo, dim, n, t_pad, gate,
                           pending > 1 ? pending : 0, static_cast<size_t>(t_pad) * dim, s, !lean));
        if (fused_ffn) {
            LPP_TRY(gate_up_swiglu(layer_of(LPP_T_W1, l, hidden, dim), layer_of(LPP_T_W3, l, hidden, dim), hidden, hi, lo, dim, t_pad,
                                   hi2, lo2, s, exact));
        } else {
            const Product gate_up[2] = {{layer_of(LPP_T_W1, l, hidden, dim), gate, hidden}, {layer_of(LPP_T_W3, l, hidden, dim), up, hidden}};
            LPP_TRY(gemm(gate_up, 2, hi, lo, dim, t_pad, false, s, nullptr, 0, nullptr, exact));
            hipLaunchKernelGGL(pf::k_swiglu_split, dim3((hidden + 255) / 256, t_pad), dim3(256), 0, s, gate, up, hi2, lo2, hidden, n);
            LPP_CHECK_LAUNCH("k_swiglu_split");
        }
        const Product w2 = {layer_of(LPP_T_W2, l, dim, hidden), x, dim};
        LPP_TRY(gemm(&w2, 1, hi2, lo2, hidden, t_pad, true, s, gate, room, &pending, exact));
    }
    LPP_HIP(hipStreamSynchronize(s));
    return LPP_OK;
}

}  // namespace

void prefill_release(lpp_model* m) {
    for (void*& p : m->pf_buf) {
        lpp_free(p);
        p = nullptr;
    }
    m->pf_cap = 0;
}

}  // namespace lpp

extern "C" {

lpp_status lpp_model_set_prefill_mode(lpp_model* m, int mode) {
    LPP_REQUIRE(m != nullptr && (mode == LPP_PREFILL_EXACT || mode == LPP_PREFILL_FAST), "lpp_model_set_prefill_mode: mode %d", mode);
    m->pf_mode = mode;
    return LPP_OK;
}

lpp_status lpp_prefill_supported(const lpp_model* m) {
    LPP_REQUIRE(m != nullptr, "lpp_prefill_supported: null model");
    const char* why = lpp::unsupported_reason(m);
    if (why != nullptr) return lpp::fail(LPP_ERR_UNSUPPORTED, "batched prefill unavailable: %s", why);
    return LPP_OK;
}

lpp_status lpp_prefill(lpp_model* m, const int* tokens, int n_tokens, int start_pos) {
    using namespace lpp;
    LPP_REQUIRE(m != nullptr && tokens != nullptr, "lpp_prefill: null argument");
    LPP_REQUIRE(n_tokens >= 0 && start_pos >= 0 && start_pos + n_tokens <= m->cfg.seq_len,
                "lpp_prefill: positions [%d, %d) outside [0, %d)", start_pos, start_pos + n_tokens, m->cfg.seq_len);
    for (int i = 0; i < n_tokens; ++i)
        LPP_REQUIRE(tokens[i] >= 0 && tokens[i] < m->cfg.vocab_size, "lpp_prefill: token %d at %d outside [0, %d)", tokens[i], i,
                    m->cfg.vocab_size);
    for (int t = 0; t < LPP_T_COUNT; ++t)
        if (!m->w_loaded[t]) return fail(LPP_ERR_STATE, "weight tensor %d has not been uploaded", t);
    LPP_TRY(lpp_prefill_supported(m));
    for (int done = 0; done < n_tokens; done += pf::kChunk) {
        const int n = n_tokens - done < pf::kChunk ? n_tokens - done : pf::kChunk;
        LPP_TRY(prefill_chunk(m, tokens + done, n, start_pos + done));
    }
    return LPP_OK;
}

lpp_status lpp_prefill_gemm(float* d_y, const void* d_w, const float* d_x, int n, int k, int n_tokens, int accumulate) {
    using namespace lpp;
    LPP_REQUIRE(d_y && d_w && d_x, "lpp_prefill_gemm: null argument");
    LPP_REQUIRE(n_tokens > 0 && n_tokens % pf::kTileTokens == 0, "lpp_prefill_gemm: n_tokens %d not a positive multiple of %d",
                n_tokens, pf::kTileTokens);
    LPP_REQUIRE(n > 0 && n % pf::kTileFeatures == 0 && k > 0 && k % 32 == 0, "lpp_prefill_gemm: n %d k %d", n, k);
    hipStream_t s = stream();
    void* hi = nullptr;
    void* lo = nullptr;
    const size_t count = static_cast<size_t>(n_tokens) * k;
    LPP_TRY(lpp_malloc(&hi, count * sizeof(pf::half_t)));
    lpp_status st = lpp_malloc(&lo, count * sizeof(pf::half_t));
    if (st == LPP_OK) {
        hipLaunchKernelGGL(pf::k_split, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s, d_x,
                           static_cast<pf::half_t*>(hi), static_cast<pf::half_t*>(lo), count);
        const Product one = {d_w, d_y, n};
        st = gemm(&one, 1, static_cast<pf::half_t*>(hi), static_cast<pf::half_t*>(lo), k, n_tokens, accumulate != 0, s);
        if (hipStreamSynchronize(s) != hipSuccess && st == LPP_OK) st = fail(LPP_ERR_HIP, "lpp_prefill_gemm: kernel failed");
    }
    lpp_free(hi);
    lpp_free(lo);
    return st;
}

}  // extern "C"

// ---------------------------------------------------------------------------
// The same product for callers that cannot allocate
// ---------------------------------------------------------------------------

namespace lpp {
namespace {

// Room for the binary16 head and remainder of the activations: kNoAllocElements each.
constexpr size_t kNoAllocElements = size_t{1} << 21;
static __device__ __align__(256) unsigned char scratch[2 * kNoAllocElements * sizeof(pf::half_t)];

// Device address of `scratch` per device.  In host code the array's name is only a handle
// for hipGetSymbolAddress; every device that loads the library holds its own copy.
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};

lpp_status scratch_address(void** out) {
    int device = -1;
    LPP_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(LPP_ERR_UNSUPPORTED, "device ordinal %d beyond %d", device, kMaxDevices - 1);
    if (g_scratch_ptr[device] == nullptr) {
        void* p = nullptr;
        LPP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (p == nullptr) return fail(LPP_ERR_HIP, "hipGetSymbolAddress returned no address for the prefill scratch");
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return LPP_OK;
}

}  // namespace

namespace {
// What the set-up returned on each device: 0 not run yet, 1 done, 2 failed (message kept).
int g_setup_state[kMaxDevices] = {};
char g_setup_message[kMaxDevices][256] = {};

lpp_status run_scratch_setup() {
    LPP_TRY((size_pipe<4, 2, 0, 32>()));
    LPP_TRY((size_pipe<4, 2, 1, 32>()));
    LPP_TRY((size_pipe<2, 2, 0, pf::kPipeTripK>()));
    LPP_TRY((size_pipe<2, 2, 1, pf::kPipeTripK>()));
    void* p = nullptr;
    return scratch_address(&p);
}
}  // namespace

lpp_status prefill_gemm_scratch_setup() {
    // (everything the allocation-free entry point would otherwise set up on its first call: a caller under
    // graph capture finds it done)
    int device = -1;
    LPP_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(LPP_ERR_UNSUPPORTED, "device ordinal %d beyond %d", device, kMaxDevices - 1);
    const lpp_status st = run_scratch_setup();
    g_setup_state[device] = st == LPP_OK ? 1 : 2;
    if (st != LPP_OK) std::snprintf(g_setup_message[device], sizeof g_setup_message[device], "%s", lpp_last_error());
    return st;
}

// The set-up's outcome on the current device; runs it if this is the first call on the device.
static lpp_status prefill_gemm_scratch_status() {
    int device = -1;
    LPP_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(LPP_ERR_UNSUPPORTED, "device ordinal %d beyond %d", device, kMaxDevices - 1);
    if (g_setup_state[device] == 0) return prefill_gemm_scratch_setup();
    if (g_setup_state[device] == 2)
        return fail(LPP_ERR_HIP, "lpp_prefill_gemm_noalloc: set-up failed on this device: %s", g_setup_message[device]);
    return LPP_OK;
}

}  // namespace lpp

extern "C" {

lpp_status lpp_prefill_gemm_noalloc(float* d_y, const void* d_w, const float* d_x, int n, int k, int n_tokens, int accumulate) {
    using namespace lpp;
    LPP_REQUIRE(d_y && d_w && d_x, "lpp_prefill_gemm_noalloc: null argument");
    LPP_REQUIRE(n_tokens > 0 && n_tokens % pf::kTileTokens == 0, "lpp_prefill_gemm_noalloc: n_tokens %d not a positive multiple of %d",
                n_tokens, pf::kTileTokens);
    LPP_REQUIRE(n > 0 && n % pf::kTileFeatures == 0 && k > 0 && k % 32 == 0, "lpp_prefill_gemm_noalloc: n %d k %d", n, k);
    const size_t count = static_cast<size_t>(n_tokens) * k;
    LPP_REQUIRE(count <= kNoAllocElements, "lpp_prefill_gemm_noalloc: n_tokens * k = %zu exceeds the built-in scratch of %zu elements",
                count, kNoAllocElements);
    hipStream_t s = stream();
    LPP_TRY(prefill_gemm_scratch_status());
    void* base = nullptr;
    LPP_TRY(scratch_address(&base));
    pf::half_t* hi = static_cast<pf::half_t*>(base);
    pf::half_t* lo = hi + kNoAllocElements;
    hipLaunchKernelGGL(pf::k_split, dim3(static_cast<unsigned>((count + 255) / 256)), dim3(256), 0, s, d_x, hi, lo, count);
    LPP_CHECK_LAUNCH("k_split");
    const Product one = {d_w, d_y, n};
    return gemm(&one, 1, hi, lo, k, n_tokens, accumulate != 0, s);
}

}  // extern "C"
