// decode_phases.hpp -- the per-token schedule of forward() (reference
// src/model.cpp:342-371 -> transformer_block :205-226 -> attention :121-160) cut
// into phases.  Between two phases every workgroup needs results of all others
// (a full activation vector); inside a phase workgroups are independent.
//
//   qkv      rmsnorm(x)        -> q,k,v GEMV -> RoPE -> q buffer, K/V cache  (fuses :216,:133-141)
//   attend   scores, softmax, value aggregation over the cache -> xb          (fuses :146-157)
//   oproj    Wo.xb + x -> x                                                   (fuses :160,:218)
//   gateup   rmsnorm(x)        -> W1,W3 GEMV -> SwiGLU -> hb                  (fuses :221-224)
//   down     W2.hb + x -> x                                                   (fuses :225-226)
//   lmhead   rmsnorm(x)        -> classifier GEMV -> logits                   (fuses :357-358)
//   sample   four short steps over vocabulary chunks + one bookkeeping step   (:366-370)
//
// Each phase is a __device__ function of (workgroup index, workgroup count); the
// kernels of fused_decode.hip run one phase per launch (a HIP graph of kernels).
// GEMV phases issue their first weight loads BEFORE calling the `pre` hook and
// staging the activations in LDS: weights never depend on activations.
// (dataflow_decode.hip, the one-kernel-per-token schedule, shares DecodeArgs, the
// sampler helpers and finish_token with this file but has its own phase code.)
//
// kCoh selects dev::Mem<kCoh> for whatever one phase hands to the next; the
// kernels here pass false (their inputs are complete before the launch).  Values
// that cross workgroups inside ONE launch (the attention split partials) always
// use dev::Mem<true>: producer and consumer may sit on different XCDs.
#pragma once

#include "lpp_device.hpp"
#include "lpp_model.hpp"
#include "sampler.hpp"

namespace lpp {
namespace ph {

using namespace dev;

struct DecodeArgs {
    int dim, hidden, n_layers, n_heads, n_kv_heads, head_size, kv_dim, vocab, seq_len, gqa;
    int max_splits;
    // weights (stacked per layer), see lpp_model
    const float* emb;
    const float* rms_att;
    const char* wq;
    const char* wk;
    const char* wv;
    const char* wo;
    const float* rms_ffn;
    const char* w1;
    const char* w2;
    const char* w3;
    const float* rms_final;
    const char* wcls;
    // run state
    float* x;
    float* xb;
    float* q;
    float* k;
    float* v;
    float* hb;
    float* logits;
    float* work;           // sampler working copy of the logits
    uint16_t* key_cache;
    uint16_t* value_cache;
    float* att_partial;    // [n_heads][max_splits][head_size + 2]
    unsigned* att_count;   // [n_kv_heads] arrival counters of the split combine
    const float2* rope;    // [seq_len][head_size/2]
    StepParams* step;
    int* history;          // ring of step->history_cap entries
    const float* uniforms; // per-step draws, or null: use step->r
    int* out_tokens;       // per-step results (may be pinned host memory), or null
    int* sampled;          // [1]
    smp::SampleScratch sample_scratch;
    unsigned long long* trace;  // optional: timeline of workgroup 0 (one-kernel-per-token schedule only)
};

// ---------------------------------------------------------------------------
// Activation staging
// ---------------------------------------------------------------------------

// xs[0..n) = src, zero padded to a multiple of 8.  n is even.
template <bool kCoh>
__device__ __forceinline__ void stage_plain(float* xs, const float* src, int n) {
    const int n_pad = (n + 7) & ~7;
    for (int i = 2 * threadIdx.x; i < n_pad; i += 2 * blockDim.x) {
        float2 v = make_float2(0.0f, 0.0f);
        if (i < n) v = Mem<kCoh>::ld2(src + i);
        xs[i] = v.x;
        xs[i + 1] = v.y;
    }
    __syncthreads();
}

// xs = rmsnorm(src) * gain, ops.cpp:20-32: (x * s) * w with s = 1/sqrtf(mean + 1e-5f).
template <bool kCoh>
__device__ __forceinline__ void stage_rmsnorm(float* xs, const float* src, const float* gain, int n) {
#pragma clang fp contract(off)
    __shared__ float scratch[16];
    float ss = 0.0f;
    for (int i = 2 * threadIdx.x; i < n; i += 2 * blockDim.x) {
        const float2 v = Mem<kCoh>::ld2(src + i);
        xs[i] = v.x;
        xs[i + 1] = v.y;
        ss += v.x * v.x;
        ss += v.y * v.y;
    }
    ss = block_sum(ss, scratch);
    ss /= static_cast<float>(n);
    ss += 1e-5f;
    const float scale = 1.0f / sqrtf(ss);
    const int n_pad = (n + 7) & ~7;
    for (int i = 2 * threadIdx.x; i < n_pad; i += 2 * blockDim.x) {
        if (i < n) {
            const float2 g = *reinterpret_cast<const float2*>(gain + i);
            xs[i] = xs[i] * scale * g.x;
            xs[i + 1] = xs[i + 1] * scale * g.y;
        } else {
            xs[i] = 0.0f;
            xs[i + 1] = 0.0f;
        }
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------
// Pipelined row-tile GEMV
// ---------------------------------------------------------------------------

// Register image of one step of a tile: kUnroll chunks of kRows rows.  Loads are
// unconditional (no branch around any of them): a lane whose columns lie beyond
// d reads column 0 instead and its activations are zeroed in fma(); row pointers
// must always be readable (callers clamp rows past the end to a valid row and
// discard the result).  Branch-free requests let the compiler count outstanding
// loads exactly, so the multiply of one step only waits for its own data while
// the next step's requests stay in flight.
template <bool kF16, int kRows, int kUnroll>
struct Tile {
    static constexpr int kPer = WTraits<kF16>::kPerLoad;
    static constexpr int kChunk = kWave * kPer;
    uintx4 w[kUnroll][kRows];

    __device__ __forceinline__ void load(const char* const (&rows)[kRows], int cg, int d) {
        const int lane = lane_id();
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int col = (cg * kUnroll + u) * kChunk + lane * kPer;
            const int safe_col = (col < d) ? col : 0;
#pragma unroll
            for (int r = 0; r < kRows; ++r)
                w[u][r] = load16_stream(rows[r] + static_cast<size_t>(safe_col) * WTraits<kF16>::kBytes);
        }
    }

    // Multiply this step and hand every register back to the memory system the
    // moment it has been used: the 16 bytes just consumed are replaced by the
    // same position of step (next_rows, next_cg).  One request leaves for each one
    // retired, so the number in flight stays constant through the whole phase.
    __device__ __forceinline__ void fma_refill(const float* xs, int cg, int d, float (&acc)[kRows],
                                               const char* const (&next_rows)[kRows], int next_cg) {
        const int lane = lane_id();
        const floatx4 zero = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int col = (cg * kUnroll + u) * kChunk + lane * kPer;
            const bool live = col < d;
            const int safe_col = live ? col : 0;
            const int ncol = (next_cg * kUnroll + u) * kChunk + lane * kPer;
            const size_t noff = static_cast<size_t>(ncol < d ? ncol : 0) * WTraits<kF16>::kBytes;
            if constexpr (kF16) {
                floatx4 xa = *reinterpret_cast<const floatx4*>(xs + safe_col);
                floatx4 xb = *reinterpret_cast<const floatx4*>(xs + safe_col + 4);
                xa = live ? xa : zero;
                xb = live ? xb : zero;
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    acc[r] = dot8(w[u][r], xa, xb, acc[r]);
                    w[u][r] = load16_stream(next_rows[r] + noff);
                }
            } else {
                floatx4 xa = *reinterpret_cast<const floatx4*>(xs + safe_col);
                xa = live ? xa : zero;
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    acc[r] = dot4(w[u][r], xa, acc[r]);
                    w[u][r] = load16_stream(next_rows[r] + noff);
                }
            }
        }
    }

    __device__ __forceinline__ void fma(const float* xs, int cg, int d, float (&acc)[kRows]) const {
        const int lane = lane_id();
        const floatx4 zero = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int col = (cg * kUnroll + u) * kChunk + lane * kPer;
            const bool live = col < d;
            const int safe_col = live ? col : 0;
            if constexpr (kF16) {
                floatx4 xa = *reinterpret_cast<const floatx4*>(xs + safe_col);
                floatx4 xb = *reinterpret_cast<const floatx4*>(xs + safe_col + 4);
                xa = live ? xa : zero;
                xb = live ? xb : zero;
#pragma unroll
                for (int r = 0; r < kRows; ++r) acc[r] = dot8(w[u][r], xa, xb, acc[r]);
            } else {
                floatx4 xa = *reinterpret_cast<const floatx4*>(xs + safe_col);
                xa = live ? xa : zero;
#pragma unroll
                for (int r = 0; r < kRows; ++r) acc[r] = dot4(w[u][r], xa, acc[r]);
            }
        }
    }
};

// Position of one wavefront in its list of work: a tile (kRows rows) and, inside
// it, a group of kUnroll 1-KiB chunks of every row.
template <int kRows>
struct Cursor {
    int tile;
    int cg;
    bool have;
    const char* rows[kRows];
};

// One wavefront walks tiles wave_g, wave_g + waves_total, ...; a tile is kRows
// rows given by row_ptr(tile, r) (always a readable row) and is consumed in steps
// of kUnroll chunks.  Two steps are always in flight: both are requested before
// pre() runs, and each register set is refilled with the step after next as soon
// as it has been multiplied.  The steady-state loop contains no conditional
// load (a conditionally refilled register set would make the compiler copy it
// and wait for every outstanding load) and no global store (on this target
// stores share the loads' wait counter, and a pending store makes every wait a
// full drain): the dot products of up to 64 (tile, row) pairs are parked one
// per lane in a single register and written out when the wavefront's work is
// done, by emit(tile, r, value, neighbour), where neighbour is the value of row
// r^1 of the same tile.  pre() runs once, after the first requests and before
// anything reads xs; every wavefront of the workgroup calls it, with or without
// work.
template <bool kF16, int kRows, int kUnroll, class RowFn, class EmitFn, class PreFn>
__device__ __forceinline__ void gemv_phase(int ntiles, int d, const float* xs, int wave_g, int waves_total,
                                           RowFn row_ptr, EmitFn emit, PreFn pre) {
    using T = Tile<kF16, kRows, kUnroll>;
    using C = Cursor<kRows>;
    static_assert(kWave % kRows == 0, "results are parked kRows per tile");
    constexpr int kParkRegs = 2;
    constexpr int kTilesPerRound = kParkRegs * kWave / kRows;  // results one round can park
    const int lane = lane_id();
    const int ncg = (d + T::kChunk * kUnroll - 1) / (T::kChunk * kUnroll);
    const int my_tiles = (wave_g < ntiles) ? (ntiles - wave_g + waves_total - 1) / waves_total : 0;

    // c <- the step after c (row pointers change only at tile boundaries)
    auto advance = [&](C& c) {
        if (c.cg + 1 < ncg) {
            c.cg += 1;
            return;
        }
        c.cg = 0;
        c.tile += waves_total;
        const int t = c.tile < ntiles ? c.tile : wave_g;  // past the end: any valid tile, never loaded
#pragma unroll
        for (int r = 0; r < kRows; ++r) c.rows[r] = row_ptr(t, r);
    };

    C next;  // next step to request
    next.tile = wave_g;
    next.cg = 0;
    next.have = true;
#pragma unroll
    for (int r = 0; r < kRows; ++r) next.rows[r] = row_ptr(wave_g < ntiles ? wave_g : 0, r);

    // A round is at most kTilesPerRound tiles: its dot products are parked in
    // registers and written out after its last multiply, outside the streaming
    // loop.  One round covers a whole phase for every shape met in practice.
    bool first_round = true;
    int tiles_done = 0;
    do {
        const int round_tiles = min(my_tiles - tiles_done, kTilesPerRound);
        const int n_steps = round_tiles * ncg;
        int use_cg = 0;  // chunk group of the next step to multiply
        int parked = 0;  // tiles of this round already reduced
        float park[kParkRegs];  // lane (slot % 64) of register (slot / 64) holds slot = k * kRows + r
#pragma unroll
        for (int p = 0; p < kParkRegs; ++p) park[p] = 0.0f;

        T ta, tb;
        if (n_steps > 0) {
            ta.load(next.rows, next.cg, d);
            advance(next);
        }
        if (n_steps > 1) {
            tb.load(next.rows, next.cg, d);
            advance(next);
        }
        if (first_round) pre();
        first_round = false;
        float acc[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r) acc[r] = 0.0f;

        auto park_if_tile_done = [&]() {
            if (use_cg + 1 == ncg) {
#pragma unroll
                for (int r = 0; r < kRows; ++r) {
                    const float sum = wave_sum(acc[r]);
                    const int slot = parked * kRows + r;
#pragma unroll
                    for (int p = 0; p < kParkRegs; ++p) park[p] = (lane + p * kWave == slot) ? sum : park[p];
                    acc[r] = 0.0f;
                }
                use_cg = 0;
                parked += 1;
            } else {
                use_cg += 1;
            }
        };
        auto consume = [&](const T& t) {
            t.fma(xs, use_cg, d, acc);
            park_if_tile_done();
        };

        int i = 0;
        for (; i + 3 < n_steps; i += 2) {
            ta.fma_refill(xs, use_cg, d, acc, next.rows, next.cg);
            advance(next);
            park_if_tile_done();
            tb.fma_refill(xs, use_cg, d, acc, next.rows, next.cg);
            advance(next);
            park_if_tile_done();
        }
        const int left = n_steps - i;  // 0..3 steps: ta holds step i, tb step i+1
        if (left >= 1) consume(ta);
        if (left == 3) {
            ta.load(next.rows, next.cg, d);
            advance(next);
        }
        if (left >= 2) consume(tb);
        if (left == 3) consume(ta);

        // write the round's results: one lane per (tile, row)
        const int first_tile = wave_g + tiles_done * waves_total;
#pragma unroll
        for (int p = 0; p < kParkRegs; ++p) {
            const float neighbour = dpp_move<kDppXor1>(park[p]);
            const int slot = lane + p * kWave;
            if (slot < parked * kRows) {
                const int k = slot / kRows;
                emit(first_tile + k * waves_total, slot - k * kRows, park[p], neighbour);
            }
        }
        tiles_done += round_tiles;
    } while (tiles_done < my_tiles);
}

__device__ __forceinline__ const char* row_at(const char* base, size_t layer_rows, int layer, int row, int d,
                                              int wbytes) {
    return base + (static_cast<size_t>(layer) * layer_rows + static_cast<size_t>(row)) * d * wbytes;
}

// Input of layer 0 is the embedding row of the current token (model.cpp:345-349);
// later layers read x.
__device__ __forceinline__ const float* layer_input(const DecodeArgs& a, int layer) {
    return layer == 0 ? a.emb + static_cast<size_t>(a.step->token) * a.dim : a.x;
}

// ---------------------------------------------------------------------------
// Phase: rmsnorm -> QKV -> RoPE -> q buffer and K/V cache
// ---------------------------------------------------------------------------
template <bool kF16, int kRows, bool kCoh, class PreFn>
__device__ __forceinline__ void phase_qkv(const DecodeArgs& a, int layer, int wg, int nwg, float* xs, PreFn pre) {
#pragma clang fp contract(off)
    static_assert(kRows % 2 == 0, "RoPE pairs must stay inside a tile");
    const int wbytes = kF16 ? 2 : 4;
    const int waves_per_wg = static_cast<int>(blockDim.x) / kWave;
    const int wave_g = wg * waves_per_wg + wave_index();
    const int total_rows = a.dim + 2 * a.kv_dim;
    const int ntiles = (total_rows + kRows - 1) / kRows;
    const int dim = a.dim, kv_dim = a.kv_dim;

    auto row_ptr = [&](int tile, int r) -> const char* {
        const int g = tile * kRows + r;
        if (g < dim) return row_at(a.wq, dim, layer, g, dim, wbytes);
        if (g < dim + kv_dim) return row_at(a.wk, kv_dim, layer, g - dim, dim, wbytes);
        const int gv = (g < total_rows ? g : total_rows - 1) - dim - kv_dim;  // past the end: a valid row, result unused
        return row_at(a.wv, kv_dim, layer, gv, dim, wbytes);
    };
    auto prologue = [&]() {
        pre();
        stage_rmsnorm<kCoh>(xs, layer_input(a, layer), a.rms_att + static_cast<size_t>(layer) * dim, dim);
    };
    const int pos = a.step->pos;
    const int hs = a.head_size;
    const float2* cs_row = a.rope + static_cast<size_t>(pos) * (hs / 2);
    // One lane per output row; rows (2j, 2j+1) of a tile are a RoPE pair, the odd
    // one being this lane's neighbour.
    auto epilogue = [&](int tile, int r, float mine, float neighbour) {
        const int g = tile * kRows + r;
        if (g >= total_rows) return;
        float out = mine;
        if (g < dim + kv_dim) {
            // ops.cpp:36-52 on the pair (i, i+1); i is the even index inside q or k.
            const int gi = (g < dim) ? g : g - dim;
            const float2 cs = cs_row[((gi & ~1) % hs) >> 1];
            out = (gi & 1) ? neighbour * cs.y + mine * cs.x   // q[i+1] = q0*sin + q1*cos
                           : mine * cs.x - neighbour * cs.y;  // q[i]   = q0*cos - q1*sin
        }
        if (g < dim) {
            Mem<kCoh>::st(a.q + g, out);
        } else {
            // model.cpp:171-176 / scatter_kv.cu:15-18.
            const bool is_k = g < dim + kv_dim;
            const int i = is_k ? g - dim : g - dim - kv_dim;
            const int head = i / hs, within = i - head * hs;
            const size_t dst = static_cast<size_t>(layer) * kv_dim * a.seq_len +
                               static_cast<size_t>(head) * a.seq_len * hs + static_cast<size_t>(pos) * hs + within;
            Mem<kCoh>::st((is_k ? a.k : a.v) + i, out);
            (is_k ? a.key_cache : a.value_cache)[dst] = f32_to_f16_bits(out);
        }
    };
    gemv_phase<kF16, kRows, 4>(ntiles, dim, xs, wave_g, nwg * waves_per_wg, row_ptr, epilogue, prologue);
}

// ---------------------------------------------------------------------------
// Phase: out = W . xs + residual   (O projection and down projection)
// ---------------------------------------------------------------------------
template <bool kF16, int kRows, bool kCoh, int kUnroll = 4, class PreFn>
__device__ __forceinline__ void phase_proj_residual(const char* w_layer, int n, int d, const float* src,
                                                    const float* residual, float* out, int wg, int nwg,
                                                    float* xs, PreFn pre) {
    const int wbytes = kF16 ? 2 : 4;
    const int waves_per_wg = static_cast<int>(blockDim.x) / kWave;
    const int wave_g = wg * waves_per_wg + wave_index();
    const int ntiles = (n + kRows - 1) / kRows;
    auto row_ptr = [&](int tile, int r) -> const char* {
        const int g = tile * kRows + r;
        return w_layer + static_cast<size_t>(g < n ? g : n - 1) * d * wbytes;  // past the end: a valid row, result unused
    };
    auto prologue = [&]() {
        pre();
        stage_plain<kCoh>(xs, src, d);
    };
    auto epilogue = [&](int tile, int r, float mine, float) {
        const int g = tile * kRows + r;
        if (g >= n) return;
        Mem<kCoh>::st(out + g, Mem<kCoh>::ld(residual + g) + mine);  // model.cpp:232,239: x[i] += xb2[i]
    };
    gemv_phase<kF16, kRows, kUnroll>(ntiles, d, xs, wave_g, nwg * waves_per_wg, row_ptr, epilogue, prologue);
}

// ---------------------------------------------------------------------------
// Phase: rmsnorm -> gate/up -> SwiGLU -> hb
// ---------------------------------------------------------------------------
template <bool kF16, int kPairRows, bool kCoh, class PreFn>
__device__ __forceinline__ void phase_gateup(const DecodeArgs& a, int layer, int wg, int nwg, float* xs, PreFn pre) {
#pragma clang fp contract(off)
    constexpr int kRows = 2 * kPairRows;
    const int wbytes = kF16 ? 2 : 4;
    const int waves_per_wg = static_cast<int>(blockDim.x) / kWave;
    const int wave_g = wg * waves_per_wg + wave_index();
    const int hidden = a.hidden, dim = a.dim;
    const int ntiles = (hidden + kPairRows - 1) / kPairRows;
    // Row 2j of a tile is gate row j, row 2j+1 the matching up row, so the two
    // halves of one output sit in neighbouring lanes.
    auto row_ptr = [&](int tile, int r) -> const char* {
        const int g = tile * kPairRows + (r >> 1);
        return row_at((r & 1) ? a.w3 : a.w1, hidden, layer, g < hidden ? g : hidden - 1, dim, wbytes);
    };
    auto prologue = [&]() {
        pre();
        stage_rmsnorm<kCoh>(xs, a.x, a.rms_ffn + static_cast<size_t>(layer) * dim, dim);
    };
    auto epilogue = [&](int tile, int r, float gate, float up) {
        if (r & 1) return;
        const int g = tile * kPairRows + (r >> 1);
        if (g >= hidden) return;
        // ops.cpp:80-85
        const float sigma = 1.0f / (1.0f + expf(-gate));
        Mem<kCoh>::st(a.hb + g, (gate * sigma) * up);
    };
    gemv_phase<kF16, kRows, 4>(ntiles, dim, xs, wave_g, nwg * waves_per_wg, row_ptr, epilogue, prologue);
}

// ---------------------------------------------------------------------------
// Phase: final rmsnorm -> classifier -> logits
// ---------------------------------------------------------------------------
template <bool kF16, int kRows, bool kCoh, class PreFn>
__device__ __forceinline__ void phase_lmhead(const DecodeArgs& a, int wg, int nwg, float* xs, PreFn pre) {
    const int wbytes = kF16 ? 2 : 4;
    const int waves_per_wg = static_cast<int>(blockDim.x) / kWave;
    const int wave_g = wg * waves_per_wg + wave_index();
    const int vocab = a.vocab, dim = a.dim;
    const int ntiles = (vocab + kRows - 1) / kRows;
    auto row_ptr = [&](int tile, int r) -> const char* {
        const int g = tile * kRows + r;
        return a.wcls + static_cast<size_t>(g < vocab ? g : vocab - 1) * dim * wbytes;
    };
    auto prologue = [&]() {
        pre();
        stage_rmsnorm<kCoh>(xs, a.x, a.rms_final, dim);
    };
    auto epilogue = [&](int tile, int r, float mine, float) {
        const int g = tile * kRows + r;
        if (g < vocab) Mem<kCoh>::st(a.logits + g, mine);
    };
    gemv_phase<kF16, kRows, 4>(ntiles, dim, xs, wave_g, nwg * waves_per_wg, row_ptr, epilogue, prologue);
}

// ---------------------------------------------------------------------------
// Phase: attention over the cache (split context)
// ---------------------------------------------------------------------------

// Number of context splits in use at this position: about 256 positions each
// (shorter pieces do not repay the cross-workgroup combine).
__device__ __forceinline__ int active_splits(int npos, int max_splits) {
    int s = (npos + 255) / 256;
    return s < 1 ? 1 : (s > max_splits ? max_splits : s);
}

template <int kGroup>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (kGroup >= 2) v += dpp_move<kDppXor1>(v);
    if constexpr (kGroup >= 4) v += dpp_move<kDppXor2>(v);
    if constexpr (kGroup >= 8) v += dpp_move<kDppHalfMirror>(v);
    if constexpr (kGroup >= 16) v += dpp_move<kDppMirror>(v);
    return v;
}

constexpr int kAttBlock = 512;   // positions per softmax sub-block
constexpr int kMaxGqa = 8;       // query heads per KV head held in registers

// LDS floats the attention phase needs.
__host__ __device__ inline int attention_lds_floats(int gqa, int head_size, int nthreads) {
    const int hs_pad = (head_size + 7) & ~7;
    return gqa * hs_pad              // q
           + gqa * kAttBlock         // scores / probabilities of one sub-block
           + 3 * gqa                 // running max, running sum, correction
           + (nthreads / kWave) * gqa * hs_pad;  // cross-wave reduction
}

// 8 binary16 values of a cache row.  The row of the position being decoded was
// stored by another workgroup earlier in the same persistent kernel; there it is
// taken from the fp32 k / v vector (coherent read) and rounded exactly as the
// cache store rounds it, so both schedules see identical values.
template <bool kCoh>
__device__ __forceinline__ uintx4 cache_row8(const uint16_t* cache_row, const float* fresh, bool is_current,
                                             int offset) {
    if constexpr (kCoh) {
        if (is_current) {
            union {
                half8_t h;
                uintx4 u;
            } c;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float2 f = Mem<true>::ld2(fresh + offset + 2 * j);
                c.h[2 * j] = static_cast<half_t>(f.x);
                c.h[2 * j + 1] = static_cast<half_t>(f.y);
            }
            return c.u;
        }
    }
    return load16(cache_row + offset);
}

// One work item: KV head `kvh`, context split `split` of `nsplits`.  kGroup lanes
// cover one position (8 binary16 each).  Sub-blocks of kAttBlock positions:
// scores -> LDS, per-head max/exp/sum by one wavefront per head, then V
// accumulation with the running-max correction (the sum the CPU forms at
// model.cpp:186-198 with the softmax of ops.cpp:56-75, regrouped).  With one
// split the result goes straight to xb; otherwise the partial (max, sum,
// unnormalised output) goes to att_partial and the last split to arrive for
// this KV head combines all of them.
template <int kGroup, bool kCoh>
__device__ __forceinline__ void attention_item(const DecodeArgs& a, int layer, int kvh, int split, int nsplits, int npos,
                               float* lds) {
    const int hs = a.head_size, gqa = a.gqa;
    const int hs_pad = kGroup * 8;
    const int nthreads = static_cast<int>(blockDim.x);
    const int nwaves = nthreads / kWave;
    const int ngroups = nthreads / kGroup;
    const int tid = static_cast<int>(threadIdx.x);
    const int sub = tid % kGroup, grp = tid / kGroup;
    const int wave = tid / kWave;

    float* qs = lds;                          // [gqa][hs_pad]
    float* sc = qs + gqa * hs_pad;            // [gqa][kAttBlock]
    float* run_max = sc + gqa * kAttBlock;    // [gqa]
    float* run_sum = run_max + gqa;           // [gqa]
    float* corr = run_sum + gqa;              // [gqa]
    float* red = corr + gqa;                  // [nwaves][gqa][hs_pad]

    const float scale = 1.0f / sqrtf(static_cast<float>(hs));  // model.cpp:188
    for (int i = tid; i < gqa * hs_pad; i += nthreads) {
        const int qh = i / hs_pad, e = i - qh * hs_pad;
        qs[i] = (e < hs) ? Mem<kCoh>::ld(a.q + static_cast<size_t>(kvh * gqa + qh) * hs + e) : 0.0f;
    }
    if (tid < gqa) {
        run_max[tid] = -INFINITY;
        run_sum[tid] = 0.0f;
    }
    const int chunk = (npos + nsplits - 1) / nsplits;
    const int t_begin = split * chunk;
    const int t_end = min(npos, t_begin + chunk);
    const int current = npos - 1;
    const size_t head_base = (static_cast<size_t>(layer) * a.n_kv_heads + kvh) * a.seq_len * hs;
    const uint16_t* kbase = a.key_cache + head_base;
    const uint16_t* vbase = a.value_cache + head_base;
    const float* k_fresh = a.k + static_cast<size_t>(kvh) * hs;
    const float* v_fresh = a.v + static_cast<size_t>(kvh) * hs;

    float acc[kMaxGqa][8];
#pragma unroll
    for (int qh = 0; qh < kMaxGqa; ++qh)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[qh][e] = 0.0f;
    __syncthreads();

    // A sub-block is `per_group` consecutive rounds of ngroups positions.  Every
    // lane requests all its K rows of the sub-block before the first multiply, and
    // all its V rows before the softmax (8 independent 16-byte loads in flight
    // each time), so a sub-block costs about two memory round trips instead of
    // two per position.
    constexpr int kMaxPerGroup = 8;
    int per_group = kAttBlock / ngroups;
    if (per_group > kMaxPerGroup) per_group = kMaxPerGroup;
    if (per_group < 1) per_group = 1;
    const int sub_block = per_group * ngroups;  // <= kAttBlock
    const bool lane_live = sub * 8 < hs;
    for (int b0 = t_begin; b0 < t_end; b0 += sub_block) {
        const int b1 = min(t_end, b0 + sub_block);
        uintx4 rows8[kMaxPerGroup];
#pragma unroll
        for (int j = 0; j < kMaxPerGroup; ++j) {
            const int t = b0 + grp + j * ngroups;
            rows8[j] = uintx4{0u, 0u, 0u, 0u};
            if (j < per_group && t < b1 && lane_live)
                rows8[j] = cache_row8<kCoh>(kbase + static_cast<size_t>(t) * hs, k_fresh, t == current, sub * 8);
        }
        // scores of this sub-block (query head outermost: only one head's q slice
        // is held in registers at a time)
#pragma unroll
        for (int qh = 0; qh < kMaxGqa; ++qh) {
            if (qh < gqa) {
                const float* qv = qs + qh * hs_pad + sub * 8;
                const floatx4 xa = *reinterpret_cast<const floatx4*>(qv);
                const floatx4 xb = *reinterpret_cast<const floatx4*>(qv + 4);
#pragma unroll
                for (int j = 0; j < kMaxPerGroup; ++j) {
                    const int t = b0 + grp + j * ngroups;
                    const float s = group_sum<kGroup>(dot8(rows8[j], xa, xb, 0.0f));
                    if (j < per_group && t < b1 && sub == 0) sc[qh * kAttBlock + (t - b0)] = s * scale;
                }
            }
        }
        // the V rows of the same positions travel while the softmax is formed
#pragma unroll
        for (int j = 0; j < kMaxPerGroup; ++j) {
            const int t = b0 + grp + j * ngroups;
            rows8[j] = uintx4{0u, 0u, 0u, 0u};
            if (j < per_group && t < b1 && lane_live)
                rows8[j] = cache_row8<kCoh>(vbase + static_cast<size_t>(t) * hs, v_fresh, t == current, sub * 8);
        }
        __syncthreads();
        // per head: new running max, probabilities, running sum, correction
        for (int qh = wave; qh < gqa; qh += nwaves) {
            float* row = sc + qh * kAttBlock;
            const int n = b1 - b0;
            float m = -INFINITY;
            for (int i = lane_id(); i < n; i += kWave) m = fmaxf(m, row[i]);
            m = wave_max(m);
            const float m_old = run_max[qh];
            const float m_new = fmaxf(m_old, m);
            float l = 0.0f;
            for (int i = lane_id(); i < n; i += kWave) {
                const float p = expf(row[i] - m_new);
                row[i] = p;
                l += p;
            }
            l = wave_sum(l);
            if (lane_id() == 0) {
                const float c = (m_old == -INFINITY) ? 0.0f : expf(m_old - m_new);
                corr[qh] = c;
                run_sum[qh] = run_sum[qh] * c + l;
                run_max[qh] = m_new;
            }
        }
        __syncthreads();
        // value accumulation from the rows already in registers
#pragma unroll
        for (int qh = 0; qh < kMaxGqa; ++qh) {
            if (qh < gqa) {
                const float c = corr[qh];
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[qh][e] *= c;
            }
        }
#pragma unroll
        for (int j = 0; j < kMaxPerGroup; ++j) {
            const int t = b0 + grp + j * ngroups;
            if (j < per_group && t < b1 && lane_live) {
                const half8_t vv = as_half8(rows8[j]);
#pragma unroll
                for (int qh = 0; qh < kMaxGqa; ++qh) {
                    if (qh < gqa) {
                        const float p = sc[qh * kAttBlock + (t - b0)];
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc[qh][e] = fmaf(static_cast<float>(vv[e]), p, acc[qh][e]);
                    }
                }
            }
        }
        __syncthreads();
    }

    // Reduce the per-group partial outputs: across the groups of a wavefront by
    // lane exchange, across wavefronts through LDS in wave order.
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
    const int stride = hs + 2;
    if (nsplits == 1) {
        // Whole context in this workgroup: normalise and finish (model.cpp:190-198).
        for (int i = tid; i < gqa * hs; i += nthreads) {
            const int qh = i / hs, e = i - qh * hs;
            float o = 0.0f;
            for (int w = 0; w < nwaves; ++w) o += red[(w * gqa + qh) * hs_pad + e];
            Mem<kCoh>::st(a.xb + static_cast<size_t>(kvh * gqa + qh) * hs + e, o / run_sum[qh]);
        }
        return;
    }
    // Partials always travel with device-coherent accesses: writer and combiner
    // are different workgroups of one launch in both schedules.
    for (int i = tid; i < gqa * hs; i += nthreads) {
        const int qh = i / hs, e = i - qh * hs;
        float o = 0.0f;
        for (int w = 0; w < nwaves; ++w) o += red[(w * gqa + qh) * hs_pad + e];
        float* part = a.att_partial + (static_cast<size_t>(kvh * gqa + qh) * a.max_splits + split) * stride;
        Mem<true>::st(part + e, o);
        if (e == 0) {
            Mem<true>::st(part + hs, run_max[qh]);
            Mem<true>::st(part + hs + 1, run_sum[qh]);
        }
    }

    // The last split to arrive for this KV head combines all of them.  The block
    // barrier waits for this workgroup's stores; the ticket is taken after it.
    __shared__ int is_last;
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket = __hip_atomic_fetch_add(&a.att_count[kvh], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = (ticket == static_cast<unsigned>(nsplits - 1)) ? 1 : 0;
        if (is_last) __hip_atomic_store(&a.att_count[kvh], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return;
    for (int i = tid; i < gqa * hs; i += nthreads) {
        const int qh = i / hs, e = i - qh * hs;
        const float* base = a.att_partial + static_cast<size_t>(kvh * gqa + qh) * a.max_splits * stride;
        float top = -INFINITY;
        for (int s = 0; s < nsplits; ++s) top = fmaxf(top, Mem<true>::ld(base + s * stride + hs));
        float o = 0.0f, l = 0.0f;
        for (int s = 0; s < nsplits; ++s) {
            const float ms = Mem<true>::ld(base + s * stride + hs);
            const float wgt = (ms == -INFINITY) ? 0.0f : expf(ms - top);
            o += Mem<true>::ld(base + s * stride + e) * wgt;
            l += Mem<true>::ld(base + s * stride + hs + 1) * wgt;
        }
        Mem<kCoh>::st(a.xb + static_cast<size_t>(kvh * gqa + qh) * hs + e, o / l);
    }
}

template <bool kCoh, class PreFn>
__device__ __forceinline__ void phase_attention(const DecodeArgs& a, int layer, int wg, int nwg, float* lds,
                                                PreFn pre) {
    pre();
    const int npos = a.step->pos + 1;
    const int nsplits = active_splits(npos, a.max_splits);
    const int items = a.n_kv_heads * nsplits;
    const int hs = a.head_size;
    for (int item = wg; item < items; item += nwg) {
        const int kvh = item / nsplits, split = item - kvh * nsplits;
        if (hs <= 8) attention_item<1, kCoh>(a, layer, kvh, split, nsplits, npos, lds);
        else if (hs <= 16) attention_item<2, kCoh>(a, layer, kvh, split, nsplits, npos, lds);
        else if (hs <= 32) attention_item<4, kCoh>(a, layer, kvh, split, nsplits, npos, lds);
        else if (hs <= 64) attention_item<8, kCoh>(a, layer, kvh, split, nsplits, npos, lds);
        else attention_item<16, kCoh>(a, layer, kvh, split, nsplits, npos, lds);
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// Sampler steps (see sampler.hpp) and the end-of-token bookkeeping
// ---------------------------------------------------------------------------

__device__ __forceinline__ float step_uniform(const DecodeArgs& a) {
    return a.uniforms ? a.uniforms[a.step->step_index] : a.step->r;
}

// Chunk c of the vocabulary: penalty, temperature, chunk maximum.
template <bool kCoh>
__device__ __forceinline__ void sample_step_scale(const DecodeArgs& a, int chunk, int c) {
    const StepParams* sp = a.step;
    smp::scale_max_chunk<kCoh>(a.logits, a.work, a.vocab, chunk, c, sp->temperature, sp->penalty,
                               sp->history_len > 0 ? a.history : nullptr, sp->history_len, a.sample_scratch);
}
// Greedy (model.cpp:272-283) finishes here in chunk 0; otherwise exponentials.
template <bool kCoh>
__device__ __forceinline__ void sample_step_exp(const DecodeArgs& a, int chunk, int nchunks, int c) {
    if (a.step->temperature == 0.0f) {
        if (c == 0) {
            const int tok = smp::argmax_over_chunks<kCoh>(nchunks, a.sample_scratch);
            if (threadIdx.x == 0) Mem<kCoh>::sti(a.sampled, tok);
        }
        return;
    }
    smp::exp_sum_chunk<kCoh>(a.work, a.vocab, chunk, nchunks, c, a.sample_scratch);
}
template <bool kCoh>
__device__ __forceinline__ void sample_step_norm(const DecodeArgs& a, int chunk, int nchunks, int c) {
    if (a.step->temperature == 0.0f) return;
    smp::normalise_chunk<kCoh>(a.work, a.vocab, chunk, nchunks, c, a.sample_scratch);
    if (c == 0 && threadIdx.x == 0) Mem<kCoh>::sti(a.sampled, a.vocab - 1);  // model.cpp:302
}
template <bool kCoh>
__device__ __forceinline__ void sample_step_search(const DecodeArgs& a, int chunk, int c) {
    if (a.step->temperature == 0.0f) return;
    smp::cdf_search_chunk<kCoh>(a.work, a.vocab, chunk, c, step_uniform(a), a.sample_scratch, a.sampled);
}

// After the sampler: publish the token, feed it back as the next input, advance
// the position and the penalty window (src/main.cpp:200-208; the window is kept
// as a ring because the penalty does not depend on the order of its entries).
// out_tokens may be pinned host memory: the 4-byte result is stored with system
// scope so the host sees it without a copy command.
__device__ __forceinline__ void finish_token(const DecodeArgs& a, int token, unsigned epoch_advance) {
    StepParams* sp = a.step;
    sp->epoch += epoch_advance;
    a.sampled[0] = token;
    if (sp->freeze) return;
    if (sp->history_cap > 0) {
        a.history[sp->history_next] = token;
        sp->history_next = (sp->history_next + 1) % sp->history_cap;
        if (sp->history_len < sp->history_cap) sp->history_len += 1;
    }
    const int index = sp->step_index;
    sp->token = token;
    sp->pos += 1;
    sp->step_index = index + 1;
    if (a.out_tokens) __hip_atomic_store(a.out_tokens + index, token, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace ph

// Persistent one-kernel-per-token schedule, implemented in dataflow_decode.hip.
size_t dataflow_tagged_bytes(const lpp_model* m);
lpp_status dataflow_launch(lpp_model* m, const ph::DecodeArgs& a, hipStream_t s);
unsigned dataflow_phases_per_token(int n_layers);
unsigned dataflow_trace_marks();
lpp_status dataflow_forget_plans(lpp_model* m, hipStream_t s, int df_xcc);
lpp_status dataflow_forget_lists(lpp_model* m, hipStream_t s);
void dataflow_partition_classes(const lpp_model* m, int* item_workgroups, int* n_xcc);
lpp_status dataflow_after_error(lpp_model* m, int code, bool* relaunch);
lpp_status dataflow_take_options(lpp_model* m, hipStream_t s);

}  // namespace lpp
