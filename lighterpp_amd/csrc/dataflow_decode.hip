// dataflow_decode.hip -- LPP_PATH_PERSISTENT: one kernel per token, no grid
// barrier, weights streamed independently of the dependency chain.
//
// The phases of forward() (reference src/model.cpp:342-371; decode_phases.hpp
// describes the split) need a full activation vector from all workgroups at
// every boundary.  Here the hand-over is the data itself: every value one phase
// gives to the next is published as ONE 8-byte device-scope store holding the
// fp32 value and a 32-bit sequence number, and a consumer polls the values it
// needs until they carry the number it expects.  A hand-over costs one memory
// round trip and nobody waits for a workgroup it does not depend on.
//
// A batch-1 decode is a chain of ~80 such hand-overs, each a couple of
// microseconds of pure latency during which a conventional GEMV kernel has
// nothing in flight.  The weights, however, do not depend on anything, and the
// order in which a wavefront will need them is fixed.  Each workgroup is
// therefore split into two kinds of wavefronts:
//
//   streaming wavefronts  walk their fixed list of weight rows across ALL phases
//       and layers of the token with kDepth 4-KiB steps always in flight in
//       registers.  They never touch global memory otherwise: activations come
//       from LDS, results go to LDS, and they only ever wait on an LDS flag.
//       While the dependency chain is stalled they already hold the next
//       phases' weights.
//   exchange wavefronts   poll the tagged inputs of a phase, stage them in LDS
//       (times the norm gain where a norm precedes the GEMV), raise the flag,
//       later pick up the row results, apply the phase's epilogue (the norm's
//       1/rms, RoPE, SwiGLU, residual) and publish.  They also run attention and
//       the sampler.  What they send and poll does queue behind weight requests
//       already in flight: the streaming wavefronts hold their refills back for
//       a moment when the exchange wavefronts are about to publish.
//
// Sequence numbers grow monotonically for the life of a model (the host hands
// every launch its base and advances it by the number of phases), so a stale
// value, even one left by a launch that gave up, is never taken for a fresh
// one.  Buffer reuse needs no further synchronisation: every buffer is consumed
// one phase after it is produced and rewritten no sooner than two phases later,
// and the inputs of each phase transitively require every workgroup to have
// finished reading the phase before the previous one.  Global polls are bounded:
// a wavefront that gives up raises a shared abort flag that ends every other
// poll, and no LDS wait depends on a global one, so the grid always drains.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <unordered_map>
#include <vector>

#include "decode_phases.hpp"

namespace lpp {
namespace df {

using namespace ph;
using namespace dev;

constexpr int kGemvWaves = 8;                      // streaming wavefronts per workgroup
constexpr int kIoWaves = 8;                        // exchange wavefronts per workgroup
constexpr int kThreads = (kGemvWaves + kIoWaves) * kWave;
constexpr int kIoThreads = kIoWaves * kWave;
constexpr int kDepth = 4;                          // weight steps a streaming wavefront keeps in flight
constexpr int kStepLoads = 4;                      // 16-byte loads per lane and step: 4 KiB of one row
constexpr int kPollBatch = 8;                      // tagged values one thread requests before checking any
constexpr int kItemPositions = 1024;               // a one-head attention work item stays within twice this many positions
constexpr int kAttScoreFloats = 512;               // half of the sampler's LDS copy of the penalty window
constexpr int kMaxHeadPad = 128;
constexpr int kShortRounds = 2;                    // cache rows per lane group a one-head work item requests at once
constexpr int kPacedSteps = 2;                     // next-phase rows a streaming wavefront sends out early after a burst
constexpr int kMaxAttHeads = 4;                    // query heads of one KV head a work item of att_xcd_item covers at most
constexpr int kItemHeads = 2;                      // the same for the items dealt out over the device (att_group_item)
constexpr int kRedStride = kMaxHeadPad + 2;        // one wavefront's partial result of one head: values, maximum, sum

typedef unsigned long long u64;
// Sequence-number base beyond which the host re-zeroes the tagged slots and restarts the count
// (a token advances the base by 5 * layers + 2; 2^32 would be reached after tens of millions of tokens).
constexpr unsigned kTagWrapGuard = 0xf0000000u;

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

// The same inside one XCD: a plain store stays in the XCD's L2 (a device-scope one writes through and drops the line),
// and a non-temporal load is not kept by the compute unit's L1, so it is served by that L2.  Only for slots that no
// other XCD touches.
// (Both statements take their address as a VECTOR operand.  An asm statement that hands a memory instruction a
// SCALAR address operand must begin with s_nop 4: the compiler may have written that register pair with a vector
// instruction (v_readlane from where it keeps spilled scalars) immediately before, a memory instruction reading it
// needs five wait states after such a write, and nobody counts wait states inside an asm statement -- the first
// request would go to whatever the pair held before.)
__device__ __forceinline__ void publish_near(u64* slot, float v, unsigned tag) {
    const u64 both = pack(v, tag);
    asm volatile("global_store_dwordx2 %0, %1, off sc0" ::"v"(slot), "v"(both) : "memory");
}
__device__ __forceinline__ u64 peek_near(const u64* slot) {
    u64 got;
    // (one statement, the wait included: the compiler sees the result only once it is in)
    asm volatile("global_load_dwordx2 %0, %1, off nt\n\ts_waitcnt vmcnt(0)" : "=v"(got) : "v"(slot) : "memory");
    return got;
}

// Tagged vectors of one model, all in one device allocation.
struct Tagged {
    u64* x;      // [dim]     residual stream, written by the O and down projections
    u64* q;      // [dim]
    u64* k;      // [kv_dim]
    u64* v;      // [kv_dim]
    u64* xb;     // [dim]     attention output
    u64* hb;     // [hidden]  SwiGLU output
    u64* part;   // [n_heads][splits_cap][head_size + 2] attention split partials
    u64* stats;  // [nwg][4]  per-workgroup sampler statistics (max, sum, argmax)
    // Copies of hb that only the compute units of one XCD write and read (gather_values): [n_xcc][near_hidden_stride]
    u64* near_hb;
    int near_hidden_stride;  // tagged values per XCD
    int n_xcc;               // XCDs the workgroups go round in turn; 1: no near copies
    int share_hidden;        // values of hb each workgroup of an XCD fetches for the others
    // Workgroup numbering by XCD: workgroup index = (ticket drawn from tickets[XCD] - ticket_base) * n_xcc + XCD.
    unsigned* tickets;       // [n_xcc] counters, drawn once per workgroup and launch
    unsigned ticket_base;    // what a counter read before this launch
    // q, k and v handed to the attention items inside the XCD that formed them (near_qkv: [n_xcc][dim + 2 kv_dim])
    u64* near_qkv;
    int near_qkv_stride;
    int local_qkv;           // nonzero: this token's q, k and v are published to near_qkv only
    int splits_cap;
    unsigned hs_magic;     // floor(2^32 / head_size) + 1: x / head_size == __umulhi(x, hs_magic) for x < 2^25
    int att_splits;        // context splits per query head at this position (worked out on the host: the search
    int att_group_splits;  // is a few dozen integer divisions); > 0: items cover two heads of a KV head, this many splits
    float inv_sqrt_head;   // 1 / sqrt(head_size), formed on the host (on the device it would sit in a vector register all token long)
    int lane_item_cap;     // contexts up to this many positions take the one-pass item of a head of size 64 (att_lane_item)
    // A KV head's context split over the workgroups of its XCD (att_xcd_item): xa_chunk > 0 switches it on.
    int xa_chunk;          // positions per workgroup (a multiple of 8, at most 8 * 64)
    int xa_active;         // workgroups of a KV head that hold positions at this context length
    int xa_ppw;            // positions per exchange wavefront: xa_chunk / 8
    u64* near_part;        // [n_xcc][workgroups per XCD][near_part_stride] partial results, read inside the XCD only
    int near_part_stride;
    // the step record, except the token id (which the previous launch left in device memory)
    int pos, history_len;
    float temperature, penalty, r;
    unsigned base;    // sequence-number base of this launch, advanced by the host once per token
    unsigned* abort;  // raised by a wavefront whose poll ran out of patience
    unsigned spin_limit;
    int trace_stride;  // timeline: 0 = workgroup 0 only; else every workgroup writes its own block of this many words
    const int* gu_first;  // [workgroups + 1] first hidden unit of each workgroup (gu_unit0)
};

// Rows of each matrix one workgroup owns (a contiguous block), and LDS sizes.
struct Blocks {
    int qkv;    // rows of the stacked [Wq; Wk; Wv], even
    int o;      // rows of Wo
    int gu;     // hidden units (one gate row and one up row each) of a workgroup from gu_split on, before the table's scaling
    int gu_a;   // the same of each of the first gu_split workgroups (those that hold the attention items of a short
    int gu_split;   // context: they park nothing and own fewer units instead)
    int park_rows;  // gate/up rows a workgroup from gu_split on keeps in LDS instead of streaming them (even; 0: none)
    int park_floats;
    int qkv_by_xcc; // > 0: the stacked [Wq; Wk; Wv] rows are dealt out per XCD, this many KV heads (with their query heads) to each
    int xa_cu_shift;  // att_xcd_item: log2 of the workgroups that share a KV head
    int xa_opc;       // att_xcd_item: attention outputs each of them combines
    int kv_floats;    // LDS behind the parked rows for what the K and V rows of a workgroup's share of a context need beyond them
    int qkv_floats;   // LDS for this token's q (a row per head of an item), k and v rows
    int kv_offset;    // where those rows start, in floats from the start of LDS (inside xs: see plan_for)
    int slice_dim;  // columns per slice of a dim-column row (slice_width)
    int down;   // rows of W2
    int cls;    // rows of the classifier
    int ns_dim, ns_hidden;  // partial sums per row of a dim-column / hidden-column matrix (slices_used)
    float dim_as_float;
    int xs_floats;
    int results_floats;
    int gather_floats;
    int red_floats;   // LDS for the cross-wavefront merge of the attention items
};

// Hidden units of a workgroup: a contiguous run, units first[wg] .. first[wg + 1] - 1 of a table the host makes
// (gu_a units for each of the first gu_split workgroups, gu for the rest, each share then scaled by what a traced
// token says about how fast the workgroup's XCD and kind get through the gate/up phase: calibrate_gateup).
__host__ __device__ inline int gu_unit0(const int* first, int wg) { return first[wg]; }
__host__ __device__ inline int gu_units(const int* first, int wg) { return first[wg + 1] - first[wg]; }
// The last rows of the workgroup's gate/up block are the parked ones.
__host__ __device__ inline int gu_parked_rows(const Blocks& b, int wg, int units) {
    if (wg < b.gu_split) return 0;
    return 2 * units < b.park_rows ? 2 * units : b.park_rows;
}

// Rows of the stacked [Wq; Wk; Wv] (dim + 2 kv_dim rows: q, then k, then v) a workgroup owns.  Plain: workgroup w
// owns rows w * qkv .. w * qkv + qkv - 1.  By XCD (qkv_by_xcc > 0): XCD x owns the rows of KV heads x * qkv_by_xcc ..
// and of the query heads that read them, listed per KV head as [its gqa query heads | its k rows | its v rows], and
// the workgroups of the XCD share that list in blocks of qkv rows: everything an attention item needs of this token
// is then formed on the XCD the item runs on.  qkv_rows() = how many of its block exist; qkv_row() = local row r as
// an index into the stacked matrix.
// (x = the workgroup's XCD, rank = its number within the XCD: wg % n_xcc and wg / n_xcc.)
__host__ __device__ inline int qkv_rows(const Blocks& b, int dim, int kv_dim, int hs, int gqa, int wg, int rank) {
    const int total = b.qkv_by_xcc > 0 ? b.qkv_by_xcc * (gqa + 2) * hs : dim + 2 * kv_dim;
    const int first = (b.qkv_by_xcc > 0 ? rank : wg) * b.qkv;
    const int n = total - first;
    return n < 0 ? 0 : (n > b.qkv ? b.qkv : n);
}
__host__ __device__ inline int qkv_row(const Blocks& b, int dim, int kv_dim, int hs, int gqa, int wg, int x, int rank, int r) {
    if (b.qkv_by_xcc <= 0) return wg * b.qkv + r;
    const int listed = rank * b.qkv + r;
    const int per_kv = (gqa + 2) * hs;
    int j = 0, o = listed;
    if (b.qkv_by_xcc > 1) {  // (the usual case, one KV head per XCD, needs no division)
        j = listed / per_kv;
        o = listed - j * per_kv;
    }
    const int kvh = x * b.qkv_by_xcc + j;
    if (o < gqa * hs) return kvh * gqa * hs + o;
    if (o < (gqa + 1) * hs) return dim + kvh * hs + (o - gqa * hs);
    return dim + kv_dim + kvh * hs + (o - (gqa + 1) * hs);
}

// Workgroup-local coordination words, accessed with relaxed workgroup-scope atomics
// (plain ds_read / ds_write): LDS executes one wavefront's operations in order, so a
// flag written after data is seen after the data.
struct Control {
    unsigned staged;                 // += 1 by every exchange wavefront once it has staged a GEMV phase
    unsigned received;               // += 1 by every exchange wavefront once the inputs of a phase (attention included) are in
    unsigned io_bar;                 // arrival counter of the exchange wavefronts' barrier
    alignas(16) unsigned progress[kGemvWaves];   // GEMV phases wavefront j has completed
    float red[2][kIoWaves];
    float redv[2][kIoWaves];
    int redi[2][kIoWaves];
    float wave_tot[kIoWaves];
    int wave_found[kIoWaves];
    int target, token;
    unsigned error;                  // an LDS wait gave up (reported by the exchange wavefronts at the end)
    unsigned long long gemv_mark[2]; // timeline: streaming wavefront 0 saw the staged flag / finished its last row
};

// (relaxed workgroup-scope atomics rather than volatile: they keep the LDS address
// space, so they compile to plain ds_read / ds_write, and are never hoisted)
template <class T>
__device__ __forceinline__ T lds_ld(const T* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ unsigned lds_peek(const unsigned* p) { return lds_ld(p); }
__device__ __forceinline__ void lds_poke(unsigned* p, unsigned v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }
// A load that stays where it is written.  (An ordinary load whose value is first used behind
// a wait loop is moved down to that use by the optimiser; fencing it in place with a memory
// clobber instead makes the compiler wait for it on the spot and park it in private memory.)
// The request is issued here and waited for at the first use of the value.
__device__ __forceinline__ float pinned_load(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
}
// (two plain floats, not a float2: an object of class type that meets another one in a
// conditional expression is selected by address and has to live in private memory for that)
__device__ __forceinline__ void pinned_load(const float2* p, float& x, float& y) {
    const unsigned long long bits =
        __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    x = __uint_as_float(static_cast<unsigned>(bits));
    y = __uint_as_float(static_cast<unsigned>(bits >> 32));
}

// Waits on LDS words are satisfied by construction (neither kind of wavefront
// ever waits for global memory before raising them); the bound only makes sure a
// mistake in that reasoning ends as a reported error instead of a hung device.
constexpr unsigned kLdsSpinLimit = 1u << 22;
template <class Ready>
__device__ __forceinline__ void lds_wait(unsigned* error_word, Ready ready) {
    unsigned spins = 0;
    while (!ready()) {
        if (++spins > kLdsSpinLimit) {
            lds_poke(error_word, 2u);  // LDS, not global: a store in flight would spoil the streaming wavefronts' load counting
            break;
        }
        __builtin_amdgcn_s_sleep(2);
    }
}

struct Ctx {
    const DecodeArgs& a;
    const Tagged& t;
    const Blocks& b;
    Control& ctl;
    unsigned base;  // sequence-number base of this token
    unsigned long long* trace;
    unsigned phase_index;
    // Step parameters as they stood when the kernel started.  The workgroup that
    // finishes the token rewrites them while slower workgroups are still in the
    // sampler, so nothing reads them from memory after the first phase began.
    int token, pos, history_len;
    float temperature, penalty, r;
    int wg, nwg;
    int xcc, rank_in_xcc;  // the XCD this workgroup runs on and its index among that XCD's workgroups
    int gu0, gun;          // this workgroup's hidden units: first, count

    __device__ __forceinline__ unsigned seq(int layer, int phase) const {
        return base + 1u + 5u * static_cast<unsigned>(layer) + static_cast<unsigned>(phase);
    }
    __device__ __forceinline__ unsigned seq_stats() const { return base + 1u + 5u * static_cast<unsigned>(a.n_layers); }
};

// x / head_size without the two dozen instructions of a run-time integer division (x < 2^25).
__device__ __forceinline__ int div_head_size(const Ctx& c, int x) {
    return static_cast<int>(__umulhi(static_cast<unsigned>(x), c.t.hs_magic));
}

__host__ __device__ inline unsigned phases_per_token(int n_layers) { return 5u * n_layers + 2u; }
// Timeline marks per phase (workgroup 0): 0 phase entered, 1 own inputs received,
// 2 inputs staged, 3 streaming wavefronts done, 4 outputs published (exchange
// thread 0); 5 staged flag seen, 6 last row done (streaming wavefront 0).
constexpr unsigned kTraceMarks = 8;
enum { kQkv = 0, kAtt = 1, kOproj = 2, kGateUp = 3, kDown = 4 };
// GEMV phases as the streaming wavefronts count them: 4 per layer, then the classifier.
enum { kGQkv = 0, kGO = 1, kGGateUp = 2, kGDown = 3, kGCls = 4 };

// ---------------------------------------------------------------------------
// Streaming wavefronts
// ---------------------------------------------------------------------------

// The order in which a streaming wavefront needs its weights is fixed by the
// model's shape, so the host lists it once: for every (workgroup, wavefront) the
// 4-KiB steps it will request, in order, across all GEMV phases of a token.
// A step is one row of the workgroup's block restricted to one column slice of
// at most kStepLoads chunks; in any one phase a wavefront works on a single
// slice, so it takes its part of the activation vector from LDS into registers
// once per phase and every step after that is multiply-adds between registers.
// (Reading the activations from LDS for every row instead makes the phase
// LDS-bandwidth bound: 8 bytes of activations for every 2 bytes of weights.)
// A row cut into several slices yields one partial sum per slice, added up by
// the exchange wavefronts in slice order.
//
// The wavefront reads its list 64 entries at a time (one entry per lane, one
// coalesced load that travels in the same in-order stream as the weights and
// is requested a whole batch ahead) and picks the entry of a step with a lane
// read.  Scalar loads would not do: they share a completion counter with LDS,
// so every wait for activations would also wait for the list.
struct StepEntry {
    unsigned long long ptr;  // first byte of the step: row start + first column of the slice
    unsigned meta;           // result slot | phase << 16 | flags
    unsigned cols;           // first column of the slice | columns of it that exist << 16
};
constexpr unsigned kStepLastRow = 1u << 29;  // this wavefront's last step of the phase
constexpr unsigned kStepValid = 1u << 31;    // cleared in the terminating entries
constexpr unsigned kStepPhaseShift = 16, kStepPhaseMask = 0x3ffu, kStepSlotMask = 0xffffu;
constexpr int kStepBatch = 64;  // entries per batch: a multiple of kDepth, at most one per lane
constexpr int kMaxSlices = kGemvWaves;

// Column slices of a d-column matrix: a power of two, at most one per streaming
// wavefront, each at most kStepLoads chunks wide.
__host__ __device__ inline int slice_count(int d, int chunk_cols) {
    const int step_cols = kStepLoads * chunk_cols;
    int n = 1;
    while (n * step_cols < d && n < kMaxSlices) n *= 2;
    return n;
}
__host__ __device__ inline int slice_width(int d, int chunk_cols) {
    const int n = slice_count(d, chunk_cols);
    const int per = (d + n - 1) / n;
    return (per + 255) / 256 * 256;  // a slice starts on a multiple of 256 columns (pack_cols)
}
// Slices that actually hold columns (rounding the width up can leave the last ones empty): a
// row's partial sums are results[row * slices_used + slice].
__host__ __device__ inline int slices_used(int d, int chunk_cols) {
    const int width = slice_width(d, chunk_cols);
    return (d + width - 1) / width;
}

template <bool kF16>
__device__ __forceinline__ void gemv_role(const DecodeArgs& a, Control& ctl, const uint4* __restrict__ steps, int j,
                                          const float* xs, float* results, bool trace_on) {
    constexpr int kPer = WTraits<kF16>::kPerLoad;
    constexpr int kBytes = WTraits<kF16>::kBytes;
    constexpr int kChunkCols = kWave * kPer;
    static_assert(kStepBatch % kDepth == 0, "batches change between rounds of the ring");
    typedef const char __attribute__((address_space(1)))* GlobalBytes;  // not generic pointers: plain global loads
    typedef const uintx4 __attribute__((address_space(1)))* GlobalVec;
    const int lane = lane_id();
    const unsigned n_phases = 4u * static_cast<unsigned>(a.n_layers) + 1u;
    const GlobalVec list = reinterpret_cast<GlobalVec>(reinterpret_cast<unsigned long long>(steps));

    uintx4 batch_a = list[lane];               // entries of the steps being requested now, one per lane
    uintx4 batch_b = list[kStepBatch + lane];  // the batch after it, requested a whole batch ahead
    uintx4 w[kDepth][kStepLoads];
    unsigned meta[kDepth];  // StepEntry::meta of the step held in w[k]
    unsigned cols[kDepth];  // StepEntry::cols

    // The loads of the step whose first byte is lo | hi << 32 into ring slot k (cols[k] describes its slice).
    auto request_at = [&](int k, unsigned lo, unsigned hi) {
        const GlobalBytes ptr =
            reinterpret_cast<GlobalBytes>(static_cast<unsigned long long>(lo) | (static_cast<unsigned long long>(hi) << 32));
        const int width = static_cast<int>(cols[k] >> 16);
#pragma unroll
        for (int u = 0; u < kStepLoads; ++u) {
            const int local = u * kChunkCols + lane * kPer;  // column inside the slice
            const int safe = (local < width) ? local : 0;    // lanes past the slice re-read its start; their activations are 0
            w[k][u] = __builtin_nontemporal_load(reinterpret_cast<GlobalVec>(ptr + static_cast<size_t>(safe) * kBytes));
        }
    };
    auto request = [&](int k, const uintx4& batch, int slot) {
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(batch[0]), slot));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(batch[1]), slot));
        meta[k] = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(batch[2]), slot));
        cols[k] = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(batch[3]), slot));
        request_at(k, lo, hi);
    };
#pragma unroll
    for (int k = 0; k < kDepth; ++k) request(k, batch_a, k);
    {
        const unsigned first = (meta[0] & kStepValid) ? ((meta[0] >> kStepPhaseShift) & kStepPhaseMask) : n_phases;
        if (lane == 0) lds_poke(&ctl.progress[j], first);
    }

    unsigned cur_p = 0xffffffffu;
    floatx4 xr[kStepLoads][kF16 ? 2 : 1];  // this wavefront's slice of the staged activations
    bool more = true;
    // Multiply the step held in ring slot k; next_meta = StepEntry::meta of the step after it.
    auto multiply = [&](int k, unsigned next_meta) {
        const unsigned mt = meta[k];
        float part[kStepLoads];  // one chain of multiply-adds per chunk: they overlap instead of queueing up
#pragma unroll
        for (int u = 0; u < kStepLoads; ++u) {
            if constexpr (kF16) part[u] = dot8(w[k][u], xr[u][0], xr[u][1], 0.0f);
            else part[u] = dot4(w[k][u], xr[u][0], 0.0f);
        }
        static_assert(kStepLoads == 4, "the partial sums are added pairwise");
        const float sum = wave_sum((part[0] + part[1]) + (part[2] + part[3]));
        if (lane == 0) results[mt & kStepSlotMask] = sum;
        if (mt & kStepLastRow) {  // everything before the next step's phase is complete
            const unsigned nm = next_meta;
            const unsigned next_p = (nm & kStepValid) ? ((nm >> kStepPhaseShift) & kStepPhaseMask) : n_phases;
            compiler_fence();
            if (lane == 0) lds_poke(&ctl.progress[j], next_p);
            if (trace_on && lane == 0) ctl.gemv_mark[1] = wall_clock64();
        }
    };
    // One pass through the ring: multiply the kDepth steps in flight and request
    // the steps whose entries sit in lanes slot0 .. slot0 + kDepth - 1 of `batch`.
    //
    // When a phase's activations arrive, the ring usually holds several steps of that
    // phase whose weights came in while the wavefront was waiting.  All of them are
    // multiplied before anything new is requested: a compute unit accepts a 4-KiB
    // request only every hundred cycles or so, with eight wavefronts asking at once a
    // request waits its turn for the better part of a microsecond, and rows that only
    // need multiplying would otherwise queue behind requests for later phases.
    unsigned ahead = 0u;  // bit k: the step in slot k has been multiplied already
    unsigned pace = 0u;
    int paced = 0;  // next-phase rows sent out early since the last burst
    constexpr int kPaceSleep = 15;
    auto run_round = [&](const uintx4& batch, int slot0) {
#pragma unroll
        for (int k = 0; k < kDepth; ++k) {
            const unsigned mt = meta[k];
            if (more && (mt & kStepValid)) {
                if (((ahead >> k) & 1u) == 0u) {
                    const unsigned p = (mt >> kStepPhaseShift) & kStepPhaseMask;
                    const bool phase_start = p != cur_p;
                    if (phase_start) {  // first step of a phase: wait for its activations, take this wavefront's slice
                        cur_p = p;
                        const unsigned need = static_cast<unsigned>(kIoWaves) * (p + 1u);
                        lds_wait(&ctl.error, [&]() { return static_cast<int>(lds_peek(&ctl.staged) - need) >= 0; });
                        compiler_fence();
                        if (trace_on && lane == 0) ctl.gemv_mark[0] = wall_clock64();
                        const int begin = static_cast<int>(cols[k] & 0xffffu), width = static_cast<int>(cols[k] >> 16);
                        const floatx4 zero = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int u = 0; u < kStepLoads; ++u) {
                            const int local = u * kChunkCols + lane * kPer;
                            const bool live = local < width;
                            const float* src = xs + begin + (live ? local : 0);
                            xr[u][0] = *reinterpret_cast<const floatx4*>(src);
                            xr[u][0] = live ? xr[u][0] : zero;
                            if constexpr (kF16) {
                                xr[u][1] = *reinterpret_cast<const floatx4*>(src + 4);
                                xr[u][1] = live ? xr[u][1] : zero;
                            }
                        }
                    }
                    multiply(k, meta[(k + 1) % kDepth]);
                    if (phase_start) {  // the steps of this phase behind it in the ring, oldest first
                        // The refills are spaced out only when this burst was all the wavefront had to do in
                        // the phase: the exchange wavefronts publish next, and their stores should not queue
                        // behind eight wavefronts' requests.  In a longer phase the requests are this phase's
                        // own rows and go out at once.
                        unsigned burst = 1u << k;
                        bool ended = (mt & kStepLastRow) != 0u;
                        bool same = true;
#pragma unroll
                        for (int i = 1; i < kDepth; ++i) {
                            const int kk = (k + i) % kDepth;
                            const unsigned m2 = meta[kk];
                            same = same && (m2 & kStepValid) && ((m2 >> kStepPhaseShift) & kStepPhaseMask) == p;
                            if (same) {
                                // (the step after the newest one in the ring is the one slot k is about to request)
                                const unsigned after =
                                    (i + 1 < kDepth)
                                        ? meta[(kk + 1) % kDepth]
                                        : static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(batch[2]), slot0 + k));
                                multiply(kk, after);
                                ahead |= 1u << kk;
                                burst |= 1u << kk;
                                ended = ended || (m2 & kStepLastRow) != 0u;
                            }
                        }
                        if (ended) {
                            pace |= burst;
                            paced = 0;
                        }
                    }
                }
                ahead &= ~(1u << k);
            } else {
                more = false;
            }
            if ((pace >> k) & 1u) {
                // A refill after a burst that finished the wavefront's rows of phase cur_p.  A row of the
                // very next GEMV phase goes out after a short pause, right behind the publishing stores
                // (it must be there when that phase's inputs are), and so does a second one; not more: where a
                // wavefront's whole ring was one phase's rows, as at dim 4096, four refills of the next phase
                // would put 128 KiB per compute unit in front of the polls.  Anything else is held until the inputs
                // of the phase after this one have arrived: from then until that phase publishes, nothing
                // of this workgroup's is on its way through the memory system, and a request costs no
                // hand-over anything; sent now, it would sit in the queues in front of the values being
                // handed over.
                pace &= ~(1u << k);
                const unsigned nm = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(batch[2]), slot0 + k));
                const unsigned nq = (nm >> kStepPhaseShift) & kStepPhaseMask;
                if ((nm & kStepValid) == 0u) {
                    // past the wavefront's last step: nothing left to hold back
                } else if (nq == cur_p + 1u && paced < kPacedSteps) {
                    ++paced;
                    __builtin_amdgcn_s_sleep(kPaceSleep);
                } else {
                    // phases in the exchange wavefronts' count (five per layer): qkv, attention, O, gate/up, down
                    const unsigned io_phase = 5u * (cur_p >> 2) + ((cur_p & 3u) == 0u ? 0u : (cur_p & 3u) + 1u);
                    const unsigned need = static_cast<unsigned>(kIoWaves) * (io_phase + 2u);
                    lds_wait(&ctl.error, [&]() { return static_cast<int>(lds_peek(&ctl.received) - need) >= 0; });
                    compiler_fence();
                }
            }
            request(k, batch, slot0 + k);
        }
    };
    // The two entry batches take turns; each is re-requested, straight into its own
    // registers, the moment its last entry has been used: a whole batch ahead.
    constexpr int kRoundsPerBatch = kStepBatch / kDepth;
    int next_batch = 2;
    int first_round = 1;  // the priming requests were round 0 of the first batch
    while (more) {
        for (int r = first_round; r < kRoundsPerBatch && more; ++r) run_round(batch_a, r * kDepth);
        first_round = 0;
        batch_a = list[next_batch * kStepBatch + lane];
        for (int r = 0; r < kRoundsPerBatch && more; ++r) run_round(batch_b, r * kDepth);
        batch_b = list[(next_batch + 1) * kStepBatch + lane];
        next_batch += 2;
    }
}

// ---------------------------------------------------------------------------
// Exchange wavefronts: synchronisation among themselves
// ---------------------------------------------------------------------------

// Index of the calling thread among the exchange threads, computed from scratch (two
// instructions the optimiser can neither hoist nor share).  Code that needs the index forms
// it where it is needed: a copy kept in a register from phase to phase does not survive the
// busiest stretches, and every reload from spill memory is a wait for all of the wavefront's
// outstanding memory operations -- the publishing stores' acknowledgements among them, which
// take microseconds.
__device__ __forceinline__ int exchange_thread_index(int iw) {
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return iw * kWave + lane;
}

// Lane exchange with an explicitly supplied lane index (byte address of the partner = (lane ^
// offset) * 4).  __shfl_xor works the index out from a value the optimiser keeps for the whole
// kernel; callers here pass one made with fresh_lane() where the exchanges happen.
__device__ __forceinline__ int fresh_lane() {
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}
__device__ __forceinline__ float lane_xor(float v, int offset, int lane) {
    return __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ offset) << 2, __float_as_int(v)));
}

struct Io {
    int it;        // thread index among the exchange threads
    int iw;        // exchange wavefront index
    unsigned gen;  // barrier generation
    int parity;    // reduction slot parity
    StepParams* step;
};

__device__ __forceinline__ void io_sync(Control& ctl, Io& io) {
    compiler_fence();
    io.gen += static_cast<unsigned>(kIoWaves);
    if (lane_id() == 0) __hip_atomic_fetch_add(&ctl.io_bar, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    const unsigned gen = io.gen;
    lds_wait(&ctl.error, [&]() { return static_cast<int>(lds_peek(&ctl.io_bar) - gen) >= 0; });
    compiler_fence();
}

// Sum over all exchange threads; every thread gets the total (wavefront order).
__device__ __forceinline__ float io_sum(Control& ctl, Io& io, float v) {
    const float s = wave_sum(v);
    float* slot = ctl.red[io.parity];
    if (lane_id() == 0) slot[io.iw] = s;
    io_sync(ctl, io);
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kIoWaves; ++w) total += lds_ld(slot + w);
    io.parity ^= 1;
    return total;
}
__device__ __forceinline__ float io_max(Control& ctl, Io& io, float v) {
    const float s = wave_max(v);
    float* slot = ctl.red[io.parity];
    if (lane_id() == 0) slot[io.iw] = s;
    io_sync(ctl, io);
    float total = lds_ld(slot);
#pragma unroll
    for (int w = 1; w < kIoWaves; ++w) total = fmaxf(total, lds_ld(slot + w));
    io.parity ^= 1;
    return total;
}

__device__ __forceinline__ void signal_staged(Control& ctl) {
    compiler_fence();
    if (lane_id() == 0) __hip_atomic_fetch_add(&ctl.staged, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// The inputs of the current phase have arrived: for a while now nothing of this workgroup's is on
// its way through the memory system, which is when the streaming wavefronts let held-back requests go.
__device__ __forceinline__ void signal_received(Control& ctl) {
    if (lane_id() == 0) __hip_atomic_fetch_add(&ctl.received, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Wait until every streaming wavefront has completed GEMV phase p.
__device__ __forceinline__ void wait_gemv(Control& ctl, int p) {
    const unsigned need = static_cast<unsigned>(p + 1);
    static_assert((kGemvWaves & (kGemvWaves - 1)) == 0, "lanes share the progress words by their low bits");
    // One word per lane, one comparison per look: while the exchange wavefronts wait here the streaming
    // wavefronts on the same SIMDs are multiplying, and every vector instruction of the wait is one they do not issue.
    const unsigned* mine = &ctl.progress[fresh_lane() & (kGemvWaves - 1)];
    lds_wait(&ctl.error, [&]() { return __builtin_amdgcn_ballot_w64(lds_ld(mine) < need) == 0ull; });
    compiler_fence();
}

__device__ __forceinline__ void mark(Ctx& c, const Io& io, int which) {
    if (c.trace && io.it == 0) {
        c.trace[kTraceMarks * c.phase_index + which] = wall_clock64();
        if (which == 4 && c.phase_index % 5u != 1u) {  // the streaming wavefront's marks of this phase are final by now
            c.trace[kTraceMarks * c.phase_index + 5] = c.ctl.gemv_mark[0];
            c.trace[kTraceMarks * c.phase_index + 6] = c.ctl.gemv_mark[1];
        }
    }
}

// ---------------------------------------------------------------------------
// Polling
// ---------------------------------------------------------------------------

// What went wrong in a launch, for the host: 1 a wait for tagged values ran out, 2 an LDS wait did, 3 an XCD was
// dealt more than its share of the workgroups.  The highest code reported stays (the host's recovery differs for 3).
__device__ __forceinline__ void report_error(StepParams* step, int code) {
    __hip_atomic_fetch_max(&step->error, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ bool poll_give_up(const Ctx& c, unsigned& spins) {
    if ((spins & 63u) == 63u && __hip_atomic_load(c.t.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u) return true;
    if (++spins > c.t.spin_limit) {
        __hip_atomic_store(c.t.abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        report_error(c.a.step, 1);
        return true;
    }
    __builtin_amdgcn_s_sleep(1);
    return false;
}

// Fetch n tagged values carrying sequence number `want` and hand each to
// sink(i, value, j, first_round), where i = thread index + (round * kBatch + j) *
// kIoThreads and j is a constant of the unrolled code; the exchange threads share
// the range.  A thread requests up
// to kPollBatch values, then re-requests only those that were not there yet.
template <int kBatch = kPollBatch, class Sink>
__device__ __forceinline__ void poll_values(const u64* src, int n, unsigned want, const Ctx& c, const Io& io, Sink sink) {
    // (opaque to the optimiser: otherwise the addresses of every poll in the layer loop are
    // computed once, ahead of the loop, and occupy registers for the whole token)
    const int lane_first = exchange_thread_index(io.iw);
    for (int first = lane_first; first < n; first += kIoThreads * kBatch) {
        u64 got[kBatch];
        unsigned pending = 0u;
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int i = first + j * kIoThreads;
            if (i < n) {
                got[j] = peek(src + i);
                pending |= 1u << j;
            }
        }
        unsigned spins = 0;
        while (true) {
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                if ((pending >> j) & 1u)
                    if (tag_of(got[j]) == want) pending &= ~(1u << j);
            if (pending == 0u) break;
            if (poll_give_up(c, spins)) break;
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                if ((pending >> j) & 1u) got[j] = peek(src + first + j * kIoThreads);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const int i = first + j * kIoThreads;
            if (i < n) sink(i, value_of(got[j]), j, first == lane_first);
        }
    }
}

// N tagged values per thread at addresses addr(j), all requested at once.
template <int N, class AddrFn>
__device__ __forceinline__ void poll_n(AddrFn addr, float (&out)[N], unsigned want, const Ctx& c) {
    static_assert(N <= 32, "pending mask is 32 bits");
    u64 got[N];
#pragma unroll
    for (int j = 0; j < N; ++j) got[j] = peek(addr(j));
    unsigned pending = (N == 32) ? 0xffffffffu : ((1u << N) - 1u);
    unsigned spins = 0;
    while (true) {
#pragma unroll
        for (int j = 0; j < N; ++j)
            if ((pending >> j) & 1u)
                if (tag_of(got[j]) == want) pending &= ~(1u << j);
        if (pending == 0u) break;
        if (poll_give_up(c, spins)) break;
#pragma unroll
        for (int j = 0; j < N; ++j)
            if ((pending >> j) & 1u) got[j] = peek(addr(j));
    }
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = value_of(got[j]);
}

// Two values per thread from slots inside this XCD's own copy (peek_near), both requested at once.
template <class AddrFn>
__device__ __forceinline__ void poll_near_2(AddrFn addr, float (&out)[2], unsigned want, const Ctx& c) {
    const u64* p0 = addr(0);
    const u64* p1 = addr(1);
    u64 g0, g1;
    unsigned spins = 0;
    while (true) {
        asm volatile("global_load_dwordx2 %0, %2, off nt\n\tglobal_load_dwordx2 %1, %3, off nt\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(g0), "=&v"(g1)
                     : "v"(p0), "v"(p1)
                     : "memory");
        if (tag_of(g0) == want && tag_of(g1) == want) break;
        if (poll_give_up(c, spins)) break;
    }
    out[0] = value_of(g0);
    out[1] = value_of(g1);
}

// The XCD a wavefront runs on.
__device__ __forceinline__ int hardware_xcc() {
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return static_cast<int>(v & 0xfu);
}

// A long vector every workgroup needs in full (the SwiGLU output), fetched in two hops.  Polled
// directly, each of the 256 compute units pulls the whole vector across the fabric between the
// XCDs, again for every attempt that comes too early: two megabytes per XCD and attempt at 8192
// values.  Here the workgroups of an XCD share that work: workgroup r of the XCD polls slice r of the vector (device scope, as before) and stores it,
// tags included, into a copy of the vector that belongs to its XCD; every workgroup then polls that
// copy.  Those stores stay in the XCD's own L2 (plain stores; a device-scope store would write
// through and drop the line), and the polls are non-temporal loads, which the compute unit's L1
// does not keep: they are served by the L2 the stores went to.  Nothing outside the XCD ever
// touches its copy, so the L2 needs no help to stay coherent.  A stale line anywhere can only
// delay a poll (a value is taken when it carries the expected sequence number), not corrupt it.
// Measured at the 1B shape: the down projection's inputs arrive 0.8 us sooner per layer; the
// dim-sized vectors (2048 to 4096 values) gain nothing from the second hop and stay with direct polls.
constexpr unsigned kNearPatience = 1024;  // polls of the near copy before a thread turns to the vector itself
template <class Sink>
__device__ __forceinline__ void gather_values(const u64* src, u64* near_all, int near_stride, int share, int n, unsigned want,
                                              const Ctx& c, const Io& io, Sink sink) {
    const int it = exchange_thread_index(io.iw);
    u64* near = near_all + static_cast<size_t>(c.xcc) * near_stride;
    for (int e = it; e < share; e += kIoThreads) {
        const int i = c.rank_in_xcc * share + e;
        if (i < n) {
            u64 got;
            unsigned spins = 0;
            while (true) {
                got = peek(src + i);
                if (tag_of(got) == want) break;
                if (poll_give_up(c, spins)) break;
            }
            asm volatile("global_store_dwordx2 %0, %1, off" ::"v"(near + i), "v"(got) : "memory");
        }
    }
    for (int first = it; first < n; first += 4 * kIoThreads) {
        // (addresses past the end re-read the thread's first value; their results are dropped)
        const u64* p0 = near + first;
        const u64* p1 = near + (first + kIoThreads < n ? first + kIoThreads : first);
        const u64* p2 = near + (first + 2 * kIoThreads < n ? first + 2 * kIoThreads : first);
        const u64* p3 = near + (first + 3 * kIoThreads < n ? first + 3 * kIoThreads : first);
        u64 g0, g1, g2, g3;
        unsigned spins = 0;
        while (true) {
            if (spins <= kNearPatience) {
                // (one statement, the wait included: the compiler sees the results only once they are in)
                asm volatile(
                    "global_load_dwordx2 %0, %4, off nt\n\t"
                    "global_load_dwordx2 %1, %5, off nt\n\t"
                    "global_load_dwordx2 %2, %6, off nt\n\t"
                    "global_load_dwordx2 %3, %7, off nt\n\t"
                    "s_waitcnt vmcnt(0)"
                    : "=&v"(g0), "=&v"(g1), "=&v"(g2), "=&v"(g3)
                    : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
                    : "memory");
            } else {
                // The near copy has not filled: should the workgroups ever not be spread over the XCDs the way the
                // slices assume, the vector itself is still where it always was.
                g0 = peek(src + (p0 - near));
                g1 = peek(src + (p1 - near));
                g2 = peek(src + (p2 - near));
                g3 = peek(src + (p3 - near));
            }
            if (tag_of(g0) == want && tag_of(g1) == want && tag_of(g2) == want && tag_of(g3) == want) break;
            if (poll_give_up(c, spins)) break;
        }
        const bool first_round = first == it;
        sink(first, value_of(g0), 0, first_round);
        if (first + kIoThreads < n) sink(first + kIoThreads, value_of(g1), 1, first_round);
        if (first + 2 * kIoThreads < n) sink(first + 2 * kIoThreads, value_of(g2), 2, first_round);
        if (first + 3 * kIoThreads < n) sink(first + 3 * kIoThreads, value_of(g3), 3, first_round);
    }
}

// ---------------------------------------------------------------------------
// Staging (exchange wavefronts)
// ---------------------------------------------------------------------------

struct Lds {
    float* xraw;     // [dim_pad]   residual stream as last received
    float* xs;       // [xs_floats] staged GEMV input; sampler tables after the classifier
    float* results;  // [results_floats] row results of the current GEMV phase
    float* sc;       // [2 * kAttScoreFloats] the sampler's copy of the penalty window (as ints)
    float* qkv;      // [kMaxAttHeads + 2][kMaxHeadPad] this token's q (per head of the item), k, v
    float* red;      // [kIoWaves][kMaxAttHeads][kRedStride] attention cross-wavefront reduction
    float* gather;   // [gather_floats] attention split partials
    float* park;     // [park_floats] parked gate/up rows (binary16), row after row
    float* kv;       // [kv_floats] K and V rows of this workgroup's share of a KV head's context (att_xcd_item)
    unsigned kv_lds; // the same area as an LDS byte address (what M0 takes for loads that land in LDS)
};

// xs = the tagged vector itself, zero padded to a multiple of 8.  (The streaming
// wavefronts are done with the previous contents: every exchange wavefront waited
// for all of them before publishing.)
// (near_all: the per-XCD copies of this vector, or nullptr for one that is polled directly)
__device__ __forceinline__ void stage_tagged(Ctx& c, Io& io, float* xs, const u64* src, u64* near_all, int near_stride, int share,
                                             int n, unsigned want) {
    const int n_pad = (n + 7) & ~7;
    for (int i = n + io.it; i < n_pad; i += kIoThreads) xs[i] = 0.0f;
    if (near_all != nullptr && c.t.n_xcc > 1)
        gather_values(src, near_all, near_stride, share, n, want, c, io, [&](int i, float v, int, bool) { xs[i] = v; });
    else
        poll_values<kPollBatch>(src, n, want, c, io, [&](int i, float v, int, bool) { xs[i] = v; });
    mark(c, io, 1);
    signal_received(c.ctl);
    signal_staged(c.ctl);
}

// xraw = the input vector (tagged x, or the embedding row for layer 0);
// xs = xraw * gain, and the return value is 1 / sqrt(mean(xraw^2) + 1e-5): the rows of
// the GEMV that follows are those of ops.cpp:20-32 once multiplied by it.  (W.(s.g.x) =
// s.(W.(g.x)): the streaming wavefronts can start the moment the last value is in,
// without waiting for a sum over all of them, a reduction across the exchange
// wavefronts that would otherwise sit in every layer's dependency chain twice; it
// now runs while they multiply.)
__device__ __forceinline__ float stage_norm(Ctx& c, Io& io, const Lds& l, const u64* tagged_x, const float* plain_x, int n,
                                            unsigned want, const float* gain) {
#pragma clang fp contract(off)
    float* xraw = l.xraw;
    float* xs = l.xs;
    const int it = exchange_thread_index(io.iw);
    // The gains do not depend on anything: request this thread's first few before polling, so that
    // their memory latency is spent while the inputs are still on their way.
    constexpr int kEarly = 4;
    float early_gain[kEarly];
#pragma unroll
    for (int e = 0; e < kEarly; ++e) {
        const int i = it + e * kIoThreads;
        early_gain[e] = (i < n) ? pinned_load(gain + i) : 0.0f;
    }
    const int n_pad = (n + 7) & ~7;
    for (int i = n + it; i < n_pad; i += kIoThreads) xs[i] = 0.0f;
    float ss = 0.0f;
    auto take = [&](int i, float v, float g) {
        xraw[i] = v;
        xs[i] = v * g;
        ss += v * v;
    };
    if (plain_x != nullptr) {
#pragma unroll
        for (int e = 0; e < kEarly; ++e) {
            const int i = it + e * kIoThreads;
            if (i < n) take(i, plain_x[i], early_gain[e]);
        }
        for (int i = it + kEarly * kIoThreads; i < n; i += kIoThreads) take(i, plain_x[i], gain[i]);
    } else {
        // (the first round of polls covers exactly the values whose gains were requested early)
        poll_values<kEarly>(tagged_x, n, want, c, io,
                    [&](int i, float v, int j, bool first_round) { take(i, v, first_round ? early_gain[j] : gain[i]); });
    }
    mark(c, io, 1);
    signal_received(c.ctl);
    signal_staged(c.ctl);
    ss = io_sum(c.ctl, io, ss);
    ss /= c.b.dim_as_float;  // n, converted on the host: here the conversion's result would be kept in (and spilled from) a vector register
    ss += 1e-5f;
    return 1.0f / sqrtf(ss);
}

// ---------------------------------------------------------------------------
// GEMV phases as the exchange wavefronts see them
// ---------------------------------------------------------------------------

// Dot product of local row r: its column slices' partial sums, in slice order.
__device__ __forceinline__ float row_result(const float* results, int r, int nslices) {
    float v = results[r * nslices];
    for (int s = 1; s < nslices; ++s) v += results[r * nslices + s];
    return v;
}

// Run fn(r) for the local rows r < nrows of GEMV phase `gphase` once the streaming
// wavefronts have finished it.  (Letting each exchange wavefront go ahead with the
// rows of "its" streaming wavefronts was tried: it starts the next phase's polling
// earlier, and the extra polling traffic cost more than the head start gained.)
template <class RowFn>
__device__ __forceinline__ void finished_rows(Ctx& c, Io& io, int gphase, int nrows, RowFn fn) {
    wait_gemv(c.ctl, gphase);
    mark(c, io, 3);
    for (int r = exchange_thread_index(io.iw); r < nrows; r += kIoThreads) fn(r);
}

__device__ __forceinline__ int block_rows(int total, int block, int wg) {
    const int n = total - wg * block;
    return n < 0 ? 0 : (n > block ? block : n);
}

// (defined with the attention items below)
template <int kHs>
__device__ __forceinline__ void xcd_att_prefetch(const Ctx& c, const Io& io, const Lds& l, int layer);

template <bool kXcd>
__device__ __forceinline__ void io_qkv(Ctx& c, Io& io, const Lds& l, int layer) {
#pragma clang fp contract(off)
    const DecodeArgs& a = c.a;
    const int dim = a.dim, kv_dim = a.kv_dim, hs = a.head_size;
    auto mod_hs = [&](int x) { return x - div_head_size(c, x) * hs; };
    const float* emb_row = (layer == 0) ? a.emb + static_cast<size_t>(c.token) * dim : nullptr;
    mark(c, io, 0);
    const float scale = stage_norm(c, io, l, c.t.x, emb_row, dim, layer == 0 ? 0u : c.seq(layer - 1, kDown),
                                   a.rms_att + static_cast<size_t>(layer) * dim);
    mark(c, io, 2);
    const int nrows = qkv_rows(c.b, dim, kv_dim, hs, a.gqa, c.wg, c.rank_in_xcc);
    const float2* cs_row = a.rope + static_cast<size_t>(c.pos) * (hs / 2);
    const unsigned tag = c.seq(layer, kQkv);
    // (cos, sin) of this thread's first row: requested while the streaming wavefronts still multiply
    const int first_row = io.it;
    const int first_g = first_row < nrows ? qkv_row(c.b, dim, kv_dim, hs, a.gqa, c.wg, c.xcc, c.rank_in_xcc, first_row) : 0;
    const bool first_rotates = first_row < nrows && first_g < dim + kv_dim;
    u64* near = c.t.local_qkv ? c.t.near_qkv + static_cast<size_t>(c.xcc) * c.t.near_qkv_stride : nullptr;
    // (a valid address either way, so that the request does not sit behind a branch)
    float first_cos, first_sin;
    pinned_load(cs_row + (first_rotates ? mod_hs(((first_g < dim) ? first_g : first_g - dim) & ~1) >> 1 : 0), first_cos, first_sin);
    // This layer's share of the context, on its way into LDS while the rows of this phase are multiplied: the phase
    // is bound by latency, the memory system has room for the bytes, and the attention's inputs are three
    // hand-over steps away.  (Requested a layer ahead, during the gate/up phase, the same bytes make that phase,
    // which is bound by bandwidth, longer by more than they take here.)
    if constexpr (kXcd) {
        if (c.t.xa_chunk > 0) {
            if (hs == 64) xcd_att_prefetch<64>(c, io, l, layer);
            else xcd_att_prefetch<128>(c, io, l, layer);
        }
    }
    // (a plain loop, not finished_rows with a closure: a local captured by reference is kept in
    // private memory across the wait, and private memory shares the load counter)
    wait_gemv(c.ctl, 4 * layer + kGQkv);
    mark(c, io, 3);
    for (int r = exchange_thread_index(io.iw); r < nrows; r += kIoThreads) {
        const int g = qkv_row(c.b, dim, kv_dim, hs, a.gqa, c.wg, c.xcc, c.rank_in_xcc, r);
        const float mine = row_result(l.results, r, c.b.ns_dim) * scale,
                    neighbour = row_result(l.results, r ^ 1, c.b.ns_dim) * scale;
        float out = mine;
        if (g < dim + kv_dim) {  // ops.cpp:36-52 on the pair (i, i+1)
            const int gi = (g < dim) ? g : g - dim;
            float cos_t = first_cos, sin_t = first_sin;
            if (r != first_row) {
                const float2 cs = cs_row[mod_hs(gi & ~1) >> 1];
                cos_t = cs.x;
                sin_t = cs.y;
            }
            out = (gi & 1) ? neighbour * sin_t + mine * cos_t : mine * cos_t - neighbour * sin_t;
        }
        // (to the attention items: across the chip, or inside this XCD when its items read nothing else)
        if (near != nullptr) publish_near(near + g, out, tag);
        if (g < dim) {
            if (near == nullptr) publish(c.t.q + g, out, tag);
            a.q[g] = out;
        } else {  // model.cpp:171-176 / scatter_kv.cu:15-18
            const bool is_k = g < dim + kv_dim;
            const int i = is_k ? g - dim : g - dim - kv_dim;
            const int head = div_head_size(c, i), within = i - head * hs;
            const size_t dst = static_cast<size_t>(layer) * kv_dim * a.seq_len +
                               static_cast<size_t>(head) * a.seq_len * hs + static_cast<size_t>(c.pos) * hs + within;
            if (near == nullptr) publish((is_k ? c.t.k : c.t.v) + i, out, tag);
            (is_k ? a.k : a.v)[i] = out;
            (is_k ? a.key_cache : a.value_cache)[dst] = f32_to_f16_bits(out);
        }
    }
    mark(c, io, 4);
    ++c.phase_index;
}

// x = xraw + W . src (model.cpp:160,218 and :225-226)
__device__ __forceinline__ void io_proj(Ctx& c, Io& io, const Lds& l, int gphase, int block, int d, int nslices,
                                        const u64* src, u64* near_all, int near_stride, int share, unsigned src_tag,
                                        unsigned out_tag) {
    mark(c, io, 0);
    stage_tagged(c, io, l.xs, src, near_all, near_stride, share, d, src_tag);
    mark(c, io, 2);
    const int row0 = c.wg * block;
    const int nrows = block_rows(c.a.dim, block, c.wg);
    finished_rows(c, io, gphase, nrows, [&](int r) {
        publish(c.t.x + row0 + r, l.xraw[row0 + r] + row_result(l.results, r, nslices), out_tag);
    });
    mark(c, io, 4);
    ++c.phase_index;
}

// Parked gate/up rows.  While the attention runs, most compute units have nothing to do and the memory
// system is nearly idle, but the streaming wavefronts can only run as far ahead as their registers
// reach.  A workgroup without an attention item therefore copies the last park_rows rows of its
// gate/up block into LDS during that time (exchange wavefront w takes parked rows w, w + 8, ...), and
// the same wavefront multiplies them out of LDS while the streaming wavefronts work through the rest
// of the block: those rows are simply absent from the streaming wavefronts' lists.  The sums are formed
// exactly as a streaming wavefront forms them (same lanes, same order), so a row gives the same bits
// whichever way it went.  Once a context is long enough for the attention items to spread beyond the
// first n_heads workgroups, the host launches with the other plan: no parked rows, uniform blocks.
__device__ __forceinline__ void park_fetch(Ctx& c, Io& io, const Lds& l, int layer) {
    const DecodeArgs& a = c.a;
    const int units = c.gun;
    const int parked = gu_parked_rows(c.b, c.wg, units);
    if (parked == 0) return;
    const int first_row = 2 * units - parked;
    const int unit0 = c.gu0;
    const int lane = fresh_lane();
    const int row_bytes = a.dim * 2;
    const int loads_per_row = (row_bytes + 1023) >> 10;  // one wavefront load covers 1 KiB
    const int mine = (parked - io.iw + kIoWaves - 1) / kIoWaves;
    const int total = mine * loads_per_row;
    constexpr int kBatch = 16;
    char* park = reinterpret_cast<char*>(l.park);
    for (int base = 0; base < total; base += kBatch) {
        uintx4 v[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int idx = base + i;
            const int jj = idx / loads_per_row, chunk = idx - jj * loads_per_row;
            const int j = io.iw + jj * kIoWaves;
            const int r = first_row + j;
            const int byte = (chunk << 10) + lane * 16;
            v[i] = uintx4{0u, 0u, 0u, 0u};
            if (idx < total && byte < row_bytes) {
                const char* row = ((r & 1) ? a.w3 : a.w1) +
                                  (static_cast<size_t>(layer) * a.hidden + unit0 + (r >> 1)) * static_cast<size_t>(row_bytes);
                v[i] = load16_stream(row + byte);
            }
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int idx = base + i;
            const int jj = idx / loads_per_row, chunk = idx - jj * loads_per_row;
            const int j = io.iw + jj * kIoWaves;
            const int byte = (chunk << 10) + lane * 16;
            if (idx < total && byte < row_bytes) *reinterpret_cast<uintx4*>(park + static_cast<size_t>(j) * row_bytes + byte) = v[i];
        }
    }
}

// results[row * ns_dim + slice] of the parked rows, from LDS: what a streaming wavefront computes for a step
// (one chain of multiply-adds per 1-KiB chunk, added pairwise, then across the wavefront).
__device__ __forceinline__ void park_multiply(Ctx& c, Io& io, const Lds& l) {
    const DecodeArgs& a = c.a;
    const int units = c.gun;
    const int parked = gu_parked_rows(c.b, c.wg, units);
    if (parked == 0) return;
    const int first_row = 2 * units - parked;
    const int lane = fresh_lane();
    const int row_bytes = a.dim * 2;
    constexpr int kChunkCols = kWave * 8;
    const char* park = reinterpret_cast<const char*>(l.park);
    for (int s = 0; s < c.b.ns_dim; ++s) {
        const int begin = s * c.b.slice_dim;
        const int width = min(c.b.slice_dim, a.dim - begin);
        floatx4 xr[kStepLoads][2];
        const floatx4 zero = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < kStepLoads; ++u) {
            const int local = u * kChunkCols + lane * 8;
            const bool live = local < width;
            const float* src = l.xs + begin + (live ? local : 0);
            xr[u][0] = *reinterpret_cast<const floatx4*>(src);
            xr[u][1] = *reinterpret_cast<const floatx4*>(src + 4);
            xr[u][0] = live ? xr[u][0] : zero;
            xr[u][1] = live ? xr[u][1] : zero;
        }
        for (int j = io.iw; j < parked; j += kIoWaves) {
            const char* row = park + static_cast<size_t>(j) * row_bytes + static_cast<size_t>(begin) * 2;
            float part[kStepLoads];
#pragma unroll
            for (int u = 0; u < kStepLoads; ++u) {
                const int local = u * kChunkCols + lane * 8;
                const uintx4 w = *reinterpret_cast<const uintx4*>(row + static_cast<size_t>(local < width ? local : 0) * 2);
                part[u] = dot8(w, xr[u][0], xr[u][1], 0.0f);
            }
            const float sum = wave_sum((part[0] + part[1]) + (part[2] + part[3]));
            if (lane == 0) l.results[(first_row + j) * c.b.ns_dim + s] = sum;
        }
    }
}

__device__ __forceinline__ void io_gateup(Ctx& c, Io& io, const Lds& l, int layer) {
#pragma clang fp contract(off)
    const DecodeArgs& a = c.a;
    mark(c, io, 0);
    const float scale =
        stage_norm(c, io, l, c.t.x, nullptr, a.dim, c.seq(layer, kOproj), a.rms_ffn + static_cast<size_t>(layer) * a.dim);
    mark(c, io, 2);
    const int unit0 = c.gu0;
    const int units = c.gun;
    const unsigned tag = c.seq(layer, kGateUp);
    if (c.b.park_rows > 0) {
        park_multiply(c, io, l);
        io_sync(c.ctl, io);  // the parked rows' sums are read by other exchange wavefronts below
    }
    finished_rows(c, io, 4 * layer + kGGateUp, 2 * units, [&](int r) {
        if (r & 1) return;  // the gate row's thread finishes the unit
        const int u = r >> 1;
        const float gate = row_result(l.results, r, c.b.ns_dim) * scale, up = row_result(l.results, r + 1, c.b.ns_dim) * scale;
        const float sigma = 1.0f / (1.0f + expf(-gate));  // ops.cpp:80-85
        publish(c.t.hb + unit0 + u, (gate * sigma) * up, tag);
    });
    mark(c, io, 4);
    ++c.phase_index;
}

// ---------------------------------------------------------------------------
// Attention (exchange wavefronts)
// ---------------------------------------------------------------------------

// exp(x) as one hardware exponential.  (About an ulp off expf; the weights it forms are
// normalised by their own sum.)
__device__ __forceinline__ float exp_fast(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }

// One attention work item: kHeads query heads that share a KV head (one head for short contexts
// and for models without grouped queries), context split `split` of `nsplits`.  kGroup lanes cover
// one position, 8 binary16 each.  K and V rows of earlier positions do not depend on this token:
// the first rows are requested before q is polled, each later pass's as soon as the registers are
// free.  The current position's k and v arrive tagged and are rounded to binary16 exactly as the
// cache store rounds them.  Every K and V row of the split is fetched ONCE and used for all kHeads
// heads (per-head items would read it once per head, which at 8K positions is four times the cache
// traffic of the Llama-3 shapes).  No score ever goes to LDS and nothing synchronises inside the
// loop: every lane group keeps its own running maximum, sum and weighted V sum per head and
// rescales them when the maximum grows; the groups' results are merged at the end, inside a
// wavefront by lane exchange, across wavefronts through LDS (the same merge the splits undergo
// later in att_combine).  model.cpp:186-198 with the softmax of ops.cpp:56-75, regrouped.
template <int kGroup, int kHeads, int kRounds>
__device__ __forceinline__ void att_group_item(Ctx& c, Io& io, const Lds& l, int layer, int h0, int split, int nsplits,
                                               int npos, bool first_item, int hs) {
    static_assert(kHeads <= kItemHeads, "LDS areas are sized for kItemHeads heads");
    const DecodeArgs& a = c.a;
    constexpr int ngroups = kIoThreads / kGroup;
    constexpr int kSub = ngroups * kRounds;
    const int kvh = h0 / a.gqa;
    const int sub = io.it % kGroup, grp = io.it / kGroup;
    const bool lane_live = sub * 8 < hs;
    const int off = lane_live ? sub * 8 : 0;

    const int chunk = (npos + nsplits - 1) / nsplits;
    const int t_begin = split * chunk;
    const int t_end = min(npos, t_begin + chunk);
    const int current = npos - 1;
    const bool has_current = current >= t_begin && current < t_end;
    const size_t head_base = (static_cast<size_t>(layer) * a.n_kv_heads + kvh) * a.seq_len * hs;
    const uint16_t* kbase = a.key_cache + head_base;
    const uint16_t* vbase = a.value_cache + head_base;

    uintx4 krow[kRounds], vrow[kRounds];
    auto request_rows = [&](uintx4 (&rows)[kRounds], const uint16_t* base, int b0) {
#pragma unroll
        for (int j = 0; j < kRounds; ++j) {
            const int t = b0 + grp + j * ngroups;
            rows[j] = uintx4{0u, 0u, 0u, 0u};
            if (t < t_end && t != current && lane_live) rows[j] = load16(base + static_cast<size_t>(t) * hs + off);
        }
    };
    request_rows(krow, kbase, t_begin);
    request_rows(vrow, vbase, t_begin);

    // q of the item's heads (and, in the last split, k and v of the current position): LDS rows
    // 0 .. kHeads-1 hold q, rows kHeads and kHeads+1 hold k and v as the cache will hold them
    const unsigned tag_in = c.seq(layer, kQkv);
    if (!first_item) io_sync(c.ctl, io);  // the previous item's readers have left the LDS areas
    {
        const int wanted = (kHeads + (has_current ? 2 : 0)) * hs;  // at most 6 * 128 <= 2 * kIoThreads
        if (io.it < wanted) {
            auto source = [&](int idx) -> const u64* {
                const int which = div_head_size(c, idx), e = idx - which * hs;
                return which < kHeads ? c.t.q + static_cast<size_t>(h0 + which) * hs + e
                                      : (which == kHeads ? c.t.k : c.t.v) + static_cast<size_t>(kvh) * hs + e;
            };
            const int second = io.it + kIoThreads < wanted ? io.it + kIoThreads : io.it;
            float in[2];
            if (c.t.local_qkv) {
                // (the same slots in this XCD's copy: q, k and v stacked as their matrices are)
                const u64* near = c.t.near_qkv + static_cast<size_t>(c.xcc) * c.t.near_qkv_stride;
                auto near_source = [&](int idx) -> const u64* {
                    const int which = div_head_size(c, idx), e = idx - which * hs;
                    return near + (which < kHeads ? static_cast<size_t>(h0 + which) * hs + e
                                                  : a.dim + (which == kHeads ? 0 : a.kv_dim) + static_cast<size_t>(kvh) * hs + e);
                };
                poll_near_2([&](int j) -> const u64* { return near_source(j == 0 ? io.it : second); }, in, tag_in, c);
            } else {
                poll_n<2>([&](int j) -> const u64* { return source(j == 0 ? io.it : second); }, in, tag_in, c);
            }
            for (int j = 0; j < 2; ++j) {
                const int idx = j == 0 ? io.it : second;
                const int which = div_head_size(c, idx), e = idx - which * hs;
                l.qkv[which * kMaxHeadPad + e] = which < kHeads ? in[j] : f16_bits_to_f32(f32_to_f16_bits(in[j]));
            }
        }
    }
    if (first_item) {
        mark(c, io, 5);
        signal_received(c.ctl);
    }
    io_sync(c.ctl, io);
    if (first_item) {
        mark(c, io, 1);
        mark(c, io, 6);
        mark(c, io, 2);
    }
    uintx4 cur_k = uintx4{0u, 0u, 0u, 0u}, cur_v = uintx4{0u, 0u, 0u, 0u};
    if (has_current && lane_live) {
        union {
            half8_t h;
            uintx4 u;
        } pk, pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            pk.h[e] = static_cast<half_t>(l.qkv[kHeads * kMaxHeadPad + off + e]);
            pv.h[e] = static_cast<half_t>(l.qkv[(kHeads + 1) * kMaxHeadPad + off + e]);
        }
        cur_k = pk.u;
        cur_v = pv.u;
    }

    const float scale = c.t.inv_sqrt_head;  // model.cpp:188
    float top[kHeads], lsum[kHeads], acc[kHeads][8];
#pragma unroll
    for (int h = 0; h < kHeads; ++h) {
        top[h] = -INFINITY;
        lsum[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = 0.0f;
    }
    for (int b0 = t_begin; b0 < t_end; b0 += kSub) {
        float score[kRounds][kHeads];
#pragma unroll
        for (int j = 0; j < kRounds; ++j) {
            const int t = b0 + grp + j * ngroups;
            const half8_t kh = as_half8((t == current) ? cur_k : krow[j]);
#pragma unroll
            for (int h = 0; h < kHeads; ++h) {
                // (q comes from LDS every time: lanes with the same `sub` read the same words, and
                // four heads of q would not fit the register file beside their accumulators)
                const floatx4 qa = *reinterpret_cast<const floatx4*>(l.qkv + h * kMaxHeadPad + off);
                const floatx4 qb = *reinterpret_cast<const floatx4*>(l.qkv + h * kMaxHeadPad + off + 4);
                float s = 0.0f;
#pragma unroll
                for (int e = 0; e < 4; ++e) s = fmaf(static_cast<float>(kh[e]), qa[e], s);
#pragma unroll
                for (int e = 0; e < 4; ++e) s = fmaf(static_cast<float>(kh[4 + e]), qb[e], s);
                s = lane_live ? s : 0.0f;
                s = group_sum<kGroup>(s) * scale;
                score[j][h] = (t < t_end) ? s : -INFINITY;
            }
        }
        if (b0 + kSub < t_end) request_rows(krow, kbase, b0 + kSub);
#pragma unroll
        for (int j = 0; j < kRounds; ++j) {
            const int t = b0 + grp + j * ngroups;
            const half8_t vh = as_half8((t == current) ? cur_v : vrow[j]);
#pragma unroll
            for (int h = 0; h < kHeads; ++h) {
                const float s = score[j][h];
                const float grown = fmaxf(top[h], s);
                const float corr = (top[h] == -INFINITY) ? 0.0f : exp_fast(top[h] - grown);
                const float p = (s == -INFINITY) ? 0.0f : exp_fast(s - grown);
                top[h] = grown;
                lsum[h] = lsum[h] * corr + p;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(static_cast<float>(vh[e]), p, acc[h][e] * corr);
            }
        }
        if (b0 + kSub < t_end) request_rows(vrow, vbase, b0 + kSub);
    }
    // the lane groups of a wavefront, by lane exchange
    const int merge_lane = fresh_lane();
#pragma unroll
    for (int h = 0; h < kHeads; ++h) {
        float all = top[h];
#pragma unroll
        for (int o = kGroup; o < kWave; o <<= 1) all = fmaxf(all, lane_xor(all, o, merge_lane));
        const float f = (top[h] == -INFINITY) ? 0.0f : exp_fast(top[h] - all);
        float ls = lsum[h] * f;
#pragma unroll
        for (int o = kGroup; o < kWave; o <<= 1) ls += lane_xor(ls, o, merge_lane);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float v = acc[h][e] * f;
#pragma unroll
            for (int o = kGroup; o < kWave; o <<= 1) v += lane_xor(v, o, merge_lane);
            acc[h][e] = v;
        }
        top[h] = all;
        lsum[h] = ls;
    }
    if (lane_id() < kGroup) {
#pragma unroll
        for (int h = 0; h < kHeads; ++h) {
            float* r = l.red + (io.iw * kHeads + h) * kRedStride;  // (as many heads per wavefront as the item covers)
            if (lane_live) {
#pragma unroll
                for (int e = 0; e < 8; ++e) r[sub * 8 + e] = acc[h][e];
            }
            if (sub == 0) {
                r[kMaxHeadPad] = top[h];
                r[kMaxHeadPad + 1] = lsum[h];
            }
        }
    }
    if (first_item) mark(c, io, 7);
    io_sync(c.ctl, io);
    if (first_item) mark(c, io, 3);
    // the wavefronts, through LDS: thread (h, e)
    const unsigned tag_out = c.seq(layer, kAtt);
    if (io.it < kHeads * hs) {
        const int h = div_head_size(c, io.it), e = io.it - h * hs;
        float all = -INFINITY;
#pragma unroll
        for (int w = 0; w < kIoWaves; ++w) all = fmaxf(all, l.red[(w * kHeads + h) * kRedStride + kMaxHeadPad]);
        float o = 0.0f, ls = 0.0f;
#pragma unroll
        for (int w = 0; w < kIoWaves; ++w) {
            const float* r = l.red + (w * kHeads + h) * kRedStride;
            const float f = (r[kMaxHeadPad] == -INFINITY) ? 0.0f : exp_fast(r[kMaxHeadPad] - all);
            o += r[e] * f;
            ls += r[kMaxHeadPad + 1] * f;
        }
        if (nsplits == 1) {
            publish(c.t.xb + static_cast<size_t>(h0 + h) * hs + e, o / ls, tag_out);
        } else {
            u64* part = c.t.part + (static_cast<size_t>(h0 + h) * c.t.splits_cap + split) * (hs + 2);
            publish(part + e, o, tag_out);
            if (e == 0) {
                publish(part + hs, all, tag_out);
                publish(part + hs + 1, ls, tag_out);
            }
        }
    }
}

// One query head of size 64 against a context of at most kIoWaves * 64 positions, no splits: the
// whole context is on the compute unit before q arrives, and nothing is fetched after.  Exchange
// wavefront w covers positions 64 w .. 64 w + 63.  Scores: a LANE holds one position's whole K row
// (eight 16-byte pieces) and forms its dot product with q alone, so the softmax needs two
// reductions across the wavefront and no other lane exchange.  Values: a lane holds two dimensions
// of 32 positions (lanes 0..31 the wavefront's first 32 positions, lanes 32..63 the other 32: a
// position's V row is one coalesced 128-byte load of half a wavefront), reads the weights the other
// lanes formed back from LDS and adds up its two dimensions; the two halves meet in one lane
// exchange.  The rows travel straight into LDS (global_load_lds: no register is held while q is
// polled), piece i of every lane side by side, so each lane reads back exactly what it requested,
// conflict-free; the room is the parked rows' area, which the workgroups that hold an item leave
// empty, and the staged-activation area, idle between the QKV and the O projection.  The
// wavefronts' partial results are merged as the lane groups' are in att_group_item.  Up to 512
// positions this costs the same few hundred instructions whatever the position, where the item
// above walks the context in passes of 128 positions, a memory round trip each.
// model.cpp:186-198, ops.cpp:56-75.
constexpr int kLaneItemPositions = kIoWaves * kWave;
constexpr int kLaneBlockFloats = 2048;  // one wavefront's K rows, or its V rows: 64 positions x 64 binary16

// Loads straight into LDS from one global address per lane: load I of a run reads SIZE bytes at address + GSTEP * I
// and lands at lds + LSTEP * I + lane * SIZE.  (The instruction's immediate offset counts for both addresses: the LDS
// base makes up the difference, so that one address register pair serves the whole run.  Spelled out with literal
// offsets: the builtin takes integer constant expressions only, and not value-dependent ones.)
#define LPP_LDS_LOAD(address, lds, SIZE, GSTEP, LSTEP, I) \
    __builtin_amdgcn_global_load_lds(address, (__attribute__((address_space(3))) void*)((lds) + ((LSTEP) - (GSTEP)) * (I)), SIZE, (GSTEP) * (I), 0)
#define LPP_LDS_LOAD4(address, lds, SIZE, GSTEP, LSTEP, I)   \
    LPP_LDS_LOAD(address, lds, SIZE, GSTEP, LSTEP, (I));     \
    LPP_LDS_LOAD(address, lds, SIZE, GSTEP, LSTEP, (I) + 1); \
    LPP_LDS_LOAD(address, lds, SIZE, GSTEP, LSTEP, (I) + 2); \
    LPP_LDS_LOAD(address, lds, SIZE, GSTEP, LSTEP, (I) + 3)

// 8-KiB block b of the room described above.
__device__ __forceinline__ float* lane_item_block(const Ctx& c, const Lds& l, int b) {
    const int in_park = c.b.park_floats / kLaneBlockFloats;
    return b < in_park ? l.park + b * kLaneBlockFloats : l.xs + (b - in_park) * kLaneBlockFloats;
}

// Does this workgroup hold a one-pass item (att_lane_item) in every layer of this token?  (One item per workgroup:
// item h goes to workgroup h.)
__device__ __forceinline__ bool lane_item_here(const Ctx& c) {
    return c.a.head_size == 64 && c.t.att_splits == 1 && c.t.att_group_splits == 0 && c.pos + 1 <= c.t.lane_item_cap &&
           c.wg < c.a.n_heads;
}

// The calling wavefront's K and V rows of head h in `layer` into its two LDS blocks.  Rows of positions the cache
// does not hold yet (the current one, and what lies past the context) are fetched all the same where that saves a
// branch, and never used.  (The host makes sure that every wavefront's 64 positions lie inside the cache's
// seq_len.)  Fetching them a layer ahead, while the gate/up phase streams, was tried for the blocks in the parked
// rows' area, which is free at any time: q then arrives 0.8 us sooner, but the compute unit finishes its gate/up
// rows 3.5 us late, its share of the bandwidth being what it is.
__device__ __forceinline__ void lane_item_fetch(const Ctx& c, const Io& io, const Lds& l, int layer, int h) {
    typedef __attribute__((address_space(1))) const void* GlobalPtr;
    const DecodeArgs& a = c.a;
    constexpr int hs = 64;
    const int npos = c.pos + 1;
    const int t0 = io.iw * kWave;
    if (t0 >= npos) return;
    const int lane = fresh_lane();
    const int half = lane >> 5, pair = lane & 31;
    const int kvh = h / a.gqa;
    const size_t head_base = (static_cast<size_t>(layer) * a.n_kv_heads + kvh) * a.seq_len * hs;
    char* kbytes = reinterpret_cast<char*>(lane_item_block(c, l, 2 * io.iw));
    char* vbytes = reinterpret_cast<char*>(lane_item_block(c, l, 2 * io.iw + 1));
    const GlobalPtr krow = reinterpret_cast<GlobalPtr>(
        reinterpret_cast<unsigned long long>(a.key_cache + head_base + static_cast<size_t>(t0 + lane) * hs));
    LPP_LDS_LOAD4(krow, kbytes, 16, 16, 1024, 0);
    LPP_LDS_LOAD4(krow, kbytes, 16, 16, 1024, 4);
    const GlobalPtr vcol = reinterpret_cast<GlobalPtr>(reinterpret_cast<unsigned long long>(
        reinterpret_cast<const char*>(a.value_cache + head_base + static_cast<size_t>(t0 + 32 * half) * hs) + 4 * pair));
    // V rows four at a time, as far as the first half-wavefront's positions reach into the context
    const int rows = min(32, npos - t0);
    LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 0);
    if (rows > 4) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 4); }
    if (rows > 8) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 8); }
    if (rows > 12) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 12); }
    if (rows > 16) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 16); }
    if (rows > 20) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 20); }
    if (rows > 24) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 24); }
    if (rows > 28) { LPP_LDS_LOAD4(vcol, vbytes, 4, 128, 256, 28); }
}

__device__ __forceinline__ void att_lane_item(Ctx& c, Io& io, const Lds& l, int layer, int h, int npos) {
    const DecodeArgs& a = c.a;
    constexpr int hs = 64;
    constexpr bool first_item = true;  // (one item per workgroup)
    const int lane = fresh_lane();
    const int kvh = h / a.gqa;
    const int current = npos - 1;
    const int t0 = io.iw * kWave, t = t0 + lane;
    const bool wave_live = t0 < npos;  // (uniform)
    const int half = lane >> 5, pair = lane & 31;
    float* kblock = lane_item_block(c, l, 2 * io.iw);
    float* vblock = lane_item_block(c, l, 2 * io.iw + 1);
    lane_item_fetch(c, io, l, layer, h);

    // q of the head, k and v of the current position: LDS row 0 holds q, rows 1 and 2 k and v as the cache will hold them
    const unsigned tag_in = c.seq(layer, kQkv);
    // Up to 64 positions the first wavefront does everything, fetching the three vectors itself: nothing is
    // exchanged between wavefronts, so the two barriers and the merge below fall away.
    const bool solo = npos <= kWave;  // (uniform)
    if (solo) {
        if (io.iw == 0) {
            float in[3];
            if (c.t.local_qkv) {
                const u64* near = c.t.near_qkv + static_cast<size_t>(c.xcc) * c.t.near_qkv_stride;
                const u64* p0 = near + static_cast<size_t>(h) * hs + lane;
                const u64* p1 = near + a.dim + static_cast<size_t>(kvh) * hs + lane;
                const u64* p2 = p1 + a.kv_dim;
                u64 g0, g1, g2;
                unsigned spins = 0;
                while (true) {
                    asm volatile(
                        "global_load_dwordx2 %0, %3, off nt\n\tglobal_load_dwordx2 %1, %4, off nt\n\t"
                        "global_load_dwordx2 %2, %5, off nt\n\ts_waitcnt vmcnt(0)"
                        : "=&v"(g0), "=&v"(g1), "=&v"(g2)
                        : "v"(p0), "v"(p1), "v"(p2)
                        : "memory");
                    if (tag_of(g0) == tag_in && tag_of(g1) == tag_in && tag_of(g2) == tag_in) break;
                    if (poll_give_up(c, spins)) break;
                }
                in[0] = value_of(g0);
                in[1] = value_of(g1);
                in[2] = value_of(g2);
            } else {
                poll_n<3>(
                    [&](int j) -> const u64* {
                        return j == 0 ? c.t.q + static_cast<size_t>(h) * hs + lane
                                      : (j == 1 ? c.t.k : c.t.v) + static_cast<size_t>(kvh) * hs + lane;
                    },
                    in, tag_in, c);
            }
            l.qkv[lane] = in[0];
            l.qkv[kMaxHeadPad + lane] = f16_bits_to_f32(f32_to_f16_bits(in[1]));
            l.qkv[2 * kMaxHeadPad + lane] = f16_bits_to_f32(f32_to_f16_bits(in[2]));
        }
    } else if (io.it < 3 * hs) {
        const int which = io.it >> 6, e = io.it & 63;
        float in[1];
        if (c.t.local_qkv) {
            const u64* src = c.t.near_qkv + static_cast<size_t>(c.xcc) * c.t.near_qkv_stride +
                             (which == 0 ? static_cast<size_t>(h) * hs + e
                                         : a.dim + (which == 1 ? 0 : a.kv_dim) + static_cast<size_t>(kvh) * hs + e);
            u64 got;
            unsigned spins = 0;
            while (true) {
                got = peek_near(src);
                if (tag_of(got) == tag_in) break;
                if (poll_give_up(c, spins)) break;
            }
            in[0] = value_of(got);
        } else {
            const u64* src = which == 0 ? c.t.q + static_cast<size_t>(h) * hs + e
                                        : (which == 1 ? c.t.k : c.t.v) + static_cast<size_t>(kvh) * hs + e;
            poll_n<1>([&](int) -> const u64* { return src; }, in, tag_in, c);
        }
        l.qkv[which * kMaxHeadPad + e] = which == 0 ? in[0] : f16_bits_to_f32(f32_to_f16_bits(in[0]));
    }
    if (first_item) {
        mark(c, io, 5);
        signal_received(c.ctl);
    }
    if (!solo) io_sync(c.ctl, io);
    if (first_item) {
        mark(c, io, 1);
        mark(c, io, 6);
        mark(c, io, 2);
    }

    float* red = l.red + io.iw * kRedStride;  // (one head)
    float top = -INFINITY, lsum = 0.0f, o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
    if (wave_live) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the rows are in
        if ((current >> 6) == io.iw) {
            // The current position's k and v take their places among the fetched rows (what the fetch brought for
            // that position is whatever the cache held before this token): from here on it is a position like any other.
            const int slot = current - t0;
            if (lane < 8) {  // lane i: piece i of the K row
                union {
                    half8_t h;
                    uintx4 u;
                } piece;
#pragma unroll
                for (int e = 0; e < 8; ++e) piece.h[e] = static_cast<half_t>(l.qkv[kMaxHeadPad + 8 * lane + e]);
                *reinterpret_cast<uintx4*>(kblock + 256 * lane + 4 * slot) = piece.u;
            } else if (lane >= 32) {  // lane 32 + d: dimensions 2 d and 2 d + 1 of the V row
                const int d = lane - 32;
                const unsigned lo = f32_to_f16_bits(l.qkv[2 * kMaxHeadPad + 2 * d]), hi = f32_to_f16_bits(l.qkv[2 * kMaxHeadPad + 2 * d + 1]);
                reinterpret_cast<unsigned*>(vblock)[64 * (slot & 31) + 32 * (slot >> 5) + d] = lo | (hi << 16);
            }
        }
        // half a K row at a time: its four pieces and the matching half of q (every lane reads the same words of q)
        // are all requested before the first multiply
        float dot = 0.0f;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            __builtin_amdgcn_sched_barrier(0);
            uintx4 kbits[4];
            floatx4 qa[4], qb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                kbits[i] = *reinterpret_cast<const uintx4*>(kblock + 256 * (4 * r + i) + 4 * lane);
                qa[i] = *reinterpret_cast<const floatx4*>(l.qkv + 8 * (4 * r + i));
                qb[i] = *reinterpret_cast<const floatx4*>(l.qkv + 8 * (4 * r + i) + 4);
            }
            __builtin_amdgcn_sched_barrier(0);  // (left alone, the scheduler pairs every read with its use: one LDS round trip per piece)
            float part[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) part[i] = dot8(kbits[i], qa[i], qb[i], 0.0f);
            dot += (part[0] + part[1]) + (part[2] + part[3]);
        }
        __builtin_amdgcn_sched_barrier(0);
        const float score = t < npos ? dot * 0.125f : -INFINITY;  // 1 / sqrt(64), model.cpp:188
        top = wave_max(score);
        const float p = (score == -INFINITY) ? 0.0f : exp_fast(score - top);
        lsum = wave_sum(p);
        float* weights = l.sc + io.iw * kWave;  // this wavefront's 64 weights (LDS serves one wavefront's accesses in order)
        weights[lane] = p;
        const unsigned* vmine = reinterpret_cast<const unsigned*>(vblock) + lane;
        const int rows = min(32, npos - t0);  // (what was fetched: lane_item_fetch)
        // sixteen positions at a time: their values and weights are all requested before the first is used
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            __builtin_amdgcn_sched_barrier(0);
            if (16 * r < rows) {
                unsigned bits[16];
                floatx4 p4[4];
#pragma unroll
                for (int j = 0; j < 16; ++j) bits[j] = vmine[64 * (16 * r + j)];
#pragma unroll
                for (int g = 0; g < 4; ++g) p4[g] = *reinterpret_cast<const floatx4*>(weights + 32 * half + 16 * r + 4 * g);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const int tv = t0 + 32 * half + 16 * r + j;
                    // (what lies past the context may be anything, NaN included: its weight is zero, the value must be too)
                    const unsigned b = tv < npos ? bits[j] : 0u;
                    float& lo = (j & 1) ? o0 : o2;
                    float& hi = (j & 1) ? o1 : o3;
                    lo = fmaf(p4[j >> 2][j & 3], f16_bits_to_f32(static_cast<uint16_t>(b & 0xffffu)), lo);
                    hi = fmaf(p4[j >> 2][j & 3], f16_bits_to_f32(static_cast<uint16_t>(b >> 16)), hi);
                }
            }
        }
        o0 += o2;
        o1 += o3;
        o0 += lane_xor(o0, 32, lane);
        o1 += lane_xor(o1, 32, lane);
    }
    const unsigned tag_out = c.seq(layer, kAtt);
    if (solo) {
        if (first_item) {
            mark(c, io, 7);
            mark(c, io, 3);
        }
        if (io.iw == 0 && lane < 32) {
            u64* out = c.t.xb + static_cast<size_t>(h) * hs + 2 * pair;
            publish(out, o0 / lsum, tag_out);
            publish(out + 1, o1 / lsum, tag_out);
        }
        return;
    }
    if (lane < 32) {
        red[2 * pair] = o0;
        red[2 * pair + 1] = o1;
    }
    if (lane == 0) {
        red[kMaxHeadPad] = top;
        red[kMaxHeadPad + 1] = lsum;
    }
    if (first_item) mark(c, io, 7);
    io_sync(c.ctl, io);
    if (first_item) mark(c, io, 3);
    if (io.it < hs) {  // the wavefronts' partial results, through LDS: thread e
        const int e = io.it;
        // (all 24 words requested before the first is used: paired with their uses by the scheduler, they cost a
        // round trip to LDS each)
        float wtop[kIoWaves], wsum[kIoWaves], wout[kIoWaves];
#pragma unroll
        for (int w = 0; w < kIoWaves; ++w) {
            const float* r = l.red + w * kRedStride;
            wtop[w] = r[kMaxHeadPad];
            wsum[w] = r[kMaxHeadPad + 1];
            wout[w] = r[e];
        }
        __builtin_amdgcn_sched_barrier(0);
        float all = -INFINITY;
#pragma unroll
        for (int w = 0; w < kIoWaves; ++w) all = fmaxf(all, wtop[w]);
        float o = 0.0f, ls = 0.0f;
#pragma unroll
        for (int w = 0; w < kIoWaves; ++w) {
            const float f = (wtop[w] == -INFINITY) ? 0.0f : exp_fast(wtop[w] - all);
            o += wout[w] * f;
            ls += wsum[w] * f;
        }
        publish(c.t.xb + static_cast<size_t>(h) * hs + e, o / ls, tag_out);
    }
}

// ---------------------------------------------------------------------------
// A KV head's context split over the workgroups of its XCD
// ---------------------------------------------------------------------------
//
// Where every KV head belongs to one XCD (its rows of Wq/Wk/Wv are formed there: qkv_row), long contexts are
// shared out among ALL workgroups of that XCD, 2^xa_cu_shift of them per KV head: workgroup `slot` of a KV head
// takes positions slot * chunk .. slot * chunk + chunk - 1, for all the query heads that read the KV head, so
// every K and V row is fetched once.  The rows do not depend on this token: each exchange wavefront requests its
// xa_ppw = chunk / 8 positions straight into LDS (global_load_lds) while the QKV rows of the layer are still
// being multiplied, so when q arrives the context is on the compute unit and what is left is arithmetic on LDS:
// a lane holds one position's whole K row and forms its scores for the heads alone; the values are summed with a
// lane per two dimensions; wavefronts, and then the workgroups of the KV head, are merged by the max-rescale
// rule of att_group_item.  The partial results and q, k, v travel inside the XCD (publish_near / peek_near); the
// second merge is itself shared out, xa_opc outputs to each workgroup, and publishes the attention output to
// the whole device.  An item's cost depends on chunk, not on the context: 8448 positions of the 1B shape are 264
// per workgroup.  model.cpp:186-198 with the softmax of ops.cpp:56-75, regrouped.

// One 16-byte request per lane straight into LDS: lane i's bytes land at lds_bytes + 16 i.  Inline assembly on
// purpose: requests made through the builtin have the compiler drain every outstanding memory operation before
// any later LDS read of the wavefront.  (The address is a vector operand; M0 is written by a scalar move.)
__device__ __forceinline__ void lds_request16(const void* from, unsigned lds_bytes) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off\n" ::"v"(from), "s"(lds_bytes) : "memory");
}

struct XcdShare {
    int kvh;         // the KV head this workgroup works for
    int slot;        // its index among that KV head's workgroups
    int group0;      // rank (within the XCD) of the KV head's first workgroup
    int t0;          // first position of the calling wavefront
    int count;       // positions of the calling wavefront at this context length (0: none)
    bool holds_current;  // the workgroup's share ends with the current position
};
// (rank, xcc, chunk: the workgroup's rank in its XCD, the XCD and xa_chunk, each passed through an empty asm
// statement by the caller.  Everything here follows from values that do not change from layer to layer; without
// an opaque input the optimiser works it all out once, ahead of the layer loop, and the results then occupy
// scalar registers -- and spill -- for the whole token, in every phase.)
__device__ __forceinline__ XcdShare xcd_share(const Ctx& c, int iw, int rank, int xcc, int chunk) {
    XcdShare x;
    const int shift = c.b.xa_cu_shift;
    const int j = rank >> shift;
    x.slot = rank - (j << shift);
    x.group0 = j << shift;
    x.kvh = xcc * c.b.qkv_by_xcc + j;
    const int npos = c.pos + 1, ppw = chunk >> 3;
    const int begin = x.slot * chunk;
    const int end = min(npos, begin + chunk);
    x.t0 = begin + iw * ppw;
    const int n = min(ppw, end - x.t0);
    x.count = n > 0 ? n : 0;
    x.holds_current = begin < npos && npos <= begin + chunk;
    return x;
}
// (does this workgroup work for a KV head at all?  An XCD with fewer KV heads than 32 >> shift leaves none idle.)

// LDS image of a workgroup's share (chunk positions p = 0 .. chunk-1): K piece-major -- the 16-byte piece i of
// position p at i * chunk * 16 + p * 16, so that a lane which holds a position reads its whole row without bank
// conflicts -- then V as the cache holds it, a position's row after the other.
template <int kHs>
__device__ __forceinline__ unsigned xcd_v_offset(int chunk) {
    return static_cast<unsigned>(chunk) * kHs * 2u;
}

// The calling wavefront's K and V rows of `layer` (its xa_ppw positions of the share, those before the current
// position: the current one's rows come with this token's k and v) on their way into l.kv.
template <int kHs>
__device__ __forceinline__ void xcd_att_prefetch(const Ctx& c, const Io& io, const Lds& l, int layer) {
    const DecodeArgs& a = c.a;
    int rank = c.rank_in_xcc, xcc = c.xcc, chunk = c.t.xa_chunk;
    asm volatile("" : "+s"(rank), "+s"(xcc), "+s"(chunk));
    const XcdShare x = xcd_share(c, io.iw, rank, xcc, chunk);
    const int before = min(x.count, c.pos - x.t0);  // rows earlier tokens left in the cache
    if (before <= 0) return;
    const int ppw = chunk >> 3;
    const int lane = fresh_lane();
    const size_t first = ((static_cast<size_t>(layer) * a.n_kv_heads + x.kvh) * a.seq_len + x.t0) * kHs;
    const unsigned k_lds = __builtin_amdgcn_readfirstlane(l.kv_lds + static_cast<unsigned>(io.iw * ppw * 16));
    const unsigned v_lds = __builtin_amdgcn_readfirstlane(l.kv_lds + xcd_v_offset<kHs>(chunk) + static_cast<unsigned>(io.iw * ppw * kHs * 2));
    if (lane < before) {
        const char* row = reinterpret_cast<const char*>(a.key_cache + first + static_cast<size_t>(lane) * kHs);
#pragma unroll
        for (int i = 0; i < kHs / 8; ++i) lds_request16(row + 16 * i, k_lds + static_cast<unsigned>(i * chunk * 16));
    }
    const char* vsrc = reinterpret_cast<const char*>(a.value_cache + first);
    const int bytes = before * kHs * 2;
    for (int at = 0; at < bytes; at += 1024)  // (uniform)
        if (at + lane * 16 < bytes) lds_request16(vsrc + at + lane * 16, v_lds + static_cast<unsigned>(at));
}

template <int kHs, int kG>
__device__ __forceinline__ void att_xcd_item(Ctx& c, Io& io, const Lds& l, int layer) {
    const DecodeArgs& a = c.a;
    static_assert(kG <= kMaxAttHeads && kG * kHs <= kIoThreads && kIoWaves % kG == 0, "one thread per (head, dimension) in the merge");
    constexpr int kPieces = kHs / 8;
    // Heads of 64: the scores are MFMA products, every wavefront scores the positions whose values it adds up
    // and is a part of its own.  Heads of 128: wavefront (head, part) scores a part's positions for one head.
    constexpr bool kMatrixScores = kHs == 64;
    constexpr int kPartWaves = kMatrixScores ? 1 : kG;  // wavefronts whose positions make up a part
    constexpr int kParts = kIoWaves / kPartWaves;       // the share's positions in kParts runs
    constexpr int kStreams = kHs == 64 ? 2 : 1;  // positions a wavefront adds up side by side (a V row is 32 or 64 lanes wide)
    const int lane = fresh_lane();
    int rank = c.rank_in_xcc, xcc = c.xcc, chunk = c.t.xa_chunk;
    asm volatile("" : "+s"(rank), "+s"(xcc), "+s"(chunk));
    const XcdShare x = xcd_share(c, io.iw, rank, xcc, chunk);
    const int ppw = chunk >> 3;
    const int share_count = min(c.pos + 1 - x.slot * chunk, chunk);  // positions of the whole share (<= 0: none)
    const bool active = x.slot < c.t.xa_active;  // (uniform over the workgroup)
    const unsigned tag_in = c.seq(layer, kQkv), tag_out = c.seq(layer, kAtt);
    u64* part_all = c.t.near_part + static_cast<size_t>(xcc) * (c.nwg / c.t.n_xcc) * c.t.near_part_stride;
    char* kbase = reinterpret_cast<char*>(l.kv);
    char* vbase = kbase + xcd_v_offset<kHs>(chunk);
    float* weights = l.gather;  // [kG][chunk] softmax weights relative to the maximum of the position's part
    float* stats = l.sc;        // [kG][kParts][2] maximum and sum of weights of head h over part

    if (active) {
        // q of the KV head's kG query heads into LDS rows 0 .. kG-1 and, where the share ends with the current
        // position, this token's k and v into that position's rows of the image, rounded as the cache store rounds
        const u64* near = c.t.near_qkv + static_cast<size_t>(xcc) * c.t.near_qkv_stride;
        const int wanted = (kG + (x.holds_current ? 2 : 0)) * kHs;  // at most 6 * 128 <= 2 * kIoThreads
        if (io.it < wanted) {
            auto source = [&](int idx) -> const u64* {
                const int which = idx / kHs, e = idx - which * kHs;
                return near + (which < kG ? static_cast<size_t>(x.kvh * kG + which) * kHs + e
                                          : a.dim + (which == kG ? 0 : a.kv_dim) + static_cast<size_t>(x.kvh) * kHs + e);
            };
            const int second = io.it + kIoThreads < wanted ? io.it + kIoThreads : io.it;
            float in[2];
            poll_near_2([&](int j) -> const u64* { return source(j == 0 ? io.it : second); }, in, tag_in, c);
            const int lc = share_count - 1;  // the current position within the share
            for (int j = 0; j < (second != io.it ? 2 : 1); ++j) {
                const int idx = j == 0 ? io.it : second;
                const int which = idx / kHs, e = idx - which * kHs;
                if (which < kG) {
                    l.qkv[which * kMaxHeadPad + e] = in[j];
                    if constexpr (kMatrixScores) {
                        // q as a binary16 head and a binary16 remainder (rows kMaxAttHeads.. of the area: heads, then
                        // remainders): products with the binary16 K rows are then exact, the sums fp32
                        half_t* q16 = reinterpret_cast<half_t*>(l.qkv + kMaxAttHeads * kMaxHeadPad);
                        const half_t head = static_cast<half_t>(in[j]);
                        q16[which * kHs + e] = head;
                        q16[(kMaxAttHeads + which) * kHs + e] = static_cast<half_t>(in[j] - static_cast<float>(head));
                    }
                } else {
                    const uint16_t bits = f32_to_f16_bits(in[j]);
                    char* at = which == kG ? kbase + (e >> 3) * chunk * 16 + lc * 16 + (e & 7) * 2 : vbase + lc * (kHs * 2) + e * 2;
                    *reinterpret_cast<uint16_t*>(at) = bits;
                }
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's requested rows are in LDS
    mark(c, io, 5);
    signal_received(c.ctl);
    io_sync(c.ctl, io);
    mark(c, io, 1);
    mark(c, io, 6);
    mark(c, io, 2);

    if (active) {
        if constexpr (kMatrixScores) {
            // Scores of the wavefront's own positions for all heads at once: sixteen 4 x 4 products per MFMA, K rows
            // (a LANE per position, as it reads them below) times q columns (lane & 3: the head), four dimensions
            // a step; lane 4 b + j ends up with head j's scores of positions 4 b .. 4 b + 3.  Every K row is read
            // once, whatever the number of heads.
            typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
            union Piece {
                uintx4 u;
                half4_t h[2];
            };
            const int w0 = io.iw * ppw;
            const int hd = lane & 3, p0 = lane & ~3;
            floatx4 acc_head = floatx4{0.0f, 0.0f, 0.0f, 0.0f}, acc_rest = acc_head;
            if (x.count > 0) {  // (uniform)
                const int my = w0 + (lane < x.count ? lane : 0);  // (lanes past the wavefront's positions read its first row; their scores are dropped)
                const char* q_head = reinterpret_cast<const char*>(l.qkv + kMaxAttHeads * kMaxHeadPad) + hd * (kHs * 2);
                const char* q_rest = q_head + kMaxAttHeads * kHs * 2;
#pragma unroll
                for (int i = 0; i < kPieces; ++i) {
                    Piece kp, qh, qr;
                    kp.u = *reinterpret_cast<const uintx4*>(kbase + i * chunk * 16 + my * 16);
                    qh.u = *reinterpret_cast<const uintx4*>(q_head + 16 * i);
                    qr.u = *reinterpret_cast<const uintx4*>(q_rest + 16 * i);
                    acc_head = __builtin_amdgcn_mfma_f32_4x4x4f16(kp.h[0], qh.h[0], acc_head, 0, 0, 0);
                    acc_rest = __builtin_amdgcn_mfma_f32_4x4x4f16(kp.h[0], qr.h[0], acc_rest, 0, 0, 0);
                    acc_head = __builtin_amdgcn_mfma_f32_4x4x4f16(kp.h[1], qh.h[1], acc_head, 0, 0, 0);
                    acc_rest = __builtin_amdgcn_mfma_f32_4x4x4f16(kp.h[1], qr.h[1], acc_rest, 0, 0, 0);
                }
            }
            // (over the lanes of a head: 4 apart inside a row of 16, then across the rows)
            auto over_head = [&](float v, auto op) {
                v = op(v, dpp_move<0x124>(v));  // row_ror:4
                v = op(v, dpp_move<0x128>(v));  // row_ror:8
                v = op(v, lane_xor(v, 16, lane));
                return op(v, lane_xor(v, 32, lane));
            };
            float sc[4];
            float top = -INFINITY;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool live = hd < kG && p0 + r < x.count;
                sc[r] = live ? (acc_head[r] + acc_rest[r]) * c.t.inv_sqrt_head : -INFINITY;  // model.cpp:188
                top = fmaxf(top, sc[r]);
            }
            top = over_head(top, [](float a, float b) { return fmaxf(a, b); });
            // Weights as a binary16 head plus a binary16 remainder, by head, wavefront and position within the
            // wavefront's 64 (zero past its positions): the values below are MFMA products too.
            float sum = 0.0f;
            half4_t w_head, w_rest;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float w = (sc[r] == -INFINITY) ? 0.0f : exp_fast(sc[r] - top);
                sum += w;
                w_head[r] = static_cast<_Float16>(w);
                w_rest[r] = static_cast<_Float16>(w - static_cast<float>(w_head[r]));
            }
            if (hd < kG) {
                half4_t* w16 = reinterpret_cast<half4_t*>(weights) + ((hd * kIoWaves + io.iw) * kWave + p0) / 4;
                w16[0] = w_head;
                w16[kMaxAttHeads * kIoWaves * kWave / 4] = w_rest;
            }
            sum = over_head(sum, [](float a, float b) { return a + b; });
            if (lane < kG) {  // (lane = head)
                stats[(lane * kParts + io.iw) * 2] = top;
                stats[(lane * kParts + io.iw) * 2 + 1] = sum;
            }
            compiler_fence();  // (the weights are read back by this wavefront alone)
        } else {
            // Scores: wavefront (h, part) takes head h over the part's positions, a LANE per position: the lane reads
            // its position's K row (pieces side by side in LDS) and forms the dot product alone; q is read once per
            // wavefront, four pieces at a time, and kept while the part's passes of 64 positions go by.
            {
                const int h = io.iw % kG, part = io.iw / kG;
                const int first = part * kG * ppw;
                const int n = min(share_count - first, kG * ppw);  // positions of the part (<= 0: none)
                float sc[kG];
#pragma unroll
                for (int j = 0; j < kG; ++j) sc[j] = 0.0f;
                if (n > 0) {  // (uniform)
#pragma unroll
                    for (int r = 0; r < kPieces / 4; ++r) {
                        compiler_fence();
                        __builtin_amdgcn_sched_barrier(0);
                        floatx4 qa[4], qb[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            qa[i] = *reinterpret_cast<const floatx4*>(l.qkv + h * kMaxHeadPad + 8 * (4 * r + i));
                            qb[i] = *reinterpret_cast<const floatx4*>(l.qkv + h * kMaxHeadPad + 8 * (4 * r + i) + 4);
                        }
#pragma unroll
                        for (int j = 0; j < kG; ++j) {
                            if (j * kWave < n) {  // (uniform)
                                const int p = j * kWave + lane;
                                const int my = first + (p < n ? p : 0);  // (lanes past the part read its first row; their scores are dropped)
                                uintx4 kbits[4];
#pragma unroll
                                for (int i = 0; i < 4; ++i) kbits[i] = *reinterpret_cast<const uintx4*>(kbase + (4 * r + i) * chunk * 16 + my * 16);
                                __builtin_amdgcn_sched_barrier(0);  // (left alone, the scheduler pairs every read with its use)
                                float part4[4];
#pragma unroll
                                for (int i = 0; i < 4; ++i) part4[i] = dot8(kbits[i], qa[i], qb[i], 0.0f);
                                sc[j] += (part4[0] + part4[1]) + (part4[2] + part4[3]);
                                // (the sum is wanted HERE: without a use in place the multiply-adds are sunk to where the
                                // score is first needed, behind every other round's reads, and all the rows wait in registers)
                                asm volatile("" : "+v"(sc[j]));
                            }
                        }
                    }
                }
                float top = -INFINITY;
#pragma unroll
                for (int j = 0; j < kG; ++j) {
                    sc[j] = (j * kWave + lane < n) ? sc[j] * c.t.inv_sqrt_head : -INFINITY;  // model.cpp:188
                    top = fmaxf(top, sc[j]);
                }
                top = wave_max(top);
                float sum = 0.0f;
#pragma unroll
                for (int j = 0; j < kG; ++j) {
                    const float w = (sc[j] == -INFINITY) ? 0.0f : exp_fast(sc[j] - top);
                    sum += w;
                    if (j * kWave + lane < kG * ppw) weights[h * chunk + first + j * kWave + lane] = w;
                }
                sum = wave_sum(sum);
                if (lane == 0) {
                    stats[(h * kParts + part) * 2] = top;
                    stats[(h * kParts + part) * 2 + 1] = sum;
                }
            }
            io_sync(c.ctl, io);
        }
        // Values: wavefront w takes its own xa_ppw positions for all heads; lane (stream, pair) adds up dimensions
        // 2 pair, 2 pair + 1 over positions stream, stream + kStreams, ...: four positions' values and weights are
        // requested before the first is used.
        if constexpr (kMatrixScores) {
            // Values: out[head][dimension] = sum over the wavefront's positions of weight x V, four positions a step:
            // weight rows (lane & 3: the head, the same in all sixteen products) times V columns (a LANE per
            // dimension, which reads its 2 bytes of four rows); lane d ends up with dimension d of every head.
            typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
            const int w0 = io.iw * ppw;
            floatx4 acc = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            const half4_t* w16 = reinterpret_cast<const half4_t*>(weights) + (((lane & 3) * kIoWaves + io.iw) * kWave) / 4;
            const char* vcol = vbase + lane * 2;
#pragma unroll 4
            for (int k0 = 0; k0 < x.count; k0 += 4) {  // (uniform)
                half4_t v;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    // (what lies past the wavefront's positions may be anything, NaN included: its weight is zero, and
                    // the value is taken from a row that has one)
                    const int at = w0 + (k0 + k < x.count ? k0 + k : 0);
                    v[k] = *reinterpret_cast<const _Float16*>(vcol + at * (kHs * 2));
                }
                const half4_t wh = w16[k0 / 4], wr = w16[kMaxAttHeads * kIoWaves * kWave / 4 + k0 / 4];
                acc = __builtin_amdgcn_mfma_f32_4x4x4f16(wh, v, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_4x4x4f16(wr, v, acc, 0, 0, 0);
            }
#pragma unroll
            for (int h = 0; h < kG; ++h) l.red[(io.iw * kMaxAttHeads + h) * kRedStride + lane] = acc[h];
        } else {
        float out[kG][2];
#pragma unroll
        for (int h = 0; h < kG; ++h) out[h][0] = out[h][1] = 0.0f;
        if (x.count > 0) {  // (uniform over the wavefront)
            const int stream = kStreams == 2 ? lane >> 5 : 0, pair = kStreams == 2 ? (lane & 31) : lane;
            const int w0 = io.iw * ppw;
            const int iters = (x.count + kStreams - 1) / kStreams;
            for (int i0 = 0; i0 < iters; i0 += 4) {
                __builtin_amdgcn_sched_barrier(0);
                unsigned bits[4];
                float wv[kG][4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int p = (i0 + u) * kStreams + stream;
                    const int at = w0 + (p < x.count ? p : 0);
                    bits[u] = *reinterpret_cast<const unsigned*>(vbase + at * (kHs * 2) + pair * 4);
#pragma unroll
                    for (int h = 0; h < kG; ++h) wv[h][u] = weights[h * chunk + at];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int p = (i0 + u) * kStreams + stream;
                    // (what lies past the share may be anything, NaN included: its weight is zero, the value must be too)
                    const unsigned b = p < x.count ? bits[u] : 0u;
                    const float lo = f16_bits_to_f32(static_cast<uint16_t>(b & 0xffffu)), hi = f16_bits_to_f32(static_cast<uint16_t>(b >> 16));
#pragma unroll
                    for (int h = 0; h < kG; ++h) {
                        const float wgt = p < x.count ? wv[h][u] : 0.0f;
                        out[h][0] = fmaf(wgt, lo, out[h][0]);
                        out[h][1] = fmaf(wgt, hi, out[h][1]);
                    }
                }
            }
            if (kStreams == 2) {
#pragma unroll
                for (int h = 0; h < kG; ++h) {
                    out[h][0] += lane_xor(out[h][0], 32, lane);
                    out[h][1] += lane_xor(out[h][1], 32, lane);
                }
            }
        }
        {
            const int pair = kStreams == 2 ? (lane & 31) : lane;
            if (kStreams == 1 || lane < 32) {
#pragma unroll
                for (int h = 0; h < kG; ++h) {
                    float* r = l.red + (io.iw * kMaxAttHeads + h) * kRedStride;
                    r[2 * pair] = out[h][0];
                    r[2 * pair + 1] = out[h][1];
                }
            }
        }
        }
    }
    mark(c, io, 7);
    io_sync(c.ctl, io);
    mark(c, io, 3);
    if (active && io.it < kG * kHs) {  // thread (h, e): this workgroup's partial result, to the XCD's copy
        const int h = io.it / kHs, e = io.it - h * kHs;
        float ptop[kParts], psum[kParts], wout[kIoWaves];
#pragma unroll
        for (int q = 0; q < kParts; ++q) {
            ptop[q] = stats[(h * kParts + q) * 2];
            psum[q] = stats[(h * kParts + q) * 2 + 1];
        }
#pragma unroll
        for (int w = 0; w < kIoWaves; ++w) wout[w] = l.red[(w * kMaxAttHeads + h) * kRedStride + e];
        __builtin_amdgcn_sched_barrier(0);
        float all = -INFINITY;
#pragma unroll
        for (int q = 0; q < kParts; ++q) all = fmaxf(all, ptop[q]);
        float o = 0.0f, ls = 0.0f;
#pragma unroll
        for (int q = 0; q < kParts; ++q) {
            const float f = (ptop[q] == -INFINITY) ? 0.0f : exp_fast(ptop[q] - all);
            ls += psum[q] * f;
#pragma unroll
            for (int w = q * kPartWaves; w < (q + 1) * kPartWaves; ++w) o += wout[w] * f;  // (a part's wavefronts)
        }
        u64* mine = part_all + static_cast<size_t>(rank) * c.t.near_part_stride + h * (kHs + 2);
        publish_near(mine + e, o, tag_out);
        if (e == 0) {
            publish_near(mine + kHs, all, tag_out);
            publish_near(mine + kHs + 1, ls, tag_out);
        }
    }
    // The second merge, shared out: this workgroup combines outputs slot * opc .. of the KV head's kG * kHs, all of
    // one query head.  Thread (e, s) fetches output e of workgroup s's partial result with that result's maximum
    // and sum, all three requested at once; the 32 workgroups of an output sit in the two 16-lane rows of half a
    // wavefront and are merged by lane exchange: no LDS, no barrier.
    const int opc = c.b.xa_opc;
    const int first_out = x.slot * opc;
    const int hd = first_out / kHs, e0 = first_out - hd * kHs;
    const int it = exchange_thread_index(io.iw);
    const int s = it & 31, e = it >> 5;
    if (e < opc) {  // (whole wavefronts)
        float val = 0.0f, top = -INFINITY, sum = 0.0f;
        if (s < c.t.xa_active) {
            const u64* theirs = part_all + static_cast<size_t>(x.group0 + s) * c.t.near_part_stride + hd * (kHs + 2);
            const u64* p0 = theirs + e0 + e;
            const u64* p1 = theirs + kHs;
            const u64* p2 = theirs + kHs + 1;
            u64 g0, g1, g2;
            unsigned spins = 0;
            while (true) {
                asm volatile(
                    "global_load_dwordx2 %0, %3, off nt\n\tglobal_load_dwordx2 %1, %4, off nt\n\t"
                    "global_load_dwordx2 %2, %5, off nt\n\ts_waitcnt vmcnt(0)"
                    : "=&v"(g0), "=&v"(g1), "=&v"(g2)
                    : "v"(p0), "v"(p1), "v"(p2)
                    : "memory");
                if (tag_of(g0) == tag_out && tag_of(g1) == tag_out && tag_of(g2) == tag_out) break;
                if (poll_give_up(c, spins)) break;
            }
            val = value_of(g0);
            top = value_of(g1);
            sum = value_of(g2);
        }
        const int lane = fresh_lane();
        auto half_max = [&](float v) {
            v = fmaxf(v, dpp_move<kDppXor1>(v));
            v = fmaxf(v, dpp_move<kDppXor2>(v));
            v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
            v = fmaxf(v, dpp_move<kDppMirror>(v));
            return fmaxf(v, lane_xor(v, 16, lane));
        };
        auto half_sum = [&](float v) {
            v += dpp_move<kDppXor1>(v);
            v += dpp_move<kDppXor2>(v);
            v += dpp_move<kDppHalfMirror>(v);
            v += dpp_move<kDppMirror>(v);
            return v + lane_xor(v, 16, lane);
        };
        const float all = half_max(top);
        const float f = (top == -INFINITY) ? 0.0f : exp_fast(top - all);
        const float o = half_sum(val * f), ls = half_sum(sum * f);
        if (s == 0) publish(c.t.xb + static_cast<size_t>(x.kvh * kG + hd) * kHs + e0 + e, o / ls, tag_out);
    }
}

// Combine the context splits of head h: collect every split's (output, max,
// sum), rescale to the common maximum and normalise.  Runs after the workgroup
// has published all of its own partials, so a workgroup waiting here never
// holds back a partial another combiner needs.
__device__ __forceinline__ void att_combine(Ctx& c, Io& io, const Lds& l, int layer, int h, int nsplits, int hs) {
    const int stride = hs + 2;
    const unsigned tag_out = c.seq(layer, kAtt);
    io_sync(c.ctl, io);  // earlier readers of gather have left
    const u64* src = c.t.part + static_cast<size_t>(h) * c.t.splits_cap * stride;
    poll_values(src, nsplits * stride, tag_out, c, io, [&](int i, float v, int, bool) { l.gather[i] = v; });
    io_sync(c.ctl, io);
    if (io.it < hs) {
        float top = -INFINITY;
        for (int s = 0; s < nsplits; ++s) top = fmaxf(top, l.gather[s * stride + hs]);
        float o = 0.0f, lsum = 0.0f;
        for (int s = 0; s < nsplits; ++s) {
            const float ms = l.gather[s * stride + hs];
            const float wgt = (ms == -INFINITY) ? 0.0f : expf(ms - top);
            o += l.gather[s * stride + io.it] * wgt;
            lsum += l.gather[s * stride + hs + 1] * wgt;
        }
        publish(c.t.xb + static_cast<size_t>(h) * hs + io.it, o / lsum, tag_out);
    }
}

// Context splits per query head.  The attention phase lasts as long as its busiest workgroup:
// (work items per workgroup) x (positions per item), plus, once there is more than one split, the
// extra hand-over in which the partial results are combined (about what 300 positions cost).  Among
// the split counts that keep an item within 2 * kItemPositions positions, the cheapest wins and the
// smaller of equals: at 8193 positions and 32 heads on 256 workgroups that is 8 splits of 1025
// positions in one round, where 9 splits of 911 would leave 32 workgroups a second item.
__host__ __device__ inline int item_splits(int npos, int cap, int n_heads, int nwg) {
    constexpr int kCombineCost = 300;
    int best = 1, best_cost = 0x7fffffff;
    int first = (npos + 2 * kItemPositions - 1) / (2 * kItemPositions);
    if (first < 1) first = 1;
    for (int s = first; s <= cap; ++s) {
        const int rounds = (n_heads * s + nwg - 1) / nwg;
        const int cost = rounds * ((npos + s - 1) / s) + (s > 1 ? kCombineCost : 0);
        if (cost < best_cost) {
            best_cost = cost;
            best = s;
        }
    }
    return best;
}

// A workgroup without an attention item still tells its streaming wavefronts when this token's
// q, k and v are out (one value stands for all: they are published within a microsecond of one
// another), so that what those held back goes out while the items are computed, not before.
__device__ __forceinline__ void idle_attention_received(Ctx& c, const Io& io, int layer) {
    (void)io;
    (void)layer;
    signal_received(c.ctl);
}

// Splits for items that cover several heads: as item_splits, with an item's length counted in
// whole passes of `sub_positions` positions (what one trip round its loop handles).
__host__ __device__ inline int group_item_splits(int npos, int cap, int n_chunks, int nwg, int sub_positions) {
    constexpr int kCombineCost = 300;
    int best = 1, best_cost = 0x7fffffff;
    for (int s = 1; s <= cap; ++s) {
        const int rounds = (n_chunks * s + nwg - 1) / nwg;
        const int passes = ((npos + s - 1) / s + sub_positions - 1) / sub_positions;
        const int cost = rounds * passes * sub_positions + (s > 1 ? kCombineCost : 0);
        if (cost < best_cost) {
            best_cost = cost;
            best = s;
        }
    }
    return best;
}

template <bool kXcd>
__device__ __forceinline__ void io_attention(Ctx& c, Io& io, const Lds& l, int layer) {
    const DecodeArgs& a = c.a;
    const int npos = c.pos + 1;
    // (Index arithmetic of this phase divides by the head size through a host-made multiplier and by the
    // split count through an opaque copy: a division by a value that does not change from layer to layer
    // has its reciprocal worked out once per token otherwise, and kept in a vector register that the busy
    // stretches of the layer loop then spill.)
    const int hs = a.head_size;
    bool first = true;
    mark(c, io, 0);
    // Long contexts of grouped-query models: one item covers the heads that share a KV head (four at a
    // time), so that the cache is read once.  Short contexts keep one item per head and no combine pass.
    if constexpr (kXcd) {
      if (c.t.xa_chunk > 0) {
        io.it = exchange_thread_index(io.iw);
        if (hs == 64) {
            if (a.gqa == 4) att_xcd_item<64, 4>(c, io, l, layer);
            else if (a.gqa == 2) att_xcd_item<64, 2>(c, io, l, layer);
            else att_xcd_item<64, 1>(c, io, l, layer);
        } else {
            if (a.gqa == 4) att_xcd_item<128, 4>(c, io, l, layer);
            else if (a.gqa == 2) att_xcd_item<128, 2>(c, io, l, layer);
            else att_xcd_item<128, 1>(c, io, l, layer);
        }
        // (after the item, through registers: the fetch then runs beside the hand-over to the next phase.  Between the
        // item's two merges it delays what every other workgroup of the XCD waits for: 770 against 702 us per token
        // at 8300 positions of the 1B shape.  Requested before the item walks its share and kept in registers until
        // nothing reads the share any more, which may lie where the rows go: 732-744 us there, 3065 against 3020 at
        // the 8B shape and 600 positions.  Requested straight into LDS as soon as the item's inputs are in, where the
        // share leaves the rows' area alone: such a request holds its wavefront until the memory pipeline has taken
        // it, a microsecond or two for a wavefront's rows, and that is on the item's path: 677 us per token against
        // 649 at the 1B shape and 600 positions.)
        park_fetch(c, io, l, layer);
        mark(c, io, 4);
        ++c.phase_index;
        return;
      }
    }
    constexpr int heads_per_item = 2;
    if (c.t.att_group_splits > 0) {
        const int n_chunks = a.n_heads / heads_per_item;
        int nsplits = c.t.att_group_splits;
        asm volatile("" : "+s"(nsplits));
        const int items = n_chunks * nsplits;
        for (int item = c.wg; item < items; item += c.nwg) {
            const int chunk = item / nsplits, split = item - chunk * nsplits;
            const int h0 = chunk * heads_per_item;
            io.it = exchange_thread_index(io.iw);
            if (hs <= 64) att_group_item<8, 2, 2>(c, io, l, layer, h0, split, nsplits, npos, first, hs);
            else att_group_item<16, 2, 2>(c, io, l, layer, h0, split, nsplits, npos, first, hs);
            first = false;
        }
        if (first) idle_attention_received(c, io, layer);
        park_fetch(c, io, l, layer);
        if (nsplits > 1) {
            // the heads of a chunk are combined by the workgroups that held its first splits
            for (int item = c.wg; item < items; item += c.nwg) {
                const int chunk = item / nsplits, split = item - chunk * nsplits;
                for (int j = split; j < heads_per_item; j += nsplits) {
                    io.it = exchange_thread_index(io.iw);
                    att_combine(c, io, l, layer, chunk * heads_per_item + j, nsplits, hs);
                }
            }
        }
        mark(c, io, 4);
        ++c.phase_index;
        return;
    }
    int nsplits = c.t.att_splits;
    asm volatile("" : "+s"(nsplits));
    // One item per head and no splits, q, k and v handed over inside the XCD: the heads of the KV heads whose rows
    // XCD x formed go to its first workgroups, in order.
    const int heads_per_xcc = a.n_heads / (c.t.n_xcc > 1 ? c.t.n_xcc : 1);
    const int items = c.t.local_qkv ? (c.rank_in_xcc < heads_per_xcc ? c.wg + 1 : 0) : a.n_heads * nsplits;
    for (int item = c.wg; item < items; item += c.nwg) {
        const int h = c.t.local_qkv ? c.xcc * heads_per_xcc + c.rank_in_xcc : item / nsplits;
        const int split = c.t.local_qkv ? 0 : item - h * nsplits;
        io.it = exchange_thread_index(io.iw);
        // lane groups of 8 cover head sizes up to 64 (lanes past the head idle), groups of 16 up to 128
        if (lane_item_here(c)) att_lane_item(c, io, l, layer, h, npos);
        else if (hs <= 64) att_group_item<8, 1, kShortRounds>(c, io, l, layer, h, split, nsplits, npos, first, hs);
        else att_group_item<16, 1, kShortRounds>(c, io, l, layer, h, split, nsplits, npos, first, hs);
        first = false;
    }
    if (first) idle_attention_received(c, io, layer);
    park_fetch(c, io, l, layer);
    if (nsplits > 1) {
        for (int item = c.wg; item < items; item += c.nwg) {
            const int h = item / nsplits, split = item - h * nsplits;
            io.it = exchange_thread_index(io.iw);
            if (split == 0) att_combine(c, io, l, layer, h, nsplits, hs);
        }
    }
    mark(c, io, 4);
    ++c.phase_index;
}

// ---------------------------------------------------------------------------
// Classifier + sampler (exchange wavefronts)
// ---------------------------------------------------------------------------

// Workgroup w owns the contiguous vocabulary rows [w*cls, ...): their logits
// stay in LDS, the sampler's per-row work happens there, and only three numbers
// per workgroup (maximum, its lowest index, sum of exponentials) are exchanged.
// The workgroup whose slice of the CDF contains the draw (or that holds the
// first maximum, for temperature 0) finishes the token (model.cpp:256-303,
// main.cpp:200-208).
__device__ __forceinline__ void io_classify_sample(Ctx& c, Io& io, const Lds& l) {
    const DecodeArgs& a = c.a;
    Control& ctl = c.ctl;
    const int vocab = a.vocab, dim = a.dim, wg = c.wg, nwg = c.nwg;
    const int it = io.it;
    mark(c, io, 0);
    const float scale = stage_norm(c, io, l, c.t.x, nullptr, dim, c.seq(a.n_layers - 1, kDown), a.rms_final);
    mark(c, io, 2);
    wait_gemv(ctl, 4 * a.n_layers);
    mark(c, io, 3);
    const int r0 = min(vocab, wg * c.b.cls);
    const int n = block_rows(vocab, c.b.cls, wg);
    const int r1 = r0 + n;
    float* lg = l.xs + 4 * nwg;  // beside the sampler tables; the streaming wavefronts are done with xs
    for (int i = it; i < n; i += kIoThreads) {
        lg[i] = row_result(l.results, i, c.b.ns_dim) * scale;
        a.logits[r0 + i] = lg[i];  // raw logits stay readable after the token
    }
    mark(c, io, 4);
    ++c.phase_index;

    const float temperature = c.temperature, penalty = c.penalty;
    const int history_len = c.history_len;
    if (penalty > 1.0f && history_len > 0) {  // model.cpp:258-270, once per occurrence
        // the window is scanned once per entry: bring it into LDS first (the attention score area is idle)
        int* window = reinterpret_cast<int*>(l.sc);
        const bool window_fits = history_len <= 2 * kAttScoreFloats;
        if (window_fits)
            for (int i = it; i < history_len; i += kIoThreads) window[i] = a.history[i];
        io_sync(ctl, io);
        const int* hist = window_fits ? window : a.history;
        for (int i = it; i < history_len; i += kIoThreads) {
            const int tok = hist[i];
            if (tok < r0 || tok >= r1) continue;
            const int count = smp::owned_count(hist, history_len, i);
            if (count > 0) lg[tok - r0] = smp::penalise(lg[tok - r0], penalty, count);
        }
        io_sync(ctl, io);
    }
    ArgMax best{-INFINITY, 0x7fffffff};
    for (int i = it; i < n; i += kIoThreads) {
        float v = lg[i];
        if (temperature != 0.0f) v = v / temperature;  // model.cpp:286-288
        lg[i] = v;
        best = argmax_better(best, ArgMax{v, r0 + i});
    }
    best = wave_argmax(best);
    {
        float* sv = ctl.redv[io.parity];
        int* si = ctl.redi[io.parity];
        if (lane_id() == 0) {
            sv[io.iw] = best.v;
            si[io.iw] = best.i;
        }
        io_sync(ctl, io);
        best = ArgMax{lds_ld(sv), lds_ld(si)};
        for (int w = 1; w < kIoWaves; ++w)
            best = argmax_better(best, ArgMax{lds_ld(sv + w), lds_ld(si + w)});
    }
    const ArgMax mine = best;
    float local_sum = 0.0f;
    if (temperature != 0.0f) {
        float part = 0.0f;
        for (int i = it; i < n; i += kIoThreads) {
            const float e = expf(lg[i] - mine.v);  // ops.cpp:65, against the local maximum
            lg[i] = e;
            part += e;
        }
        local_sum = io_sum(ctl, io, part);
    }
    const unsigned tag = c.seq_stats();
    if (it == 0) {
        publish(c.t.stats + wg * 4 + 0, mine.v, tag);
        publish(c.t.stats + wg * 4 + 1, local_sum, tag);
        publish(c.t.stats + wg * 4 + 2, __int_as_float(mine.i), tag);
        publish(c.t.stats + wg * 4 + 3, 0.0f, tag);
    }
    // every workgroup reads all statistics and reaches the same decision
    float* st_max = l.xs;            // [nwg]  (the streaming wavefronts are done with xs)
    float* st_sum = l.xs + nwg;      // [nwg]
    float* st_arg = l.xs + 2 * nwg;  // [nwg] (int bits)
    float* st_cum = l.xs + 3 * nwg;  // [nwg] mass before the workgroup
    poll_values(c.t.stats, nwg * 4, tag, c, io, [&](int i, float v, int, bool) {
        const int w = i >> 2, f = i & 3;
        if (f == 0) st_max[w] = v;
        else if (f == 1) st_sum[w] = v;
        else if (f == 2) st_arg[w] = v;
    });
    io_sync(ctl, io);
    mark(c, io, 2);
    if (temperature == 0.0f) {  // model.cpp:272-283: first maximum wins
        if (io.iw == 0) {  // one wavefront, a few workgroups per lane
            ArgMax g{-INFINITY, 0x7fffffff};
            for (int w = lane_id(); w < nwg; w += kWave) g = argmax_better(g, ArgMax{st_max[w], __float_as_int(st_arg[w])});
            g = wave_argmax(g);
            if (lane_id() == 0) {
                ctl.token = (g.i == 0x7fffffff) ? 0 : g.i;
                ctl.target = (g.i == 0x7fffffff) ? 0 : g.i / c.b.cls;  // the workgroup that owns the winning row
            }
        }
        io_sync(ctl, io);
    } else {
        float top = -INFINITY;
        for (int w = it; w < nwg; w += kIoThreads) top = fmaxf(top, st_max[w]);
        top = io_max(ctl, io, top);
        float mass = 0.0f;
        for (int w = it; w < nwg; w += kIoThreads) {
            const float mw = (st_max[w] == -INFINITY) ? 0.0f : st_sum[w] * expf(st_max[w] - top);
            st_cum[w] = mw;
            mass += mw;
        }
        const float total = io_sum(ctl, io, mass);
        const float r = c.r;
        if (io.iw == 0) {
            // Running mass in workgroup order = index order of the CDF (model.cpp:294-301): every
            // lane takes a run of consecutive workgroups, a scan across the lanes gives each run's start.
            const int per_lane = (nwg + kWave - 1) / kWave;
            const int w0 = lane_id() * per_lane, w1 = min(nwg, w0 + per_lane);
            float run = 0.0f;
            for (int w = w0; w < w1; ++w) run += st_cum[w] / total;
            float cum = wave_inclusive_scan(run) - run;
            int target = 0x7fffffff;
            for (int w = w0; w < w1; ++w) {
                const float before = cum;
                cum += st_cum[w] / total;
                st_cum[w] = before;
                if (target == 0x7fffffff && r < cum) target = w;
            }
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) target = min(target, __shfl_xor(target, o));
            if (lane_id() == 0) {
                ctl.target = target == 0x7fffffff ? -1 : target;
                ctl.token = vocab - 1;  // model.cpp:302 when no bucket is reached
            }
        }
        io_sync(ctl, io);
        if (lds_ld(&ctl.target) == wg) {
            // inside the target workgroup: p_i = e_i * exp(m_w - top) / total, running sum in index order
            const float f = expf(mine.v - top) / total;
            const float before = st_cum[wg];
            const int per_thread = (n + kIoThreads - 1) / kIoThreads;
            const int begin = it * per_thread, end = min(n, begin + per_thread);
            float chunk_sum = 0.0f;
            for (int i = begin; i < end; ++i) chunk_sum += lg[i] * f;
            const float incl = wave_inclusive_scan(chunk_sum);
            if (lane_id() == kWave - 1) ctl.wave_tot[io.iw] = incl;
            io_sync(ctl, io);
            float offset = before;
            for (int w = 0; w < io.iw; ++w) offset += lds_ld(&ctl.wave_tot[w]);
            offset += incl - chunk_sum;
            float run = 0.0f;
            int found = 0x7fffffff;
            for (int i = begin; i < end; ++i) {
                run += lg[i] * f;
                if (found == 0x7fffffff && r < offset + run) found = r0 + i;
            }
#pragma unroll
            for (int o = 32; o >= 1; o >>= 1) found = min(found, __shfl_xor(found, o));
            if (lane_id() == 0) ctl.wave_found[io.iw] = found;
            io_sync(ctl, io);
            if (it == 0) {
                int f0 = lds_ld(&ctl.wave_found[0]);
                for (int w = 1; w < kIoWaves; ++w) f0 = min(f0, lds_ld(&ctl.wave_found[w]));
                ctl.token = (f0 == 0x7fffffff) ? r1 - 1 : f0;  // rounding left the bucket short: its last row
            }
        }
    }
    // Exactly one workgroup finishes the token: the target, or (no bucket reached) the last one.
    if (it == 0) {
        const int target = lds_ld(&ctl.target);
        const bool finisher = (target == wg) || (target < 0 && wg == nwg - 1);
        // A launch in which some wait was given up delivers nothing: the step record stays as it was, so the
        // host can launch the same token again.
        if (finisher && __hip_atomic_load(c.t.abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u)
            finish_token(a, lds_ld(&ctl.token), 0u);
    }
    mark(c, io, 4);
    ++c.phase_index;
}

template <bool kF16, bool kXcd>
__device__ __forceinline__ void io_role(Ctx& c, Io& io, const Lds& l) {
    const DecodeArgs& a = c.a;
    // The thread index is made opaque before every phase: per-thread addresses are then formed
    // where they are used instead of once for the whole token, where they would occupy (and
    // overflow) the register file for the length of the layer loop.
    auto fresh = [&]() { io.it = exchange_thread_index(io.iw); };
    for (int layer = 0; layer < a.n_layers; ++layer) {
        fresh();
        io_qkv<kXcd>(c, io, l, layer);
        fresh();
        io_attention<kXcd>(c, io, l, layer);
        fresh();
        io_proj(c, io, l, 4 * layer + kGO, c.b.o, a.dim, c.b.ns_dim, c.t.xb, nullptr, 0, 0, c.seq(layer, kAtt),
                c.seq(layer, kOproj));
        fresh();
        io_gateup(c, io, l, layer);
        fresh();
        io_proj(c, io, l, 4 * layer + kGDown, c.b.down, a.hidden, c.b.ns_hidden, c.t.hb, c.t.near_hb, c.t.near_hidden_stride,
                c.t.share_hidden, c.seq(layer, kGateUp), c.seq(layer, kDown));
    }
    fresh();
    io_classify_sample(c, io, l);
    if (io.it == 0 && lds_peek(&c.ctl.error) != 0u) report_error(a.step, 2);
}

// ---------------------------------------------------------------------------
// The kernel
// ---------------------------------------------------------------------------

// (kXcd: with the item that splits a context over an XCD, att_xcd_item.  A second instance of the kernel rather than
// a branch in the one: merely compiled in, that item's registers cost every other plan 5 us per token at the 1B shape.)
template <bool kF16, bool kXcd>
__global__ __launch_bounds__(kThreads) void k_decode_dataflow(DecodeArgs a, Tagged t, Blocks b,
                                                              const uint4* __restrict__ row_lists, int row_list_stride) {
    extern __shared__ __align__(16) float lds[];
    __shared__ Control ctl;
    __shared__ int numbered;
    const int nwg = gridDim.x;
    // Workgroups are numbered by where they run: XCD + n_xcc * (the order in which the XCD's workgroups got here).
    // Which rows, attention items and slices a workgroup owns then says which XCD's L2 they pass through, whatever
    // the order in which the hardware handed the workgroups out.  An XCD that does not get its share of the
    // workgroups (they are handed out in turn: it always has) ends the launch with an error.
    if (threadIdx.x == 0) {
        int number = blockIdx.x;
        if (t.n_xcc > 1) {
            const int x = hardware_xcc() % t.n_xcc;
            const unsigned order = __hip_atomic_fetch_add(t.tickets + x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - t.ticket_base;
            if (order < static_cast<unsigned>(nwg / t.n_xcc)) {
                number = static_cast<int>(order) * t.n_xcc + x;
            } else {
                __hip_atomic_store(t.abort, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_max(&a.step->error, 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        numbered = number;
    }
    const int dim_pad = (a.dim + 7) & ~7;
    Lds l;
    l.xraw = lds;
    l.xs = l.xraw + dim_pad;
    // (a share of a context whose rows run on beyond xs has the parked rows' area next, then what it needs beyond
    // that: plan_for)
    bool share_runs_on = false;
    if constexpr (kXcd) share_runs_on = t.xa_chunk * a.head_size > b.xs_floats - dim_pad;
    l.results = l.xs + b.xs_floats + (share_runs_on ? b.park_floats + b.kv_floats : 0);
    l.sc = l.results + b.results_floats;
    l.qkv = l.sc + 2 * kAttScoreFloats;
    l.red = l.qkv + b.qkv_floats;
    l.gather = l.red + b.red_floats;
    l.park = share_runs_on ? l.xs + b.xs_floats : l.gather + b.gather_floats;
    l.kv = lds + b.kv_offset;
    // (the LDS address is taken from the array itself, where the address space is plain to the compiler, and the
    // area's offset added as a number: a pointer that has been through a structure is not reliably traced back)
    l.kv_lds = static_cast<unsigned>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds)) +
               static_cast<unsigned>((l.kv - lds) * sizeof(float));
    for (unsigned i = threadIdx.x; i < sizeof(Control) / sizeof(unsigned); i += blockDim.x)
        reinterpret_cast<unsigned*>(&ctl)[i] = 0u;
    __syncthreads();  // the only workgroup-wide barrier: the two kinds of wavefronts part ways here
    const int wg = __builtin_amdgcn_readfirstlane(numbered);
    const int wave = wave_index();
    if (wave < kGemvWaves) {
        gemv_role<kF16>(a, ctl, row_lists + static_cast<size_t>(wg * kGemvWaves + wave) * row_list_stride, wave, l.xs,
                        l.results, (wg == 0 || t.trace_stride > 0) && wave == 0 && a.trace != nullptr);
    } else {
        // (kept inside the vocabulary whatever a launch that gave up left in the record: it indexes the embedding)
        const int token_in = min(max(__builtin_amdgcn_readfirstlane(a.step->token), 0), a.vocab - 1);
        unsigned long long* my_trace = nullptr;
        if (a.trace != nullptr && (wg == 0 || t.trace_stride > 0)) my_trace = a.trace + static_cast<size_t>(wg) * t.trace_stride;
        const int n_xcc = t.n_xcc > 1 ? t.n_xcc : 1;
        Ctx c{a, t, b, ctl, t.base, my_trace, 0u,
              token_in, t.pos, t.history_len, t.temperature, t.penalty, t.r, wg, nwg, wg % n_xcc, wg / n_xcc,
              gu_unit0(t.gu_first, wg), gu_units(t.gu_first, wg)};
        Io io{static_cast<int>(threadIdx.x) - kGemvWaves * kWave, wave - kGemvWaves, 0u, 0, a.step};
        if (c.trace && io.it == 0) c.trace[kTraceMarks * phases_per_token(a.n_layers)] = wall_clock64();
        io_role<kF16, kXcd>(c, io, l);
    }
}

// Which XCD each workgroup of a launch of this shape lands on.
__global__ void k_probe_xcc(int* out) {
    if (threadIdx.x == 0) out[blockIdx.x] = hardware_xcc();
}

}  // namespace df

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------

namespace {

int splits_cap_for(const lpp_model* m) {
    // enough for long-context items of a few hundred positions each
    const int s = (m->cfg.seq_len + 127) / 128;
    return s < 1 ? 1 : (s > 64 ? 64 : s);
}

struct Plan {
    int grid;
    df::Blocks blocks;
    size_t lds_bytes;
    std::vector<int> gu_first;  // [grid + 1] first hidden unit of every workgroup (df::gu_unit0)
};

// The hidden units dealt out: workgroup w's share is its block of the plan (gu_a or gu units) times its weight
// (lpp_model::df_gu_weight, 1 until a traced token has said otherwise), scaled so that the shares add up to
// hidden_dim, with boundaries rounded on the running sum.  most = the largest share.
std::vector<int> gateup_table(const lpp_model* m, const df::Blocks& b, int grid, int* most) {
    std::vector<double> share(grid);
    double total = 0.0;
    for (int w = 0; w < grid; ++w) {
        const double weight = static_cast<size_t>(w) < m->df_gu_weight.size() ? m->df_gu_weight[w] : 1.0;
        share[w] = (w < b.gu_split ? b.gu_a : b.gu) * weight;
        total += share[w];
    }
    std::vector<int> first(grid + 1, 0);
    double run = 0.0;
    *most = 0;
    for (int w = 0; w < grid; ++w) {
        run += share[w] * m->cfg.hidden_dim / total;
        int end = w + 1 == grid ? m->cfg.hidden_dim : static_cast<int>(run + 0.5);
        if (end < first[w]) end = first[w];
        if (end > m->cfg.hidden_dim) end = m->cfg.hidden_dim;
        first[w + 1] = end;
        if (end - first[w] > *most) *most = end - first[w];
    }
    return first;
}

constexpr int kMaxXcc = 8;
constexpr int kMaxPerXcc = 32;  // workgroups of one XCD the XCD-wide attention split is laid out for

// The split of a KV head's context over the workgroups of its XCD (att_xcd_item) at npos positions, for a plan whose
// Wq/Wk/Wv rows are dealt out per XCD; chunk 0 where it does not apply.
struct XcdAttention {
    int chunk, active, ppw, cu_shift, opc, kv_floats;
};
XcdAttention xcd_attention_for(const lpp_model* m, const df::Blocks& b, int grid, int npos) {
    XcdAttention x = {};
    if (test_option(LPP_OPT_DECODE_XCD_ATTENTION) == 0 || b.qkv_by_xcc <= 0 || m->df_xcc <= 1) return x;
    const int hs = m->head_size, g = m->gqa;
    if ((hs != 64 && hs != 128) || (g != 1 && g != 2 && g != 4)) return x;
    const int per_xcc = grid / m->df_xcc;
    if (per_xcc > kMaxPerXcc || per_xcc % b.qkv_by_xcc != 0) return x;
    const int n_cu = per_xcc / b.qkv_by_xcc;  // workgroups that share a KV head
    if ((n_cu & (n_cu - 1)) != 0 || (g * hs) % n_cu != 0) return x;
    const int opc = g * hs / n_cu;            // outputs each of them combines: all of one head, at most 16
    if (opc > hs || hs % opc != 0 || opc > df::kMaxHeadPad / 8) return x;
    const int chunk = ((npos + n_cu - 1) / n_cu + 7) & ~7;
    if (chunk > df::kIoWaves * df::kWave) return x;
    while ((1 << x.cu_shift) < n_cu) ++x.cu_shift;
    x.chunk = chunk;
    x.active = (npos + chunk - 1) / chunk;
    x.ppw = chunk / df::kIoWaves;
    x.opc = opc;
    x.kv_floats = chunk * hs;  // eight wavefronts x ppw positions x (K row + V row) of binary16
    return x;
}

// parking: keep the last gate/up rows of most workgroups in LDS (short contexts); false: every row streams.
// xa (chunk > 0): the plan of att_xcd_item -- every workgroup holds a share of a KV head's context, with room for
// four heads in the merge areas, and every workgroup parks gate/up rows in what LDS is left.  The share's rows take
// LDS that nothing else uses while the item runs: the part of xs that only the down phase uses (beyond the first
// dim floats: between two down phases nothing else is staged there), then the parked rows' area, which follows xs
// (the rows of a layer are multiplied before the next layer's share is requested, and fetched after the item has
// read the share for the last time), then an area of their own for what is still missing.  The rows parked do
// not depend on the position, so a growing context keeps its step lists until the share no longer fits at all.
Plan plan_for(const lpp_model* m, bool parking, const XcdAttention* xa = nullptr) {
    const lpp_config& c = m->cfg;
    Plan p;
    p.grid = compute_units();
    auto per = [&](int total) { return (total + p.grid - 1) / p.grid; };
    df::Blocks& b = p.blocks;
    b.qkv = (per(c.dim + 2 * m->kv_dim) + 1) & ~1;  // RoPE pairs stay inside one workgroup
    b.qkv_by_xcc = 0;
    {
        // Per XCD where the KV heads divide among the XCDs (qkv_row): whole KV heads with their query heads.
        const bool allowed = test_option(LPP_OPT_DECODE_XCD_QKV) != 0;
        const int n = m->df_xcc;
        if (allowed && n > 1 && c.n_kv_heads % n == 0 && p.grid % n == 0 && c.n_heads / n <= p.grid / n) {
            const int rows = (c.dim + 2 * m->kv_dim) / n, wgs = p.grid / n;
            b.qkv_by_xcc = c.n_kv_heads / n;
            b.qkv = ((rows + wgs - 1) / wgs + 1) & ~1;
        }
    }
    b.o = per(c.dim);
    b.gu = per(c.hidden_dim);
    b.down = per(c.dim);
    b.cls = per(c.vocab_size);
    const int dim_pad = (c.dim + 7) & ~7;
    int xs = (c.hidden_dim + 7) & ~7;
    if (dim_pad > xs) xs = dim_pad;
    if (4 * p.grid + b.cls > xs) xs = (4 * p.grid + b.cls + 7) & ~7;  // sampler tables and the workgroup's logits
    b.xs_floats = xs;
    const int chunk_cols = c.weight_precision == LPP_WEIGHT_FP16 ? 512 : 256;
    b.ns_dim = df::slices_used(c.dim, chunk_cols);
    b.ns_hidden = df::slices_used(c.hidden_dim, chunk_cols);
    b.dim_as_float = static_cast<float>(c.dim);
    int slots = b.qkv * b.ns_dim;  // one partial sum per row and column slice
    if (b.o * b.ns_dim > slots) slots = b.o * b.ns_dim;
    if (2 * b.gu * b.ns_dim > slots) slots = 2 * b.gu * b.ns_dim;
    if (b.down * b.ns_hidden > slots) slots = b.down * b.ns_hidden;
    if (b.cls * b.ns_dim > slots) slots = b.cls * b.ns_dim;
    b.results_floats = (slots + 7) & ~7;
    b.gather_floats = (splits_cap_for(m) * (m->head_size + 2) + 7) & ~7;
    b.red_floats = df::kIoWaves * df::kItemHeads * df::kRedStride;
    b.qkv_floats = (df::kMaxAttHeads + 2) * df::kMaxHeadPad;
    b.xa_cu_shift = 0;
    b.xa_opc = 0;
    b.kv_floats = 0;
    b.kv_offset = 0;
    const bool xcd = xa != nullptr && xa->chunk > 0;
    if (xcd) {
        b.red_floats = df::kIoWaves * df::kMaxAttHeads * df::kRedStride;
        b.gather_floats = df::kMaxAttHeads * df::kIoWaves * df::kWave;  // (the weights of a share; nothing is gathered)
        b.xa_cu_shift = xa->cu_shift;
        b.xa_opc = xa->opc;
        b.kv_offset = 2 * dim_pad;  // xraw, then the first dim floats of xs
    }
    b.slice_dim = df::slice_width(c.dim, chunk_cols);
    b.gu_a = b.gu;
    b.gu_split = 0;
    b.park_rows = 0;
    b.park_floats = 0;
    auto lds_floats = [&]() {
        return static_cast<size_t>(dim_pad + b.xs_floats + b.results_floats + 2 * df::kAttScoreFloats +
                                   b.qkv_floats + b.red_floats + b.gather_floats + b.park_floats +
                                   b.kv_floats);
    };
    // Parked gate/up rows: whatever LDS is left (binary16 models; the workgroups that hold the attention
    // items of a short context, one per query head, park nothing and own that many fewer hidden units).
    if (parking && c.weight_precision == LPP_WEIGHT_FP16 && c.n_heads < p.grid) {
        constexpr size_t kLdsBytes = 160 * 1024, kReserve = 2048;  // the rest is for the kernel's static LDS
        // (the plan with parked rows only ever runs items of one head: a wavefront's partial result of one head each)
        if (!xcd) {
            b.red_floats = df::kIoWaves * df::kRedStride;
            b.qkv_floats = 3 * df::kMaxHeadPad;
        }
        const size_t used = lds_floats() * sizeof(float);
        const size_t row_bytes = static_cast<size_t>(c.dim) * 2;
        int rows = used + kReserve < kLdsBytes ? static_cast<int>((kLdsBytes - kReserve - used) / row_bytes) : 0;
        rows &= ~1;                                 // whole hidden units
        const int cap = 4 * df::kIoWaves;  // a handful of rows per exchange wavefront is plenty
        if (rows > cap) rows = cap;
        // units of an ordinary workgroup if the first n_heads own rows / 2 fewer (att_xcd_item: all workgroups alike)
        const int gu = xcd ? b.gu : (c.hidden_dim + c.n_heads * (rows / 2) + p.grid - 1) / p.grid;
        if (rows >= 2 && gu - rows / 2 >= 1 && 2 * gu - rows >= df::kGemvWaves) {
            b.gu = gu;
            b.gu_a = xcd ? gu : gu - rows / 2;
            b.gu_split = xcd ? 0 : c.n_heads;
            b.park_rows = rows;
            b.park_floats = static_cast<int>((static_cast<size_t>(rows) * row_bytes + 31) / 32 * 8);
            if (2 * b.gu * b.ns_dim > slots) {
                slots = 2 * b.gu * b.ns_dim;
                b.results_floats = (slots + 7) & ~7;
            }
        }
    }
    {
        int most = 0;
        p.gu_first = gateup_table(m, b, p.grid, &most);
        if (2 * most * b.ns_dim > slots) {
            slots = 2 * most * b.ns_dim;
            b.results_floats = (slots + 7) & ~7;
        }
    }
    // Order of the areas: xraw, xs, partial sums, scores, q/k/v, merge, gather, parked rows -- unless a share's rows run
    // on beyond xs: then the parked rows follow xs, whatever the share needs beyond them comes next, and the rest after.
    // (the kernel tells the two orders apart by the same comparison: chunk positions x head_size floats)
    if (xcd && xa->kv_floats > b.xs_floats - dim_pad) {
        const int in_place = b.xs_floats - dim_pad + b.park_floats;
        b.kv_floats = xa->kv_floats > in_place ? xa->kv_floats - in_place : 0;
    }
    p.lds_bytes = lds_floats() * sizeof(float);
    return p;
}

constexpr int kGridCap = 1024;  // workgroups the statistics table has room for
// Tagged values of one XCD's copy of an n-value vector: whole 128-byte lines.
size_t near_stride(int n) { return (static_cast<size_t>(n) + 15) / 16 * 16; }

size_t tagged_count(const lpp_model* m, int grid_cap) {
    const lpp_config& c = m->cfg;
    return static_cast<size_t>(c.dim) * 3 + static_cast<size_t>(m->kv_dim) * 2 + c.hidden_dim +
           static_cast<size_t>(c.n_heads) * splits_cap_for(m) * (m->head_size + 2) + 4u * grid_cap +
           32u + static_cast<size_t>(kMaxXcc) * (near_stride(c.hidden_dim) + near_stride(c.dim + 2 * m->kv_dim)) +
           static_cast<size_t>(kMaxXcc) * kMaxPerXcc * near_stride(m->gqa * (m->head_size + 2));
}

// Positions a one-head attention item of a head of size 64 can keep on the compute unit (att_lane_item): two 8-KiB
// blocks per 64 positions in the parked rows' area and the staged-activation area of plan p, whole blocks of 64
// positions inside the cache; 0 where that item does not apply.
int lane_item_positions(const lpp_model* m, const Plan& p) {
    const bool off = test_option(LPP_OPT_DECODE_LANE_ITEM) == 0;
    if (off || m->head_size != 64 || m->cfg.n_heads > p.grid) return 0;
    const int blocks = p.blocks.park_floats / df::kLaneBlockFloats + p.blocks.xs_floats / df::kLaneBlockFloats;
    int cap = blocks / 2 * df::kWave;
    if (cap > df::kLaneItemPositions) cap = df::kLaneItemPositions;
    const int in_cache = m->cfg.seq_len / df::kWave * df::kWave;
    return cap < in_cache ? cap : in_cache;
}

df::Tagged tagged_of(const lpp_model* m, bool generating, int lane_item_cap) {
    const lpp_config& c = m->cfg;
    df::Tagged t;
    df::u64* p = static_cast<df::u64*>(m->tagged);
    t.x = p;            p += c.dim;
    t.q = p;            p += c.dim;
    t.k = p;            p += m->kv_dim;
    t.v = p;            p += m->kv_dim;
    t.xb = p;           p += c.dim;
    t.hb = p;           p += c.hidden_dim;
    t.part = p;         p += static_cast<size_t>(c.n_heads) * splits_cap_for(m) * (m->head_size + 2);
    t.stats = p;        p += 4u * kGridCap;
    p = reinterpret_cast<df::u64*>((reinterpret_cast<uintptr_t>(p) + 127) & ~static_cast<uintptr_t>(127));
    t.near_hidden_stride = static_cast<int>(near_stride(c.hidden_dim));
    t.near_hb = p;      p += static_cast<size_t>(kMaxXcc) * t.near_hidden_stride;
    t.near_qkv_stride = static_cast<int>(near_stride(c.dim + 2 * m->kv_dim));
    t.near_qkv = p;     p += static_cast<size_t>(kMaxXcc) * t.near_qkv_stride;
    t.near_part_stride = static_cast<int>(near_stride(m->gqa * (m->head_size + 2)));
    t.near_part = p;
    t.xa_chunk = t.xa_active = t.xa_ppw = 0;
    t.tickets = m->sync_words + 96;
    t.ticket_base = m->df_ticket_base;
    {
        const int nwg = m->persist_grid > 0 ? m->persist_grid : compute_units();
        t.n_xcc = (m->df_xcc > 1 && m->df_xcc <= kMaxXcc && nwg % m->df_xcc == 0) ? m->df_xcc : 1;
        const int per_xcc = nwg / t.n_xcc;
        t.share_hidden = (c.hidden_dim + per_xcc - 1) / per_xcc;
    }
    t.splits_cap = splits_cap_for(m);
    t.hs_magic = static_cast<unsigned>((1ull << 32) / static_cast<unsigned long long>(m->head_size)) + 1u;
    t.pos = m->df_pos;
    {
        const int npos = m->df_pos + 1, nwg = m->persist_grid > 0 ? m->persist_grid : compute_units();
        t.att_splits = df::item_splits(npos, t.splits_cap, c.n_heads, nwg);
        // (a head of size 64 takes up to 512 positions in one item whose cost does not grow with the context)
        t.inv_sqrt_head = 1.0f / sqrtf(static_cast<float>(m->head_size));
        t.lane_item_cap = lane_item_cap;
        if (npos <= t.lane_item_cap) t.att_splits = 1;
        t.local_qkv = 0;  // (set by the launch once the plan is chosen)
        t.att_group_splits = 0;
        if (m->gqa % 2 == 0 && t.att_splits > 1) {
            const int sub_positions = (m->head_size <= 64 ? df::kIoThreads / 8 : df::kIoThreads / 16) * 2;
            t.att_group_splits = df::group_item_splits(npos, t.splits_cap, c.n_heads / 2, nwg, sub_positions);
        }
    }
    t.history_len = m->df_history_len;
    t.temperature = m->df_temperature;
    t.penalty = m->df_penalty;
    // model.cpp:291: one draw per step; a generate call brings them as an array (absent: zeros)
    t.r = generating ? (m->df_uniforms_host ? m->df_uniforms_host[m->df_step_index] : 0.0f) : m->df_r;
    t.base = m->df_base;
    t.abort = m->sync_words + 65;
    t.spin_limit = m->spin_limit;
    t.trace_stride = m->df_trace_stride;
    return t;
}

// Step lists of the streaming wavefronts: [workgroup][wavefront][stride]
// entries.  After a wavefront's last step the list continues with entries
// without kStepValid that point at a readable row: the wavefront requests up to
// a ring of steps past its last one and reads whole batches of entries.
lpp_status build_step_lists(lpp_model* m, const Plan& p, int which) {
    const lpp_config& c = m->cfg;
    const df::Blocks& b = p.blocks;
    const int L = c.n_layers, dim = c.dim, hidden = c.hidden_dim, kv = m->kv_dim;
    const size_t wb = c.weight_precision == LPP_WEIGHT_FP16 ? 2 : 4;
    const int chunk_cols = static_cast<int>(1024 / wb);
    const size_t rb_dim = static_cast<size_t>(dim) * wb, rb_hidden = static_cast<size_t>(hidden) * wb;
    const int n_xcc = m->df_xcc > 1 ? m->df_xcc : 1;
    auto base = [&](int t) { return reinterpret_cast<unsigned long long>(m->w[t]); };
    auto block_rows = [](int total, int block, int wg) {
        const int n = total - wg * block;
        return n < 0 ? 0 : (n > block ? block : n);
    };
    // steps of a wavefront in a phase of nrows rows and d columns: it works on one slice and, of the
    // wavefronts sharing that slice, takes one row of every (kGemvWaves / nslices)
    auto own = [&](int nrows, int d, int j) {
        const int share = df::kGemvWaves / df::slice_count(d, chunk_cols);
        (void)j;
        return (nrows + share - 1) / share;  // an upper bound for every wavefront
    };
    // gate/up rows of a workgroup that go through the streaming wavefronts: all but the parked ones at the block's end
    auto gu_streamed = [&](int wg) {
        const int units = df::gu_units(p.gu_first.data(), wg);
        return 2 * units - df::gu_parked_rows(b, wg, units);
    };
    int longest = 0;
    for (int wg = 0; wg < p.grid; ++wg)
        for (int j = 0; j < df::kGemvWaves; ++j) {
            const int n = L * (own(df::qkv_rows(b, dim, kv, m->head_size, m->gqa, wg, wg / n_xcc), dim, j) + own(block_rows(dim, b.o, wg), dim, j) +
                               own(gu_streamed(wg), dim, j) +
                               own(block_rows(dim, b.down, wg), hidden, j)) +
                          own(block_rows(c.vocab_size, b.cls, wg), dim, j);
            if (n > longest) longest = n;
        }
    // whole batches, plus the three batches a wavefront may request past its last step
    const int stride = ((longest + df::kDepth + df::kStepBatch - 1) / df::kStepBatch + 3) * df::kStepBatch;
    LPP_REQUIRE(4 * L + 1 <= static_cast<int>(df::kStepPhaseMask), "persistent decode: too many layers for the step lists");
    LPP_REQUIRE(b.results_floats <= static_cast<int>(df::kStepSlotMask) + 1 && dim < 65536 && hidden < 65536,
                "persistent decode: shape too large for the step lists");
    std::vector<df::StepEntry> host(static_cast<size_t>(p.grid) * df::kGemvWaves * stride);
    // columns of every matrix row the lists (and the parked rows) account for, keyed by the row's first byte
    std::unordered_map<unsigned long long, int> covered;
    for (int wg = 0; wg < p.grid; ++wg)
        for (int j = 0; j < df::kGemvWaves; ++j) {
            df::StepEntry* out = host.data() + (static_cast<size_t>(wg) * df::kGemvWaves + j) * stride;
            int n = 0;
            auto phase_rows = [&](int phase, int nrows, int d, auto row_address) {
                const int nslices = df::slice_count(d, chunk_cols), width = df::slice_width(d, chunk_cols);
                const int slice = j % nslices, rank = j / nslices, share = df::kGemvWaves / nslices;
                const int begin = slice * width;
                const int exist = d - begin < 0 ? 0 : (d - begin > width ? width : d - begin);
                if (exist == 0) return;
                // Of every `share` consecutive rows this wavefront takes one, and not always the same
                // one: with a fixed residue its rows would sit at a fixed stride in memory.  (Which of a
                // workgroup's wavefronts streams which rows does not change how long a bandwidth-bound
                // phase takes: the wavefront launched first on each SIMD runs ahead of its neighbour,
                // but handing it more rows only widens its lead; the phase ends when the bytes are in.)
                const int first = n;
                for (int i = 0; i * share < nrows; ++i) {
                    const int r = i * share + (rank + i) % share;
                    if (r >= nrows) continue;
                    out[n].ptr = row_address(r) + static_cast<size_t>(begin) * wb;
                    out[n].meta = static_cast<unsigned>(r * df::slices_used(d, chunk_cols) + slice) |
                                  (static_cast<unsigned>(phase) << df::kStepPhaseShift) | df::kStepValid;
                    out[n].cols = static_cast<unsigned>(begin) | (static_cast<unsigned>(exist) << 16);
                    covered[row_address(r)] += exist;
                    ++n;
                }
                if (n > first) out[n - 1].meta |= df::kStepLastRow;
            };
            for (int l = 0; l < L; ++l) {
                phase_rows(4 * l + df::kGQkv, df::qkv_rows(b, dim, kv, m->head_size, m->gqa, wg, wg / n_xcc), dim, [&](int r) {
                    const int g = df::qkv_row(b, dim, kv, m->head_size, m->gqa, wg, wg % n_xcc, wg / n_xcc, r);
                    if (g < dim) return base(LPP_T_WQ) + (static_cast<size_t>(l) * dim + g) * rb_dim;
                    if (g < dim + kv) return base(LPP_T_WK) + (static_cast<size_t>(l) * kv + (g - dim)) * rb_dim;
                    return base(LPP_T_WV) + (static_cast<size_t>(l) * kv + (g - dim - kv)) * rb_dim;
                });
                phase_rows(4 * l + df::kGO, block_rows(dim, b.o, wg), dim,
                           [&](int r) { return base(LPP_T_WO) + (static_cast<size_t>(l) * dim + wg * b.o + r) * rb_dim; });
                // local row 2u = gate row of hidden unit u, 2u + 1 = its up row
                phase_rows(4 * l + df::kGGateUp, gu_streamed(wg), dim, [&](int r) {
                    return base((r & 1) ? LPP_T_W3 : LPP_T_W1) +
                           (static_cast<size_t>(l) * hidden + df::gu_unit0(p.gu_first.data(), wg) + (r >> 1)) * rb_dim;
                });
                phase_rows(4 * l + df::kGDown, block_rows(dim, b.down, wg), hidden, [&](int r) {
                    return base(LPP_T_W2) + (static_cast<size_t>(l) * dim + wg * b.down + r) * rb_hidden;
                });
            }
            phase_rows(4 * L, block_rows(c.vocab_size, b.cls, wg), dim,
                       [&](int r) { return base(LPP_T_WCLS) + (static_cast<size_t>(wg) * b.cls + r) * rb_dim; });
            for (; n < stride; ++n) {
                out[n].ptr = base(LPP_T_WCLS);
                out[n].meta = 0;
                out[n].cols = 0;
            }
        }
    // Every column of every row must be multiplied exactly once per token: by a step, or as a parked row.
    for (int wg = 0; wg < p.grid; ++wg) {
        const int units = df::gu_units(p.gu_first.data(), wg), parked = df::gu_parked_rows(b, wg, units);
        for (int l = 0; l < L; ++l)
            for (int r = 2 * units - parked; r < 2 * units; ++r)
                covered[base((r & 1) ? LPP_T_W3 : LPP_T_W1) + (static_cast<size_t>(l) * hidden + df::gu_unit0(p.gu_first.data(), wg) + (r >> 1)) * rb_dim] += dim;
    }
    {
        const struct { int tensor; size_t rows; int cols; } all[] = {
            {LPP_T_WQ, static_cast<size_t>(L) * dim, dim},       {LPP_T_WK, static_cast<size_t>(L) * kv, dim},
            {LPP_T_WV, static_cast<size_t>(L) * kv, dim},        {LPP_T_WO, static_cast<size_t>(L) * dim, dim},
            {LPP_T_W1, static_cast<size_t>(L) * hidden, dim},    {LPP_T_W3, static_cast<size_t>(L) * hidden, dim},
            {LPP_T_W2, static_cast<size_t>(L) * dim, hidden},    {LPP_T_WCLS, static_cast<size_t>(c.vocab_size), dim}};
        size_t expected = 0;
        for (const auto& t : all) {
            expected += t.rows;
            for (size_t r = 0; r < t.rows; ++r) {
                const auto it = covered.find(base(t.tensor) + r * static_cast<size_t>(t.cols) * wb);
                if (it == covered.end() || it->second != t.cols)
                    return fail(LPP_ERR_STATE, "persistent decode: step lists cover %d of %d columns of row %zu of tensor %d",
                                it == covered.end() ? 0 : it->second, t.cols, r, t.tensor);
            }
        }
        // (a tied classifier shares no rows with the other matrices: it is its own binary16 copy)
        if (covered.size() != expected) return fail(LPP_ERR_STATE, "persistent decode: step lists name %zu rows, the model has %zu",
                                                    covered.size(), expected);
    }
    lpp_free(m->df_rows[which]);
    m->df_rows[which] = nullptr;
    lpp_free(m->df_gu_first[which]);
    m->df_gu_first[which] = nullptr;
    void* d = nullptr;
    LPP_TRY(lpp_malloc(&d, p.gu_first.size() * sizeof(int)));
    m->df_gu_first[which] = static_cast<int*>(d);
    LPP_TRY(lpp_memcpy_h2d(d, p.gu_first.data(), p.gu_first.size() * sizeof(int)));
    d = nullptr;
    LPP_TRY(lpp_malloc(&d, host.size() * sizeof(df::StepEntry)));
    m->df_rows[which] = d;
    m->df_row_stride[which] = stride;
    LPP_TRY(lpp_memcpy_h2d(d, host.data(), host.size() * sizeof(df::StepEntry)));
    return LPP_OK;
}

}  // namespace

size_t dataflow_tagged_bytes(const lpp_model* m) { return tagged_count(m, kGridCap) * sizeof(df::u64); }

// A streaming wavefront covers one column slice of at most kStepLoads 1-KiB chunks per row, and a
// row has at most one slice per streaming wavefront: rows beyond 8 x 4 KiB (8192 fp32 or 16384
// binary16 columns) do not fit.  nullptr when the shape fits, else the reason.
const char* dataflow_unsupported_reason(const lpp_model* m) {
    const lpp_config& c = m->cfg;
    const int chunk_cols = c.weight_precision == LPP_WEIGHT_FP16 ? 512 : 256;
    const int widest = c.hidden_dim > c.dim ? c.hidden_dim : c.dim;
    if (df::slice_width(widest, chunk_cols) > df::kStepLoads * chunk_cols)
        return "persistent decode: weight rows wider than 32 KiB (8192 fp32 or 16384 binary16 columns)";
    if (m->head_size > df::kMaxHeadPad) return "persistent decode: head_size exceeds 128";
    return nullptr;
}

lpp_status dataflow_take_options(lpp_model* m, hipStream_t s);

template <bool kF16>
static lpp_status launch_impl(lpp_model* m, const ph::DecodeArgs& a, hipStream_t s) {
    if (const char* why = dataflow_unsupported_reason(m)) return fail(LPP_ERR_UNSUPPORTED, "%s", why);
    LPP_TRY(dataflow_take_options(m, s));
    if (m->df_xcc == 0) {
        // Workgroups are handed to the XCDs in turn.  The per-XCD hand-overs rely on every XCD getting an equal share
        // of them, so it is measured, not assumed: anything but workgroup w on XCD (first + w) % n switches them off.
        m->df_xcc = 1;
        if (test_option(LPP_OPT_DECODE_XCD_HANDOVERS) != 0) {
            const int grid = compute_units();
            void* d = nullptr;
            LPP_TRY(lpp_malloc(&d, static_cast<size_t>(grid) * sizeof(int)));
            hipLaunchKernelGGL(df::k_probe_xcc, dim3(grid), dim3(df::kThreads), 0, s, static_cast<int*>(d));
            std::vector<int> where(grid);
            const hipError_t e = hipMemcpyAsync(where.data(), d, where.size() * sizeof(int), hipMemcpyDeviceToHost, s);
            const hipError_t e2 = hipStreamSynchronize(s);
            lpp_free(d);
            LPP_HIP(e);
            LPP_HIP(e2);
            int n = 0;
            for (int x : where) n = x + 1 > n ? x + 1 : n;
            bool in_turn = n > 1 && n <= kMaxXcc && grid % n == 0;
            for (int w = 0; w < grid && in_turn; ++w) in_turn = where[w] == (where[0] + w) % n;
            if (in_turn) m->df_xcc = n;
        }
    }
    // Two plans: with parked gate/up rows while only the first n_heads workgroups hold an attention item
    // (one split per head), without them at longer contexts.  Each has its own step lists.
    const bool parking_allowed = test_option(LPP_OPT_DECODE_PARKING) != 0;
    const Plan parked_plan = plan_for(m, parking_allowed);
    const int lane_cap = lane_item_positions(m, parked_plan);
    df::Tagged tagged = tagged_of(m, a.uniforms != nullptr, lane_cap);
    // Contexts beyond what the plan with parked gate/up rows covers (one work item per head: the one-pass item's
    // reach for heads of size 64, the cost model's choice otherwise): a KV head's context is split over the
    // workgroups of its XCD, if the shape allows and the rows fit LDS.  That plan parks gate/up rows as well, fewer
    // of them (its merge areas hold four heads), and has step lists of its own (without parking it shares those of
    // the plan without).
    constexpr size_t kLdsLimit = 160 * 1024 - 2048;
    Plan xcd_plan = plan_for(m, false);
    XcdAttention xa = {};
    {
        const int npos = m->df_pos + 1;
        const bool wanted = m->head_size == 64 ? npos > lane_cap : (tagged.att_splits > 1 || tagged.att_group_splits > 0);
        if (wanted) xa = xcd_attention_for(m, xcd_plan.blocks, xcd_plan.grid, npos);
        if (xa.chunk > 0) {
            xcd_plan = plan_for(m, parking_allowed, &xa);
            if (xcd_plan.lds_bytes > kLdsLimit) xa.chunk = 0;
        }
    }
    if (xa.chunk > 0) {
        tagged.xa_chunk = xa.chunk;
        tagged.xa_active = xa.active;
        tagged.xa_ppw = xa.ppw;
        tagged.att_splits = 1;
        tagged.att_group_splits = 0;
    }
    const bool use_parked = xa.chunk == 0 && parked_plan.blocks.park_rows > 0 && tagged.att_splits == 1 && tagged.att_group_splits == 0;
    const Plan p = xa.chunk > 0 ? xcd_plan : (use_parked ? parked_plan : plan_for(m, false));
    // (step lists: [0] every row streamed, [1] the parked plan's, [2] those of att_xcd_item's plan with parked rows)
    const int which = xa.chunk > 0 ? (xcd_plan.blocks.park_rows > 0 ? 2 : 0) : (use_parked ? 1 : 0);
    // q, k and v stay inside the XCD that formed them while every head's item sits on that XCD: one item per head
    tagged.local_qkv = (p.blocks.qkv_by_xcc > 0 && tagged.att_splits == 1 && tagged.att_group_splits == 0) ? 1 : 0;
    // Sequence numbers are compared for equality, so they must not come round to values that slots
    // written long ago (split partials of a longer context, say) may still hold: well before the
    // 32-bit count wraps, drain the stream, clear every tagged slot and start again from zero.
    if (m->df_base > df::kTagWrapGuard) {
        LPP_HIP(hipStreamSynchronize(s));
        LPP_TRY(lpp_memset(m->tagged, 0, dataflow_tagged_bytes(m)));
        LPP_HIP(hipStreamSynchronize(s));
        m->df_base = 0;
        tagged.base = 0;
    }
    if (m->persist_grid == 0) {
        LPP_REQUIRE(p.grid <= kGridCap, "persistent decode: %d compute units exceed the statistics table", p.grid);
        LPP_REQUIRE(m->head_size <= df::kMaxHeadPad, "persistent decode: head_size %d exceeds %d", m->head_size,
                    df::kMaxHeadPad);
        const size_t lds_most = kLdsLimit;  // (every launch brings its own size, up to what a compute unit has)
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&df::k_decode_dataflow<kF16, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_most)) != hipSuccess ||
            hipFuncSetAttribute(reinterpret_cast<const void*>(&df::k_decode_dataflow<kF16, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_most)) != hipSuccess)
            return fail(LPP_ERR_UNSUPPORTED, "persistent decode needs %zu bytes of LDS per workgroup", lds_most);
        int per_cu = 0, per_cu_xcd = 0;
        LPP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, df::k_decode_dataflow<kF16, false>, df::kThreads, lds_most));
        LPP_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu_xcd, df::k_decode_dataflow<kF16, true>, df::kThreads, lds_most));
        if (per_cu < 1 || per_cu_xcd < 1)
            return fail(LPP_ERR_UNSUPPORTED, "persistent decode kernel does not fit a compute unit (LDS %zu bytes)", lds_most);
        m->persist_grid = p.grid;
    }
    bool moved = false;  // a weight tensor changed its address: both lists are stale
    for (int t = 0; t < LPP_T_COUNT && !moved; ++t) moved = m->df_rows_key[t] != m->w[t];
    if (moved) {
        LPP_HIP(hipStreamSynchronize(s));  // a launch still running may be reading the old lists
        for (int i = 0; i < 3; ++i) {
            lpp_free(m->df_rows[i]);
            m->df_rows[i] = nullptr;
        }
        for (int t = 0; t < LPP_T_COUNT; ++t) m->df_rows_key[t] = m->w[t];
    }
    // (both lists at once: a generation loop that grows past the short contexts must not stop to build the other one)
    if (m->df_rows[which] == nullptr) LPP_TRY(build_step_lists(m, p, which));
    if (which < 2 && parked_plan.blocks.park_rows > 0 && m->df_rows[1 - which] == nullptr)
        LPP_TRY(build_step_lists(m, use_parked ? plan_for(m, false) : parked_plan, 1 - which));
    if (which != 2 && m->df_rows[2] == nullptr && parking_allowed) {
        // (the third as well, where a context of a thousand positions would take att_xcd_item's plan with parked rows)
        const Plan plain = plan_for(m, false);
        const XcdAttention probe = xcd_attention_for(m, plain.blocks, plain.grid, m->cfg.seq_len < 1024 ? m->cfg.seq_len : 1024);
        if (probe.chunk > 0) {
            const Plan later = plan_for(m, true, &probe);
            if (later.blocks.park_rows > 0 && later.lds_bytes <= kLdsLimit) LPP_TRY(build_step_lists(m, later, 2));
        }
    }
    // (test hook: a ticket base one launch behind makes every workgroup's ticket look like one too many for its XCD)
    if (tagged.n_xcc > 1 && take_forced_ticket_failure()) tagged.ticket_base -= static_cast<unsigned>(m->persist_grid / tagged.n_xcc);
    LPP_REQUIRE(p.lds_bytes <= kLdsLimit, "persistent decode: %zu bytes of LDS per workgroup", p.lds_bytes);
    tagged.gu_first = m->df_gu_first[which];
    if (xa.chunk > 0)
        hipLaunchKernelGGL((df::k_decode_dataflow<kF16, true>), dim3(m->persist_grid), dim3(df::kThreads), p.lds_bytes, s, a,
                           tagged, p.blocks, static_cast<const uint4*>(m->df_rows[which]), m->df_row_stride[which]);
    else
        hipLaunchKernelGGL((df::k_decode_dataflow<kF16, false>), dim3(m->persist_grid), dim3(df::kThreads), p.lds_bytes, s, a,
                           tagged, p.blocks, static_cast<const uint4*>(m->df_rows[which]), m->df_row_stride[which]);
    LPP_CHECK_LAUNCH("k_decode_dataflow");
    m->df_base += df::phases_per_token(m->cfg.n_layers);
    if (tagged.n_xcc > 1) m->df_ticket_base += static_cast<unsigned>(m->persist_grid / tagged.n_xcc);  // one ticket per workgroup
    if (!m->df_freeze) {  // what finish_token does to the device's record
        if (m->df_history_cap > 0 && m->df_history_len < m->df_history_cap) m->df_history_len += 1;
        m->df_pos += 1;
        m->df_step_index += 1;
    }
    return LPP_OK;
}

lpp_status dataflow_launch(lpp_model* m, const ph::DecodeArgs& a, hipStream_t s) {
    return m->cfg.weight_precision == LPP_WEIGHT_FP16 ? launch_impl<true>(m, a, s) : launch_impl<false>(m, a, s);
}

// Forget the step lists, the launch sizing and the per-XCD ticket counts; df_xcc = 0 has the next launch probe the
// device again, 1 leaves the per-XCD hand-overs off for this model.
lpp_status dataflow_forget_plans(lpp_model* m, hipStream_t s, int df_xcc) {
    LPP_HIP(hipStreamSynchronize(s));  // a launch still running may be reading the lists and drawing tickets
    for (int i = 0; i < 3; ++i) {
        lpp_free(m->df_rows[i]);
        m->df_rows[i] = nullptr;
    }
    if (df_xcc != m->df_xcc) {  // the weights are per XCD: a new numbering starts from even shares
        m->df_gu_weight.clear();
        m->df_calibrated = false;
    }
    m->df_xcc = df_xcc;
    m->persist_grid = 0;
    m->df_ticket_base = 0;
    if (m->sync_words != nullptr) LPP_TRY(lpp_memset(m->sync_words + 96, 0, kMaxXcc * sizeof(unsigned)));
    return LPP_OK;
}

// A test hook changed what the plans may use: forget what was derived under the old settings (calibration included).
lpp_status dataflow_take_options(lpp_model* m, hipStream_t s) {
    if (m->df_options_epoch == test_options_epoch()) return LPP_OK;
    LPP_TRY(dataflow_forget_plans(m, s, 0));
    m->df_options_epoch = test_options_epoch();
    return LPP_OK;
}

// The step lists alone (the partition of the hidden units changed): rebuilt at the next launch.
lpp_status dataflow_forget_lists(lpp_model* m, hipStream_t s) {
    LPP_HIP(hipStreamSynchronize(s));
    for (int i = 0; i < 3; ++i) {
        lpp_free(m->df_rows[i]);
        m->df_rows[i] = nullptr;
    }
    return LPP_OK;
}
// Workgroups that hold the attention items of a short context (they own fewer hidden units and park no rows); the
// XCDs the workgroups are numbered by (1: not numbered by XCD).
void dataflow_partition_classes(const lpp_model* m, int* item_workgroups, int* n_xcc) {
    const Plan p = plan_for(m, test_option(LPP_OPT_DECODE_PARKING) != 0);
    *item_workgroups = p.blocks.gu_split;
    *n_xcc = m->df_xcc > 1 ? m->df_xcc : 1;
}

// After a launch that left a code in StepParams::error (the stream is idle, the step record is as the launch found it:
// a launch that gave up delivers no token).  Whatever the code, the ticket counters and the abort flag start afresh.
// Code 3 (an XCD was dealt more than its share of the workgroups): the per-XCD hand-overs are switched off for this
// model and *relaunch is set -- sequence numbers never repeat, so the same token can simply be launched again.
// Code 1 (a wait for inputs ran out) under the per-XCD scheme switches it off as well: the hand-overs inside an XCD
// rest on how its L2 serves plain stores and non-temporal loads, and the device-scope path does not.
lpp_status dataflow_after_error(lpp_model* m, int code, bool* relaunch) {
    *relaunch = false;
    if (code == 0) return LPP_OK;
    hipStream_t s = stream();
    const bool had_xcd_scheme = m->df_xcc > 1;
    LPP_TRY(dataflow_forget_plans(m, s, (code == 3 || had_xcd_scheme) ? 1 : m->df_xcc));
    LPP_TRY(lpp_memset(m->sync_words + 64, 0, 2 * sizeof(unsigned)));
    int zero = 0;
    LPP_HIP(hipMemcpyAsync(&m->step->error, &zero, sizeof zero, hipMemcpyHostToDevice, s));
    LPP_HIP(hipStreamSynchronize(s));
    if (code == 3) {
        *relaunch = true;
        return LPP_OK;
    }
    return fail(LPP_ERR_HIP, code == 2 ? "decode kernel: a wait inside a workgroup ran out"
                                       : "decode kernel gave up waiting for its inputs");
}

unsigned dataflow_phases_per_token(int n_layers) { return df::phases_per_token(n_layers); }
unsigned dataflow_trace_marks() { return df::kTraceMarks; }

}  // namespace lpp
