// lpp_device.hpp -- device-side building blocks for the gfx950 kernels:
// wave64 reductions over DPP, 16-byte weight loads, binary16 helpers and the
// row-tile dot product every GEMV-shaped kernel in the library is built from.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace lpp {
namespace dev {

constexpr int kWave = 64;

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uintx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int lane_id() { return static_cast<int>(threadIdx.x) & (kWave - 1); }
// Wavefront number inside the workgroup, as a scalar the compiler knows to be
// uniform (keeps row pointers and loop bounds in SGPRs).
__device__ __forceinline__ int wave_index() {
    return __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave);
}

// One DPP move: every lane reads the lane the control word selects inside its
// row of 16 (quad permutes and mirrors touch only in-range lanes).
template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, true));
}
template <int kCtrl>
__device__ __forceinline__ int dpp_move_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, kCtrl, 0xf, 0xf, true);
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16

// Sum over the 16 lanes of each DPP row; every lane of the row gets the sum.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<kDppXor1>(v);
    v += dpp_move<kDppXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);
    v += dpp_move<kDppMirror>(v);
    return v;
}

// Sum over the whole wavefront, returned wave-uniform.  Fixed association:
// ((row0 + row1) + (row2 + row3)) over butterfly row sums.
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (a + b) + (c + d);
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<kDppXor1>(v));
    v = fmaxf(v, dpp_move<kDppXor2>(v));
    v = fmaxf(v, dpp_move<kDppHalfMirror>(v));
    v = fmaxf(v, dpp_move<kDppMirror>(v));
    float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// (value, index) pair ordered as the CPU argmax orders candidates: larger value
// first, and among equal values the smaller index (model.cpp:275-281 keeps the
// first maximum because it replaces only on strict >).
struct ArgMax {
    float v;
    int i;
};
__device__ __forceinline__ ArgMax argmax_better(ArgMax a, ArgMax b) {
    bool take_b = (b.v > a.v) || (b.v == a.v && b.i < a.i);
    return take_b ? b : a;
}
__device__ __forceinline__ ArgMax wave_argmax(ArgMax m) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        ArgMax o;
        o.v = __shfl_xor(m.v, off);
        o.i = __shfl_xor(m.i, off);
        m = argmax_better(m, o);
    }
    return m;
}

// Inclusive prefix sum across the wavefront (lane order).
__device__ __forceinline__ float wave_inclusive_scan(float v) {
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        float up = __shfl_up(v, off);
        if (lane >= off) v += up;
    }
    return v;
}

__device__ __forceinline__ uintx4 load16(const void* p) {
    return *reinterpret_cast<const uintx4*>(p);
}
// Streaming 16-byte load for data read exactly once (weights): bypass-friendly
// hint so the lines do not displace the activations in the caches.
__device__ __forceinline__ uintx4 load16_stream(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(p));
}

__device__ __forceinline__ half8_t as_half8(uintx4 v) {
    union {
        uintx4 u;
        half8_t h;
    } c;
    c.u = v;
    return c.h;
}
__device__ __forceinline__ floatx4 as_float4(uintx4 v) {
    union {
        uintx4 u;
        floatx4 f;
    } c;
    c.u = v;
    return c.f;
}

// Round-to-nearest-even fp32 -> binary16 bit pattern and back.
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    union {
        half_t h;
        uint16_t u;
    } c;
    c.h = static_cast<half_t>(f);
    return c.u;
}
__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
    union {
        half_t h;
        uint16_t u;
    } c;
    c.u = b;
    return static_cast<float>(c.h);
}

// acc += dot(8 binary16 weights, 8 fp32 activations), fp32 multiply-add.
__device__ __forceinline__ float dot8(uintx4 wbits, floatx4 xa, floatx4 xb, float acc) {
    half8_t w = as_half8(wbits);
    acc = fmaf(static_cast<float>(w[0]), xa[0], acc);
    acc = fmaf(static_cast<float>(w[1]), xa[1], acc);
    acc = fmaf(static_cast<float>(w[2]), xa[2], acc);
    acc = fmaf(static_cast<float>(w[3]), xa[3], acc);
    acc = fmaf(static_cast<float>(w[4]), xb[0], acc);
    acc = fmaf(static_cast<float>(w[5]), xb[1], acc);
    acc = fmaf(static_cast<float>(w[6]), xb[2], acc);
    acc = fmaf(static_cast<float>(w[7]), xb[3], acc);
    return acc;
}
__device__ __forceinline__ float dot4(uintx4 wbits, floatx4 xa, float acc) {
    floatx4 w = as_float4(wbits);
    acc = fmaf(w[0], xa[0], acc);
    acc = fmaf(w[1], xa[1], acc);
    acc = fmaf(w[2], xa[2], acc);
    acc = fmaf(w[3], xa[3], acc);
    return acc;
}

// Weight element traits: how many elements one 16-byte load carries.
template <bool kF16>
struct WTraits;
template <>
struct WTraits<true> {
    static constexpr int kPerLoad = 8;
    static constexpr int kBytes = 2;
};
template <>
struct WTraits<false> {
    static constexpr int kPerLoad = 4;
    static constexpr int kBytes = 4;
};

// Row-tile dot product: one wavefront computes kRows dot products of length d
// against the activation vector xs (LDS or any generic pointer, 16-byte
// aligned, at least ceil(d / kPerLoad) * kPerLoad floats readable).
// Each lane owns kPerLoad consecutive columns of every 64*kPerLoad-column
// chunk, so a wave load covers 1 KiB of one row, fully coalesced.  kUnroll
// chunks of all rows are requested before the first multiply-add, i.e.
// kRows*kUnroll 16-byte loads are in flight per lane.  Rows whose pointer is
// null contribute 0.  d must be a multiple of kPerLoad and rows 16-byte aligned.
// Results are wave-uniform.
template <bool kF16, int kRows, int kUnroll>
__device__ __forceinline__ void wave_rows_dot(const char* const (&rows)[kRows], const float* xs,
                                              int d, float (&result)[kRows]) {
    constexpr int kPer = WTraits<kF16>::kPerLoad;
    constexpr int kChunk = kWave * kPer;  // columns per wave load
    const int lane = lane_id();
    float acc[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = 0.0f;

    const int nchunks = (d + kChunk - 1) / kChunk;
    for (int c0 = 0; c0 < nchunks; c0 += kUnroll) {
        uintx4 wv[kUnroll][kRows];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int col = (c0 + u) * kChunk + lane * kPer;
            const bool live = col < d;
#pragma unroll
            for (int r = 0; r < kRows; ++r) {
                if (live && rows[r] != nullptr) {
                    wv[u][r] = load16_stream(rows[r] + static_cast<size_t>(col) * WTraits<kF16>::kBytes);
                } else {
                    wv[u][r] = uintx4{0u, 0u, 0u, 0u};
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int col = (c0 + u) * kChunk + lane * kPer;
            if (col < d) {
                if constexpr (kF16) {
                    floatx4 xa = *reinterpret_cast<const floatx4*>(xs + col);
                    floatx4 xb = *reinterpret_cast<const floatx4*>(xs + col + 4);
#pragma unroll
                    for (int r = 0; r < kRows; ++r) acc[r] = dot8(wv[u][r], xa, xb, acc[r]);
                } else {
                    floatx4 xa = *reinterpret_cast<const floatx4*>(xs + col);
#pragma unroll
                    for (int r = 0; r < kRows; ++r) acc[r] = dot4(wv[u][r], xa, acc[r]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) result[r] = wave_sum(acc[r]);
}

// Accessors for values that cross workgroups INSIDE one kernel.  The eight XCDs
// of the device have separate L2 caches, and whole-cache acquire/release fences
// cost tens of microseconds here; instead, every such value is written through
// and read around the non-coherent cache levels with device-scope accesses
// (sc1).  kCoherent = false is the ordinary access for kernels whose inputs were
// complete before launch.
template <bool kCoherent>
struct Mem {
    static __device__ __forceinline__ float ld(const float* p) {
        if constexpr (kCoherent) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else return *p;
    }
    static __device__ __forceinline__ int ldi(const int* p) {
        if constexpr (kCoherent) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else return *p;
    }
    static __device__ __forceinline__ void st(float* p, float v) {
        if constexpr (kCoherent) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else *p = v;
    }
    static __device__ __forceinline__ void sti(int* p, int v) {
        if constexpr (kCoherent) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else *p = v;
    }
    // Two adjacent floats (8-byte aligned) in one access.
    static __device__ __forceinline__ float2 ld2(const float* p) {
        if constexpr (kCoherent) {
            union {
                unsigned long long u;
                float2 f;
            } c;
            c.u = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                    __HIP_MEMORY_SCOPE_AGENT);
            return c.f;
        } else {
            return *reinterpret_cast<const float2*>(p);
        }
    }
};

// Block-wide sum for blocks of up to 16 wavefronts; scratch is 16 floats of LDS.
// Every thread gets the total.  Contains two block barriers.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    const int nwaves = (static_cast<int>(blockDim.x) + kWave - 1) / kWave;
    float s = wave_sum(v);
    __syncthreads();
    if (lane_id() == 0) scratch[wave] = s;
    __syncthreads();
    float total = 0.0f;
    for (int i = 0; i < nwaves; ++i) total += scratch[i];
    return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    const int nwaves = (static_cast<int>(blockDim.x) + kWave - 1) / kWave;
    float s = wave_max(v);
    __syncthreads();
    if (lane_id() == 0) scratch[wave] = s;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < nwaves; ++i) total = fmaxf(total, scratch[i]);
    return total;
}

}  // namespace dev
}  // namespace lpp
