// ops_gemv.hip -- lpp_gemv and lpp_convert_f32_to_f16.
//
// Replaces cuda_gemv / gemv_f16_kernel / gemv_kernel / convert_f32_to_f16_kernel
// (reference src/matmul.cu:9-161).  The reference launches one 256-thread block
// per output row and, for binary16 weights, first casts x to binary16 and
// accumulates in half2.  Here a wavefront owns a tile of rows, every lane keeps
// kRows*kUnroll 16-byte weight loads in flight, x stays fp32 (staged once per
// workgroup in LDS) and accumulation is fp32.
#include "lpp_device.hpp"
#include "lpp_internal.hpp"

namespace lpp {
namespace {

using namespace dev;

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;
constexpr int kMaxLdsFloats = 16384;  // 64 KiB of x per workgroup

// x is copied to LDS padded with zeros up to a multiple of 8 floats so the row
// tile may read whole 16-byte groups.
template <bool kF16, int kRows, int kUnroll>
__global__ __launch_bounds__(kGemvThreads) void gemv_rows_kernel(float* __restrict__ out,
                                                                 const float* __restrict__ x,
                                                                 const char* __restrict__ w, int n,
                                                                 int d) {
    extern __shared__ __align__(16) float xs[];
    const int d_pad = (d + 7) & ~7;
    for (int i = threadIdx.x; i < d_pad; i += kGemvThreads) xs[i] = (i < d) ? x[i] : 0.0f;
    __syncthreads();

    const size_t row_bytes = static_cast<size_t>(d) * WTraits<kF16>::kBytes;
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    const int ntiles = (n + kRows - 1) / kRows;
    const int waves_total = static_cast<int>(gridDim.x) * kGemvWaves;
    for (int tile = static_cast<int>(blockIdx.x) * kGemvWaves + wave; tile < ntiles;
         tile += waves_total) {
        const int row0 = tile * kRows;
        const char* rows[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r)
            rows[r] = (row0 + r < n) ? w + static_cast<size_t>(row0 + r) * row_bytes : nullptr;
        float sums[kRows];
        wave_rows_dot<kF16, kRows, kUnroll>(rows, xs, d, sums);
        if (lane_id() < kRows && row0 + lane_id() < n) {
            float v = sums[0];
#pragma unroll
            for (int r = 1; r < kRows; ++r)
                if (lane_id() == r) v = sums[r];
            out[row0 + lane_id()] = v;
        }
    }
}

// Any shape, any alignment: one wavefront per row, scalar loads.  Only taken
// when d is not a multiple of the 16-byte vector width, the weight pointer is
// misaligned or x does not fit in LDS.
template <bool kF16>
__global__ __launch_bounds__(kGemvThreads) void gemv_generic_kernel(float* __restrict__ out,
                                                                    const float* __restrict__ x,
                                                                    const void* __restrict__ w,
                                                                    int n, int d) {
    const int wave = static_cast<int>(threadIdx.x) / kWave;
    const int waves_total = static_cast<int>(gridDim.x) * kGemvWaves;
    for (int row = static_cast<int>(blockIdx.x) * kGemvWaves + wave; row < n; row += waves_total) {
        float acc = 0.0f;
        const size_t base = static_cast<size_t>(row) * d;
        for (int c = lane_id(); c < d; c += kWave) {
            float wv;
            if constexpr (kF16) wv = static_cast<float>(reinterpret_cast<const half_t*>(w)[base + c]);
            else wv = reinterpret_cast<const float*>(w)[base + c];
            acc = fmaf(wv, x[c], acc);
        }
        acc = wave_sum(acc);
        if (lane_id() == 0) out[row] = acc;
    }
}

__global__ __launch_bounds__(256) void convert_f32_to_f16_kernel(uint16_t* __restrict__ dst,
                                                                 const float* __restrict__ src,
                                                                 size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += stride) dst[i] = f32_to_f16_bits(src[i]);
}

template <bool kF16, int kRows, int kUnroll>
lpp_status launch_rows(float* out, const float* x, const void* w, int n, int d) {
    const int ntiles = (n + kRows - 1) / kRows;
    int blocks = (ntiles + kGemvWaves - 1) / kGemvWaves;
    const int cap = compute_units() * 8;  // up to 8 resident workgroups of 4 waves per CU
    if (blocks > cap) blocks = cap;
    const size_t lds = static_cast<size_t>((d + 7) & ~7) * sizeof(float);
    hipLaunchKernelGGL((gemv_rows_kernel<kF16, kRows, kUnroll>), dim3(blocks), dim3(kGemvThreads),
                       lds, stream(), out, x, static_cast<const char*>(w), n, d);
    LPP_CHECK_LAUNCH("gemv_rows_kernel");
    return LPP_OK;
}

template <bool kF16>
lpp_status gemv_dispatch(float* out, const float* x, const void* w, int n, int d) {
    constexpr int kPer = WTraits<kF16>::kPerLoad;
    const bool vector_ok = (d % kPer == 0) && (reinterpret_cast<uintptr_t>(w) % 16 == 0) &&
                           (d <= kMaxLdsFloats);
    if (!vector_ok) {
        int blocks = (n + kGemvWaves - 1) / kGemvWaves;
        const int cap = compute_units() * 8;
        if (blocks > cap) blocks = cap;
        hipLaunchKernelGGL((gemv_generic_kernel<kF16>), dim3(blocks), dim3(kGemvThreads), 0,
                           stream(), out, x, w, n, d);
        LPP_CHECK_LAUNCH("gemv_generic_kernel");
        return LPP_OK;
    }
    // Tile choice: enough wave tiles to cover every SIMD several times over for
    // small matrices, more rows per wave (more loads in flight) for large ones.
    const int chunks = (d + kWave * kPer - 1) / (kWave * kPer);
    const long waves_wanted = static_cast<long>(compute_units()) * 8;
    if (chunks >= 8) {
        // Long rows: one or two rows, four chunks in flight each.
        if (n / 2 >= waves_wanted) return launch_rows<kF16, 2, 4>(out, x, w, n, d);
        return launch_rows<kF16, 1, 4>(out, x, w, n, d);
    }
    if (n / 4 >= waves_wanted) return launch_rows<kF16, 4, 4>(out, x, w, n, d);
    if (n / 2 >= waves_wanted) return launch_rows<kF16, 2, 4>(out, x, w, n, d);
    return launch_rows<kF16, 1, 4>(out, x, w, n, d);
}

}  // namespace
}  // namespace lpp

extern "C" {

lpp_status lpp_convert_f32_to_f16(lpp_half* d_dst, const float* d_src, int n) {
    LPP_REQUIRE(n >= 0, "lpp_convert_f32_to_f16: n = %d", n);
    if (n == 0) return LPP_OK;
    LPP_REQUIRE(d_dst && d_src, "lpp_convert_f32_to_f16: null pointer");
    int blocks = (n + 255) / 256;
    const int cap = lpp::compute_units() * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(lpp::convert_f32_to_f16_kernel, dim3(blocks), dim3(256), 0, lpp::stream(),
                       d_dst, d_src, static_cast<size_t>(n));
    LPP_CHECK_LAUNCH("convert_f32_to_f16_kernel");
    return LPP_OK;
}

lpp_status lpp_gemv(float* d_out, const float* d_x, const void* d_w, void* d_workspace, int n,
                    int d, int precision) {
    (void)d_workspace;
    LPP_REQUIRE(n >= 0 && d >= 0, "lpp_gemv: n = %d, d = %d", n, d);
    if (n == 0) return LPP_OK;
    LPP_REQUIRE(d_out && d_x && d_w, "lpp_gemv: null pointer");
    LPP_REQUIRE(static_cast<const void*>(d_out) != static_cast<const void*>(d_x),
                "lpp_gemv: out must not alias x");
    // matmul.cu:142-145: every precision other than FP16 takes the fp32 kernel.
    if (precision == LPP_WEIGHT_FP16) return lpp::gemv_dispatch<true>(d_out, d_x, d_w, n, d);
    return lpp::gemv_dispatch<false>(d_out, d_x, d_w, n, d);
}

}  // extern "C"
