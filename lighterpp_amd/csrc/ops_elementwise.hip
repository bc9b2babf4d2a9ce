// ops_elementwise.hip -- lpp_rmsnorm, lpp_rope, lpp_swiglu, lpp_residual_add,
// lpp_scatter_kv and the fill kernel behind lpp_memset.
//
// Replace cuda_rmsnorm (reference src/RMSNorm.cu:11-71), cuda_rope
// (src/rope.cu:7-38), cuda_swiglu (src/swiglu.cu:6-33), cuda_residual_add
// (src/residual.cu:5-31) and cuda_scatter_kv (src/scatter_kv.cu:6-26).  The
// arithmetic follows the CPU operators (src/ops.cpp) so that everything that
// can be bit-exact is: true division, 1/sqrtf, no fused multiply-add where the
// CPU build has none.
#include "lpp_device.hpp"
#include "lpp_internal.hpp"

namespace lpp {
namespace {

using namespace dev;

constexpr int kNormThreads = 1024;

// ops.cpp:20-32.  One workgroup; the sum of squares is a tree instead of the
// CPU's running sum, the rest is the same expression: (x * s) * w with
// s = 1 / sqrtf(mean + 1e-5f).
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(float* out, const float* x,
                                                               const float* __restrict__ w,
                                                               int n) {
#pragma clang fp contract(off)
    __shared__ float scratch[16];
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += kNormThreads) {
        float v = x[i];
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    ss /= static_cast<float>(n);
    ss += 1e-5f;
    const float scale = 1.0f / sqrtf(ss);
    for (int i = threadIdx.x; i < n; i += kNormThreads) out[i] = x[i] * scale * w[i];
}

// ops.cpp:34-54 with (cos, sin) read from the host-built table row of `pos`.
__global__ __launch_bounds__(256) void rope_kernel(float* q, float* k, const float2* __restrict__ cs_row,
                                                   int dim, int kv_dim, int head_size) {
#pragma clang fp contract(off)
    const int pair = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    const int i = pair * 2;
    if (i >= dim) return;
    const float2 cs = cs_row[(i % head_size) >> 1];
    const float c = cs.x, s = cs.y;
    const float a = q[i], b = q[i + 1];
    q[i] = a * c - b * s;
    q[i + 1] = a * s + b * c;
    if (i < kv_dim) {
        const float ka = k[i], kb = k[i + 1];
        k[i] = ka * c - kb * s;
        k[i + 1] = ka * s + kb * c;
    }
}

// ops.cpp:78-87: (g * (1 / (1 + expf(-g)))) * u.
__global__ __launch_bounds__(256) void swiglu_kernel(float* hb, const float* h1, const float* h3,
                                                     int size) {
#pragma clang fp contract(off)
    int i = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    const int stride = static_cast<int>(gridDim.x) * 256;
    for (; i < size; i += stride) {
        const float g = h1[i];
        const float u = h3[i];
        const float sigma = 1.0f / (1.0f + expf(-g));
        hb[i] = (g * sigma) * u;
    }
}

// model.cpp:232,239.
__global__ __launch_bounds__(256) void residual_add_kernel(float* out, const float* a,
                                                           const float* b, int n) {
    int i = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    const int stride = static_cast<int>(gridDim.x) * 256;
    for (; i < n; i += stride) out[i] = a[i] + b[i];
}

// model.cpp:171-176 index logic (dst = layer*(kv_dim*seq_len) + head*(seq_len*hs)
// + pos*hs + i), evaluated in 64 bits; value rounded to nearest-even binary16.
__global__ __launch_bounds__(256) void scatter_kv_kernel(uint16_t* key_cache, uint16_t* value_cache,
                                                         const float* __restrict__ k,
                                                         const float* __restrict__ v, int layer,
                                                         int pos, int n_kv_heads, int head_size,
                                                         int seq_len) {
    const int idx = static_cast<int>(blockIdx.x) * 256 + static_cast<int>(threadIdx.x);
    const int kv_dim = n_kv_heads * head_size;
    if (idx >= kv_dim) return;
    const int head = idx / head_size;
    const int within = idx - head * head_size;
    const size_t dst = static_cast<size_t>(layer) * kv_dim * seq_len +
                       static_cast<size_t>(head) * seq_len * head_size +
                       static_cast<size_t>(pos) * head_size + within;
    key_cache[dst] = f32_to_f16_bits(k[idx]);
    value_cache[dst] = f32_to_f16_bits(v[idx]);
}

__global__ __launch_bounds__(256) void fill_bytes_kernel(unsigned char* p, unsigned char value,
                                                         size_t bytes) {
    // 16 bytes per thread where alignment allows, single bytes at the ragged ends.
    const size_t tid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t nthreads = static_cast<size_t>(gridDim.x) * 256;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
    size_t head = (16 - (addr & 15)) & 15;
    if (head > bytes) head = bytes;
    const size_t nvec = (bytes - head) / 16;
    const size_t tail_start = head + nvec * 16;
    const uint32_t word = 0x01010101u * value;
    uintx4* vec = reinterpret_cast<uintx4*>(p + head);
    for (size_t i = tid; i < nvec; i += nthreads) vec[i] = uintx4{word, word, word, word};
    for (size_t i = tid; i < head; i += nthreads) p[i] = value;
    for (size_t i = tail_start + tid; i < bytes; i += nthreads) p[i] = value;
}

int grid_for(long work_items, int per_block, int max_blocks_per_cu) {
    long blocks = (work_items + per_block - 1) / per_block;
    const long cap = static_cast<long>(compute_units()) * max_blocks_per_cu;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return static_cast<int>(blocks);
}

}  // namespace
}  // namespace lpp

extern "C" {

lpp_status lpp_rmsnorm(float* d_out, const float* d_x, const float* d_w, int n) {
    LPP_REQUIRE(n > 0, "lpp_rmsnorm: n = %d", n);
    LPP_REQUIRE(d_out && d_x && d_w, "lpp_rmsnorm: null pointer");
    hipLaunchKernelGGL(lpp::rmsnorm_kernel, dim3(1), dim3(lpp::kNormThreads), 0, lpp::stream(),
                       d_out, d_x, d_w, n);
    LPP_CHECK_LAUNCH("rmsnorm_kernel");
    return LPP_OK;
}

lpp_status lpp_rope(float* d_q, float* d_k, int pos, int dim, int kv_dim, int head_size,
                    float rope_base) {
    LPP_REQUIRE(d_q != nullptr, "lpp_rope: null q");
    LPP_REQUIRE(pos >= 0, "lpp_rope: pos = %d", pos);
    LPP_REQUIRE(dim > 0 && head_size > 0 && dim % 2 == 0 && head_size % 2 == 0,
                "lpp_rope: dim = %d and head_size = %d must be positive and even", dim, head_size);
    LPP_REQUIRE(kv_dim >= 0 && kv_dim <= dim && kv_dim % 2 == 0, "lpp_rope: kv_dim = %d", kv_dim);
    LPP_REQUIRE(kv_dim == 0 || d_k != nullptr, "lpp_rope: null k");
    const float2* table = nullptr;
    LPP_TRY(lpp::rope_table(head_size, rope_base, pos + 1, &table));
    const float2* row = table + static_cast<size_t>(pos) * (head_size / 2);
    const int pairs = dim / 2;
    hipLaunchKernelGGL(lpp::rope_kernel, dim3((pairs + 255) / 256), dim3(256), 0, lpp::stream(),
                       d_q, d_k, row, dim, kv_dim, head_size);
    LPP_CHECK_LAUNCH("rope_kernel");
    return LPP_OK;
}

lpp_status lpp_swiglu(float* d_hb, const float* d_h1, const float* d_h3, int size) {
    LPP_REQUIRE(size >= 0, "lpp_swiglu: size = %d", size);
    if (size == 0) return LPP_OK;
    LPP_REQUIRE(d_hb && d_h1 && d_h3, "lpp_swiglu: null pointer");
    hipLaunchKernelGGL(lpp::swiglu_kernel, dim3(lpp::grid_for(size, 256, 8)), dim3(256), 0,
                       lpp::stream(), d_hb, d_h1, d_h3, size);
    LPP_CHECK_LAUNCH("swiglu_kernel");
    return LPP_OK;
}

lpp_status lpp_residual_add(float* d_out, const float* d_a, const float* d_b, int n) {
    LPP_REQUIRE(n >= 0, "lpp_residual_add: n = %d", n);
    if (n == 0) return LPP_OK;
    LPP_REQUIRE(d_out && d_a && d_b, "lpp_residual_add: null pointer");
    hipLaunchKernelGGL(lpp::residual_add_kernel, dim3(lpp::grid_for(n, 256, 8)), dim3(256), 0,
                       lpp::stream(), d_out, d_a, d_b, n);
    LPP_CHECK_LAUNCH("residual_add_kernel");
    return LPP_OK;
}

lpp_status lpp_scatter_kv(lpp_half* d_key_cache, lpp_half* d_value_cache, const float* d_k,
                          const float* d_v, int layer, int pos, int n_kv_heads, int head_size,
                          int seq_len) {
    LPP_REQUIRE(d_key_cache && d_value_cache && d_k && d_v, "lpp_scatter_kv: null pointer");
    LPP_REQUIRE(layer >= 0 && n_kv_heads > 0 && head_size > 0 && seq_len > 0,
                "lpp_scatter_kv: layer = %d, n_kv_heads = %d, head_size = %d, seq_len = %d", layer,
                n_kv_heads, head_size, seq_len);
    LPP_REQUIRE(pos >= 0 && pos < seq_len, "lpp_scatter_kv: pos = %d outside [0, %d)", pos, seq_len);
    const int kv_dim = n_kv_heads * head_size;
    hipLaunchKernelGGL(lpp::scatter_kv_kernel, dim3((kv_dim + 255) / 256), dim3(256), 0,
                       lpp::stream(), d_key_cache, d_value_cache, d_k, d_v, layer, pos, n_kv_heads,
                       head_size, seq_len);
    LPP_CHECK_LAUNCH("scatter_kv_kernel");
    return LPP_OK;
}

// A fill kernel rather than hipMemsetAsync, so the call is safe to record into a
// HIP graph.
lpp_status lpp_memset(void* d_ptr, int value, size_t bytes) {
    if (bytes == 0) return LPP_OK;
    LPP_REQUIRE(d_ptr != nullptr, "lpp_memset: null pointer");
    hipLaunchKernelGGL(lpp::fill_bytes_kernel, dim3(lpp::grid_for(static_cast<long>(bytes / 16 + 1), 256, 8)),
                       dim3(256), 0, lpp::stream(), static_cast<unsigned char*>(d_ptr),
                       static_cast<unsigned char>(value), bytes);
    LPP_CHECK_LAUNCH("fill_bytes_kernel");
    return LPP_OK;
}

}  // extern "C"
