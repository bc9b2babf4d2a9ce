// lpp_kernels_compat.h -- drop-in for the reference's src/kernels.cuh.
//
// A Lighter++ source tree built against liblpp_hip.so includes this header
// where it used to include "kernels.cuh": model.cpp, loader.cpp, main.cpp and
// runtests.cpp keep calling the same twelve cuda_* wrappers (kernels.cuh:24-36)
// with the same argument meaning; each forwards to the C ABI of lpp.h.  The
// reference's wrappers return void and abort on a launch error through
// checkCuda (kernels.cuh:14-21); these do the same by checking the status the
// C ABI returns, so a failure prints the library's message and exits instead of
// passing silently.
//
// C++ only (the reference's wrappers are C++ free functions).  No CUDA or HIP
// header is needed by the including file: device pointers are plain pointers.
#pragma once

#include <stdio.h>
#include <stdlib.h>

#include "lpp.h"

enum WeightPrecision : int;  // defined by the reference's model.h:8-12

// kernels.cuh:11.  main.cpp:130 refuses models whose hidden_dim exceeds this; the
// HIP kernels stage up to 16384 floats of activations in LDS.
#define MAX_SHARED_FLOATS 16384

// Binary16 storage type standing in for CUDA's __half in the signatures below.
typedef lpp_half __half;

// kernels.cuh:14-21, for status codes of this library.
#define checkCuda(call)                                                          \
    {                                                                            \
        const lpp_status lpp_compat_status = (call);                             \
        if (lpp_compat_status != LPP_OK) {                                       \
            printf("Error: %s:%d, ", __FILE__, __LINE__);                        \
            printf("code:%d, reason: %s\n", lpp_compat_status, lpp_last_error()); \
            exit(1);                                                             \
        }                                                                        \
    }

// kernels.cuh:24
inline void cuda_convert_f32_to_f16(void* dst, float* src, int n) {
    checkCuda(lpp_convert_f32_to_f16(static_cast<lpp_half*>(dst), src, n));
}

// kernels.cuh:26
inline void cuda_gemv(float* d_out, float* d_x, void* d_w, void* d_workspace, int n, int d,
                      WeightPrecision precision) {
    checkCuda(lpp_gemv(d_out, d_x, d_w, d_workspace, n, d, static_cast<int>(precision)));
}

// kernels.cuh:27
inline void cuda_rmsnorm(float* d_out, float* d_x, float* d_w, int n) {
    checkCuda(lpp_rmsnorm(d_out, d_x, d_w, n));
}

// kernels.cuh:28
inline void cuda_rope(float* d_q, float* d_k, int pos, int dim, int kv_dim, int head_size,
                      float rope_base) {
    checkCuda(lpp_rope(d_q, d_k, pos, dim, kv_dim, head_size, rope_base));
}

// kernels.cuh:29
inline void cuda_swiglu(float* d_hb, float* d_h1, float* d_h3, int size) {
    checkCuda(lpp_swiglu(d_hb, d_h1, d_h3, size));
}

// kernels.cuh:30
inline void cuda_softmax_multihead(float* d_out, float* d_x, int n_heads, int seq_len, int att_stride) {
    checkCuda(lpp_softmax_multihead(d_out, d_x, n_heads, seq_len, att_stride));
}

// kernels.cuh:31
inline void cuda_scale_multihead(float* d_att, float scale, int n_heads, int seq_len, int att_stride) {
    checkCuda(lpp_scale_multihead(d_att, scale, n_heads, seq_len, att_stride));
}

// kernels.cuh:32
inline void cuda_aggregation_multihead(float* d_out, const __half* d_v, const float* d_att, int n_heads,
                                       int seq_len, int head_size, int gqa_factor, int att_stride) {
    checkCuda(lpp_aggregation_multihead(d_out, d_v, d_att, n_heads, seq_len, head_size, gqa_factor,
                                        att_stride));
}

// kernels.cuh:33
inline void cuda_residual_add(float* d_out, const float* d_a, const float* d_b, int n) {
    checkCuda(lpp_residual_add(d_out, d_a, d_b, n));
}

// kernels.cuh:34
inline void cuda_scatter_kv(__half* d_key_cache, __half* d_value_cache, const float* d_k, const float* d_v,
                            int layer, int pos, int n_kv_heads, int head_size, int seq_len) {
    checkCuda(lpp_scatter_kv(d_key_cache, d_value_cache, d_k, d_v, layer, pos, n_kv_heads, head_size,
                             seq_len));
}

// kernels.cuh:35
inline void cuda_multihead_gemv(float* d_out, float* d_q, __half* d_k_cache, int layer, int pos, int n_heads,
                                int n_kv_heads, int head_size, int seq_len) {
    checkCuda(lpp_multihead_gemv(d_out, d_q, d_k_cache, layer, pos, n_heads, n_kv_heads, head_size, seq_len));
}

// kernels.cuh:36.  The reference's wrapper draws the uniform from libc on every
// call, greedy or not (sample.cu:211); so does this one, which keeps the rand()
// stream of a caller in step with the reference.
inline void cuda_sample(float* d_logits, int vocab_size, float temperature, float topp, float penalty,
                        int* d_history, int history_len, int* d_sampled_token, unsigned int* d_rng_state) {
    const float rand_val = (float)rand() / (float)RAND_MAX;
    checkCuda(lpp_sample(d_logits, vocab_size, temperature, topp, penalty, d_history, history_len,
                         d_sampled_token, d_rng_state, rand_val));
}
