// ops_sample.hip -- lpp_sample.
//
// Replaces cuda_sample / fused_sample_kernel (reference src/sample.cu:6-214)
// with the semantics of the CPU sampler it is checked against
// (src/model.cpp:256-303).  The reference kernel is a single 256-thread block
// that walks the vocabulary in 501 serial rows; here the vocabulary is cut into
// chunks, one workgroup each, and the few cross-chunk values (maxima, sums,
// chunk masses) travel through a small device-resident scratch area between
// short launches on the same stream.  Calls that overlap on one device share
// that scratch and therefore must not run concurrently.
#include "lpp_internal.hpp"
#include "sampler.hpp"

namespace lpp {
namespace {

using namespace smp;

__device__ float g_chunk_max[kMaxChunks];
__device__ int g_chunk_arg[kMaxChunks];
__device__ float g_chunk_sum[kMaxChunks];
__device__ float g_chunk_prob[kMaxChunks];

__device__ __forceinline__ SampleScratch scratch() {
    return SampleScratch{g_chunk_max, g_chunk_arg, g_chunk_sum, g_chunk_prob};
}

__global__ __launch_bounds__(kSampleThreads) void penalty_kernel(float* logits, int vocab, float penalty,
                                                                 const int* history, int history_len) {
    penalty_all(logits, vocab, penalty, history, history_len);
}

__global__ __launch_bounds__(kSampleThreads) void scale_max_kernel(float* logits, int vocab, int chunk,
                                                                   float temperature) {
    scale_max_chunk<false>(logits, logits, vocab, chunk, blockIdx.x, temperature, 1.0f, nullptr, 0, scratch());
}

__global__ __launch_bounds__(kSampleThreads) void argmax_final_kernel(int nchunks, int* result) {
    const int a = argmax_over_chunks<false>(nchunks, scratch());
    if (threadIdx.x == 0) result[0] = a;
}

__global__ __launch_bounds__(kSampleThreads) void exp_sum_kernel(float* logits, int vocab, int chunk,
                                                                 int nchunks) {
    exp_sum_chunk<false>(logits, vocab, chunk, nchunks, blockIdx.x, scratch());
}

__global__ __launch_bounds__(kSampleThreads) void normalise_kernel(float* logits, int vocab, int chunk,
                                                                   int nchunks, int* result) {
    normalise_chunk<false>(logits, vocab, chunk, nchunks, blockIdx.x, scratch());
    if (blockIdx.x == 0 && threadIdx.x == 0) result[0] = vocab - 1;  // model.cpp:302 fallback
}

__global__ __launch_bounds__(kSampleThreads) void cdf_search_kernel(const float* probs, int vocab, int chunk,
                                                                    float r, int* result) {
    cdf_search_chunk<false>(probs, vocab, chunk, blockIdx.x, r, scratch(), result);
}

}  // namespace
}  // namespace lpp

extern "C" {

lpp_status lpp_sample(float* d_logits, int vocab_size, float temperature, float topp, float penalty,
                      const int* d_history, int history_len, int* d_sampled_token,
                      unsigned int* d_rng_state, float r) {
    using namespace lpp;
    (void)topp;         // sample.cu:210: accepted, never read
    (void)d_rng_state;  // model.cpp:366 passes nullptr
    LPP_REQUIRE(d_logits && d_sampled_token, "lpp_sample: null pointer");
    LPP_REQUIRE(vocab_size > 0, "lpp_sample: vocab_size = %d", vocab_size);
    LPP_REQUIRE(history_len >= 0, "lpp_sample: history_len = %d", history_len);

    const int chunk = chunk_size_for(vocab_size);
    const int nchunks = (vocab_size + chunk - 1) / chunk;
    hipStream_t s = stream();

    if (penalty > 1.0f && d_history != nullptr && history_len > 0) {
        hipLaunchKernelGGL(penalty_kernel, dim3(1), dim3(kSampleThreads), 0, s, d_logits, vocab_size, penalty,
                           d_history, history_len);
        LPP_CHECK_LAUNCH("penalty_kernel");
    }
    hipLaunchKernelGGL(scale_max_kernel, dim3(nchunks), dim3(kSampleThreads), 0, s, d_logits, vocab_size,
                       chunk, temperature);
    LPP_CHECK_LAUNCH("scale_max_kernel");
    if (temperature == 0.0f) {
        hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(kSampleThreads), 0, s, nchunks, d_sampled_token);
        LPP_CHECK_LAUNCH("argmax_final_kernel");
        return LPP_OK;
    }
    hipLaunchKernelGGL(exp_sum_kernel, dim3(nchunks), dim3(kSampleThreads), 0, s, d_logits, vocab_size, chunk,
                       nchunks);
    LPP_CHECK_LAUNCH("exp_sum_kernel");
    hipLaunchKernelGGL(normalise_kernel, dim3(nchunks), dim3(kSampleThreads), 0, s, d_logits, vocab_size, chunk,
                       nchunks, d_sampled_token);
    LPP_CHECK_LAUNCH("normalise_kernel");
    hipLaunchKernelGGL(cdf_search_kernel, dim3(nchunks), dim3(kSampleThreads), 0, s, d_logits, vocab_size, chunk,
                       r, d_sampled_token);
    LPP_CHECK_LAUNCH("cdf_search_kernel");
    return LPP_OK;
}

}  // extern "C"
