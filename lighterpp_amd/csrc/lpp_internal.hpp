// lpp_internal.hpp -- shared by the host translation units of liblpp_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>

#include "lpp.h"

namespace lpp {

// Records a message for lpp_last_error() and returns `code`.
lpp_status fail(lpp_status code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Stream every launch of the library goes to.
hipStream_t stream();

// Number of compute units of the current device (cached after lpp_init).
int compute_units();

#define LPP_HIP(call)                                                                   \
    do {                                                                                \
        hipError_t lpp_e_ = (call);                                                     \
        if (lpp_e_ != hipSuccess)                                                       \
            return ::lpp::fail(LPP_ERR_HIP, "%s failed: %s (%s:%d)", #call,             \
                               hipGetErrorString(lpp_e_), __FILE__, __LINE__);          \
    } while (0)

#define LPP_TRY(call)                              \
    do {                                           \
        lpp_status lpp_s_ = (call);                \
        if (lpp_s_ != LPP_OK) return lpp_s_;       \
    } while (0)

#define LPP_REQUIRE(cond, ...)                                                 \
    do {                                                                       \
        if (!(cond)) return ::lpp::fail(LPP_ERR_INVALID_ARG, __VA_ARGS__);     \
    } while (0)

// After a kernel launch: surface launch-configuration errors.
#define LPP_CHECK_LAUNCH(name)                                                          \
    do {                                                                                \
        hipError_t lpp_e_ = hipGetLastError();                                          \
        if (lpp_e_ != hipSuccess)                                                       \
            return ::lpp::fail(LPP_ERR_HIP, "launch of %s failed: %s", name,            \
                               hipGetErrorString(lpp_e_));                              \
    } while (0)

// Device table of (cos, sin) per position and frequency index, computed on the
// host with powf/cosf/sinf in the reference's operation order (ops.cpp:36-40).
// Layout: [pos][head_size/2] float2.  Grows on demand; the returned pointer
// stays valid until the next call that has to grow the same table.
lpp_status rope_table(int head_size, float rope_base, int min_positions, const float2** d_table);

// Resolves, for the current device, the address of the device-resident scratch that
// lpp_prefill_gemm_noalloc works in (prefill.hip); lpp_init calls it once per device.  What it
// returned is kept per device and handed out by prefill_gemm_scratch_status(): the allocation-free
// entry point reports a failed set-up, nothing else in the library depends on it.
lpp_status prefill_gemm_scratch_setup();

// Test hooks (lpp_set_test_option).  The epoch changes whenever an option a model has acted on changes.
int test_option(int option);
unsigned test_options_epoch();
// LPP_OPT_DECODE_FAIL_TICKETS: counts a launch; true for the launch that is to fail.
bool take_forced_ticket_failure();

// Launch helpers implemented in the .hip files and used by the model code.
namespace k {

struct DecodeShape {
    int dim, hidden, n_layers, n_heads, n_kv_heads, head_size, kv_dim, vocab, seq_len;
    int w_f16;
};

}  // namespace k
}  // namespace lpp
