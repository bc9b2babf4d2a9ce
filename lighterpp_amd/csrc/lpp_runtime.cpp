// lpp_runtime.cpp -- section C of lpp.h: device selection, the launch stream,
// raw device memory and error reporting.  The reference gets all of this from
// the CUDA runtime's implicit default stream and unchecked cudaMalloc/cudaMemcpy
// calls (model.cpp:58-80, 349, 370); here every call is checked and reported.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "lpp_internal.hpp"

namespace lpp {
namespace {

thread_local char g_error[512] = "";

struct Runtime {
    std::mutex mu;
    bool ready = false;
    int device = -1;
    int cus = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t current = nullptr;
};
Runtime g_rt;

struct RopeTable {
    float2* d = nullptr;
    int positions = 0;
};
std::map<std::tuple<int, int, uint32_t>, RopeTable> g_rope;  // key: device, head_size, base bits

// Test hooks (lpp_set_test_option): which of its alternatives the library may pick by itself.
int g_test_options[LPP_OPT_COUNT] = {1, 1, 1, 1, 0, 1, 1, 1, 1, 1, 1};
unsigned g_test_epoch = 1;  // advanced by every change a model has to act on

}  // namespace

int test_option(int option) { return (option >= 0 && option < LPP_OPT_COUNT) ? g_test_options[option] : 0; }
unsigned test_options_epoch() { return g_test_epoch; }
bool take_forced_ticket_failure() {
    if (g_test_options[LPP_OPT_DECODE_FAIL_TICKETS] <= 0) return false;
    g_test_options[LPP_OPT_DECODE_FAIL_TICKETS] -= 1;
    return g_test_options[LPP_OPT_DECODE_FAIL_TICKETS] == 0;
}

lpp_status fail(lpp_status code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

// First use selects device 0 and creates the stream, so an operator called
// before lpp_init behaves like the reference's implicit-context launches.
hipStream_t stream() {
    if (!g_rt.ready) (void)lpp_init(0);
    return g_rt.current;
}
int compute_units() { return g_rt.cus > 0 ? g_rt.cus : 256; }

lpp_status rope_table(int head_size, float rope_base, int min_positions, const float2** d_table) {
    if (!g_rt.ready) LPP_TRY(lpp_init(0));
    uint32_t base_bits;
    std::memcpy(&base_bits, &rope_base, sizeof base_bits);
    std::lock_guard<std::mutex> lock(g_rt.mu);
    RopeTable& t = g_rope[std::make_tuple(g_rt.device, head_size, base_bits)];
    if (t.positions < min_positions) {
        int want = t.positions > 0 ? t.positions : 256;
        while (want < min_positions) want *= 2;
        const int half = head_size / 2;
        std::vector<float2> host(static_cast<size_t>(want) * half);
        // ops.cpp:36-40: freq = 1/powf(base, idx/head_size) with idx = 2*j (the even
        // member of the pair, modulo head_size); angle = (float)pos * freq.
        std::vector<float> freq(half);
        for (int j = 0; j < half; ++j)
            freq[j] = 1.0f / powf(rope_base, (2 * j) / static_cast<float>(head_size));
        for (int p = 0; p < want; ++p) {
            for (int j = 0; j < half; ++j) {
                float angle = p * freq[j];
                host[static_cast<size_t>(p) * half + j] = make_float2(cosf(angle), sinf(angle));
            }
        }
        float2* fresh = nullptr;
        if (hipMalloc(&fresh, host.size() * sizeof(float2)) != hipSuccess)
            return fail(LPP_ERR_OOM, "rope table: hipMalloc of %zu bytes failed",
                        host.size() * sizeof(float2));
        // Kernels already queued may still read the old table: drain before swapping.
        LPP_HIP(hipStreamSynchronize(g_rt.current));
        LPP_HIP(hipMemcpy(fresh, host.data(), host.size() * sizeof(float2), hipMemcpyHostToDevice));
        if (t.d) LPP_HIP(hipFree(t.d));
        t.d = fresh;
        t.positions = want;
    }
    *d_table = t.d;
    return LPP_OK;
}

}  // namespace lpp

using lpp::fail;

extern "C" {

const char* lpp_last_error(void) { return lpp::g_error; }

const char* lpp_version(void) { return "lighterpp_amd 0.1 (gfx950)"; }

lpp_status lpp_device_count(int* count) {
    LPP_REQUIRE(count != nullptr, "lpp_device_count: null output");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return LPP_OK;
}

lpp_status lpp_init(int device) {
    std::lock_guard<std::mutex> lock(lpp::g_rt.mu);
    if (lpp::g_rt.ready && lpp::g_rt.device == device) return LPP_OK;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(LPP_ERR_HIP, "lpp_init: no HIP device visible");
    }
    LPP_REQUIRE(device >= 0 && device < n, "lpp_init: device %d out of range (0..%d)", device, n - 1);
    LPP_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    LPP_HIP(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(LPP_ERR_UNSUPPORTED, "lpp_init: device is %s; this library carries gfx950 code only",
                    prop.gcnArchName);
    if (lpp::g_rt.own_stream == nullptr || lpp::g_rt.device != device) {
        hipStream_t s = nullptr;
        LPP_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        lpp::g_rt.own_stream = s;
    }
    lpp::g_rt.current = lpp::g_rt.own_stream;
    lpp::g_rt.device = device;
    lpp::g_rt.cus = prop.multiProcessorCount;
    lpp::g_rt.ready = true;
    // What the allocation-free prefill GEMM needs on this device is set up here, so that it never has to do so
    // itself; a failure is that entry point's to report (prefill_gemm_scratch_status), not the whole library's.
    lpp::prefill_gemm_scratch_setup();
    return LPP_OK;
}

lpp_status lpp_set_stream(void* hip_stream) {
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    lpp::g_rt.current = hip_stream ? static_cast<hipStream_t>(hip_stream) : lpp::g_rt.own_stream;
    return LPP_OK;
}

lpp_status lpp_get_stream(void** hip_stream) {
    LPP_REQUIRE(hip_stream != nullptr, "lpp_get_stream: null output");
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    *hip_stream = static_cast<void*>(lpp::g_rt.current);
    return LPP_OK;
}

lpp_status lpp_synchronize(void) {
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    LPP_HIP(hipStreamSynchronize(lpp::g_rt.current));
    return LPP_OK;
}

lpp_status lpp_malloc(void** d_ptr, size_t bytes) {
    LPP_REQUIRE(d_ptr != nullptr, "lpp_malloc: null output");
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    *d_ptr = nullptr;
    if (bytes == 0) return LPP_OK;
    hipError_t e = hipMalloc(d_ptr, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *d_ptr = nullptr;
        return fail(LPP_ERR_OOM, "lpp_malloc: hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    return LPP_OK;
}

lpp_status lpp_free(void* d_ptr) {
    if (d_ptr == nullptr) return LPP_OK;
    LPP_HIP(hipFree(d_ptr));
    return LPP_OK;
}

lpp_status lpp_malloc_host(void** h_ptr, size_t bytes) {
    LPP_REQUIRE(h_ptr != nullptr, "lpp_malloc_host: null output");
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    *h_ptr = nullptr;
    if (bytes == 0) return LPP_OK;
    hipError_t e = hipHostMalloc(h_ptr, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *h_ptr = nullptr;
        return fail(LPP_ERR_OOM, "lpp_malloc_host: hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    return LPP_OK;
}

lpp_status lpp_free_host(void* h_ptr) {
    if (h_ptr == nullptr) return LPP_OK;
    LPP_HIP(hipHostFree(h_ptr));
    return LPP_OK;
}

// The three copies are stream-ordered with the kernels and return when done.
lpp_status lpp_memcpy_h2d(void* d_dst, const void* h_src, size_t bytes) {
    if (bytes == 0) return LPP_OK;
    LPP_REQUIRE(d_dst && h_src, "lpp_memcpy_h2d: null pointer");
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    LPP_HIP(hipMemcpyAsync(d_dst, h_src, bytes, hipMemcpyHostToDevice, lpp::g_rt.current));
    LPP_HIP(hipStreamSynchronize(lpp::g_rt.current));
    return LPP_OK;
}

lpp_status lpp_memcpy_d2h(void* h_dst, const void* d_src, size_t bytes) {
    if (bytes == 0) return LPP_OK;
    LPP_REQUIRE(h_dst && d_src, "lpp_memcpy_d2h: null pointer");
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    LPP_HIP(hipMemcpyAsync(h_dst, d_src, bytes, hipMemcpyDeviceToHost, lpp::g_rt.current));
    LPP_HIP(hipStreamSynchronize(lpp::g_rt.current));
    return LPP_OK;
}

lpp_status lpp_memcpy_d2d(void* d_dst, const void* d_src, size_t bytes) {
    if (bytes == 0) return LPP_OK;
    LPP_REQUIRE(d_dst && d_src, "lpp_memcpy_d2d: null pointer");
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    LPP_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, lpp::g_rt.current));
    return LPP_OK;
}

lpp_status lpp_set_test_option(int option, int value) {
    LPP_REQUIRE(option >= 0 && option < LPP_OPT_COUNT, "lpp_set_test_option: no option %d", option);
    if (lpp::g_test_options[option] != value) {
        lpp::g_test_options[option] = value;
        if (option != LPP_OPT_DECODE_FAIL_TICKETS) lpp::g_test_epoch += 1;
    }
    return LPP_OK;
}

lpp_status lpp_get_test_option(int option, int* value) {
    LPP_REQUIRE(option >= 0 && option < LPP_OPT_COUNT && value != nullptr, "lpp_get_test_option: no option %d", option);
    *value = lpp::g_test_options[option];
    return LPP_OK;
}

lpp_status lpp_device_info(char* name, size_t name_cap, int* compute_units, size_t* hbm_bytes) {
    if (!lpp::g_rt.ready) LPP_TRY(lpp_init(0));
    hipDeviceProp_t prop;
    LPP_HIP(hipGetDeviceProperties(&prop, lpp::g_rt.device));
    if (name && name_cap > 0) snprintf(name, name_cap, "%s (%s)", prop.name, prop.gcnArchName);
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (hbm_bytes) *hbm_bytes = prop.totalGlobalMem;
    return LPP_OK;
}

}  // extern "C"
