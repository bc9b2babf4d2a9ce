// lpp_synth.cpp -- deterministic synthetic tensors and host-side binary16
// conversion.  The reference has no generator (its weights come from model
// files, src/loader.cpp); benchmarks and tests of this library run on seeded
// random-init weights, and both the GPU path and the CPU checker must see the
// same bytes, so the generator lives here, on the host, and is counter-based:
// element i of stream `seed` depends on (seed, i) only.
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "lpp_internal.hpp"

namespace lpp {
namespace {

inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// Uniform in (0, 1] with 53 bits.
inline double unit_open0(uint64_t bits) { return (static_cast<double>(bits >> 11) + 1.0) * (1.0 / 9007199254740992.0); }

// Box-Muller on two independent hashes of (seed, index); one normal per index so
// that any slice can be generated on its own.
inline double normal_at(uint64_t seed, uint64_t index) {
    const uint64_t key = splitmix64(seed ^ 0xD1B54A32D192ED03ull) + index * 2ull;
    const double u1 = unit_open0(splitmix64(key));
    const double u2 = unit_open0(splitmix64(key + 1ull));
    return std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586476925286766559 * u2);
}

// loader.cpp:346-379 states the widening; this is the same mapping written for
// bulk use.
inline float half_bits_to_float(uint16_t h) {
    const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
    int e = (h >> 10) & 0x1f;
    uint32_t m = h & 0x3ffu;
    uint32_t bits;
    if (e == 31) {
        bits = sign | 0x7f800000u | (m << 13);
    } else if (e == 0 && m == 0) {
        bits = sign;
    } else {
        if (e == 0) {
            e = 1;
            while (!(m & 0x400u)) {
                m <<= 1;
                --e;
            }
            m &= 0x3ffu;
        }
        bits = sign | (static_cast<uint32_t>(e + 112) << 23) | (m << 13);
    }
    float f;
    std::memcpy(&f, &bits, sizeof f);
    return f;
}

// Round to nearest even.
inline uint16_t float_to_half_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, sizeof x);
    const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
    const uint32_t ax = x & 0x7fffffffu;
    if (ax > 0x7f800000u) return static_cast<uint16_t>(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
    if (ax >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);
    if (ax <= 0x33000000u) return sign;
    const int e = static_cast<int>(ax >> 23) - 127;
    const uint32_t m = (ax & 0x7fffffu) | 0x800000u;
    const int shift = (e < -14) ? (13 + (-14 - e)) : 13;
    uint32_t keep = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (keep & 1u))) ++keep;
    if (e < -14) return static_cast<uint16_t>(sign | keep);
    return static_cast<uint16_t>(sign | static_cast<uint16_t>((static_cast<uint32_t>(e + 14) << 10) + keep));
}

template <typename Fn>
void parallel_for(size_t n, Fn fn) {
    unsigned hw = std::thread::hardware_concurrency();
    size_t workers = hw ? hw : 4;
    if (workers > 16) workers = 16;
    if (n < (1u << 16)) workers = 1;
    if (workers <= 1) {
        fn(0, n);
        return;
    }
    std::vector<std::thread> pool;
    const size_t per = (n + workers - 1) / workers;
    for (size_t w = 0; w < workers; ++w) {
        const size_t lo = w * per, hi = (lo + per < n) ? lo + per : n;
        if (lo >= hi) break;
        pool.emplace_back([=] { fn(lo, hi); });
    }
    for (auto& t : pool) t.join();
}

}  // namespace
}  // namespace lpp

extern "C" {

lpp_status lpp_synth_normal_f32(float* h_dst, size_t n, uint64_t seed, uint64_t first_index, float std) {
    LPP_REQUIRE(h_dst != nullptr || n == 0, "lpp_synth_normal_f32: null destination");
    lpp::parallel_for(n, [=](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; ++i)
            h_dst[i] = static_cast<float>(lpp::normal_at(seed, first_index + i) * static_cast<double>(std));
    });
    return LPP_OK;
}

lpp_status lpp_synth_normal_f16(lpp_half* h_dst, size_t n, uint64_t seed, uint64_t first_index, float std) {
    LPP_REQUIRE(h_dst != nullptr || n == 0, "lpp_synth_normal_f16: null destination");
    lpp::parallel_for(n, [=](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; ++i) {
            const float f = static_cast<float>(lpp::normal_at(seed, first_index + i) * static_cast<double>(std));
            h_dst[i] = lpp::float_to_half_bits(f);
        }
    });
    return LPP_OK;
}

lpp_status lpp_synth_uniform_f32(float* h_dst, size_t n, uint64_t seed, uint64_t first_index) {
    LPP_REQUIRE(h_dst != nullptr || n == 0, "lpp_synth_uniform_f32: null destination");
    const uint64_t key = lpp::splitmix64(seed ^ 0x2545F4914F6CDD1Dull);
    for (size_t i = 0; i < n; ++i) {
        // 24 random bits -> [0, 1) exactly representable in fp32.
        const uint64_t bits = lpp::splitmix64(key + first_index + i);
        h_dst[i] = static_cast<float>(bits >> 40) * (1.0f / 16777216.0f);
    }
    return LPP_OK;
}

lpp_status lpp_synth_token_ids(int* h_dst, size_t n, uint64_t seed, int vocab_size) {
    LPP_REQUIRE(h_dst != nullptr || n == 0, "lpp_synth_token_ids: null destination");
    LPP_REQUIRE(vocab_size > 0, "lpp_synth_token_ids: vocab_size = %d", vocab_size);
    const uint64_t key = lpp::splitmix64(seed ^ 0x9FB21C651E98DF25ull);
    for (size_t i = 0; i < n; ++i)
        h_dst[i] = static_cast<int>(lpp::splitmix64(key + i) % static_cast<uint64_t>(vocab_size));
    return LPP_OK;
}

lpp_status lpp_f16_to_f32_host(float* h_dst, const lpp_half* h_src, size_t n) {
    LPP_REQUIRE((h_dst && h_src) || n == 0, "lpp_f16_to_f32_host: null pointer");
    lpp::parallel_for(n, [=](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; ++i) h_dst[i] = lpp::half_bits_to_float(h_src[i]);
    });
    return LPP_OK;
}

lpp_status lpp_f32_to_f16_host(lpp_half* h_dst, const float* h_src, size_t n) {
    LPP_REQUIRE((h_dst && h_src) || n == 0, "lpp_f32_to_f16_host: null pointer");
    lpp::parallel_for(n, [=](size_t lo, size_t hi) {
        for (size_t i = lo; i < hi; ++i) h_dst[i] = lpp::float_to_half_bits(h_src[i]);
    });
    return LPP_OK;
}

}  // extern "C"
