// Shared helpers of the C++ call-site test programs: failure counting, host<->device copies,
// seeded inputs in either storage type, and the comparison rules (bit-exact; fp32 1e-5 relative;
// fp16 2 ulp and 1e-2 absolute, with the ulp taken relative to the operands where results cancel).
#pragma once
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "isp_oracle.h"
#include "src/utils/tensor.h"

static int g_failures = 0;
#define EXPECT(cond, ...)                                   \
    do {                                                    \
        if (!(cond)) {                                      \
            g_failures++;                                   \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                       \
            std::printf("\n");                              \
        }                                                   \
    } while (0)

// ---- host <-> storage conversion through the oracle's binary16 routines
template <typename T> struct Host;
template <> struct Host<float> {
    using Store = float;
    static float to(float x) { return x; }
    static float from(float x) { return x; }
};
template <> struct Host<half> {
    using Store = uint16_t;
    static uint16_t to(float x) { return isp_oracle_f2h(x); }
    static float from(uint16_t x) { return isp_oracle_h2f(x); }
};

template <typename S>
S* to_device(const std::vector<S>& h) {
    S* d = nullptr;
    CHECK(hipMalloc((void**)&d, h.size() * sizeof(S) + 16));
    CHECK(hipMemcpy(d, h.data(), h.size() * sizeof(S), hipMemcpyHostToDevice));
    return d;
}
template <typename S>
std::vector<S> to_host(const S* d, size_t n) {
    std::vector<S> h(n);
    CHECK(hipMemcpy(h.data(), d, n * sizeof(S), hipMemcpyDeviceToHost));
    return h;
}

template <typename T>
std::vector<typename Host<T>::Store> randn(size_t n, float scale, std::mt19937& gen, float shift = 0.f) {
    std::normal_distribution<float> dist(0.f, 1.f);
    std::vector<typename Host<T>::Store> v(n);
    for (auto& x : v) x = Host<T>::to(shift + scale * dist(gen));
    return v;
}

static double f16_ulp(double at) {
    at = std::fabs(at);
    if (at < std::ldexp(1.0, -14)) at = std::ldexp(1.0, -14);
    return std::ldexp(1.0, (int)std::floor(std::log2(at)) - 10);
}

// fp32: |err| <= 1e-5 * scale; fp16: <= 2 ulp (ulp taken at max(|ref|, magnitude/4096)) and <= 1e-2.
template <typename T>
void compare(const std::vector<typename Host<T>::Store>& got,
             const std::vector<typename Host<T>::Store>& ref, const char* what,
             const std::function<double(size_t)>& magnitude = nullptr) {
    EXPECT(got.size() == ref.size(), "%s: size", what);
    size_t bad = 0, differ = 0;
    for (size_t i = 0; i < got.size(); i++) {
        const double g = Host<T>::from(got[i]), r = Host<T>::from(ref[i]);
        if (got[i] == ref[i]) continue;
        differ++;
        const double err = std::fabs(g - r);
        const double mag = magnitude ? magnitude(i) : std::fabs(r);
        if (std::is_same<T, float>::value) {
            if (err > 1e-5 * std::max(mag, std::fabs(r)) + 1e-30) bad++;
        } else {
            const double ulps = err / f16_ulp(std::max(std::fabs(r), mag / 4096.0));
            if (ulps > 2.0 || (err > 1e-2 && ulps > 1.0)) bad++;
        }
        if (bad == 1 && bad > 0 && err > 0) {
            static bool shown = false;
            if (!shown) { std::printf("  first mismatch %s[%zu]: got %.9g ref %.9g\n", what, i, g, r); shown = true; }
        }
    }
    EXPECT(bad == 0, "%s: %zu of %zu elements out of tolerance", what, bad, got.size());
    if (!std::is_same<T, float>::value)
        EXPECT(differ * 50 <= got.size() + 50, "%s: %zu elements differ from the oracle", what, differ);
}


template <typename F>
bool throws(F f) {
    try { f(); } catch (const std::runtime_error& e) { return std::strstr(e.what(), "[oneLLM][ERROR]") != nullptr; }
    return false;
}
