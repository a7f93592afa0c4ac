// Shared pieces of the two host harnesses: seeded s4 generators, device buffers, timing.
// The harnesses are the counterparts of the reference's test/test_correctness.cu and
// test/benchmark.cu: plain host C++ that packs operands with pack(), uploads them, calls the
// library through include/int4linear.h and checks / times the result.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "int4linear.h"

#define HIP_OK(expr)                                                                       \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #expr,           \
                         hipGetErrorString(e_));                                           \
            std::exit(2);                                                                  \
        }                                                                                  \
    } while (0)

namespace harness {

// splitmix64: tiny, seedable, identical on every host.
struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next()
    {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double unit() { return ((next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
};

// Uniform integers in [-8, 7], one per int (the packer's input format).
inline std::vector<int> uniform_s4(uint64_t seed, size_t count)
{
    Rng r(seed);
    std::vector<int> v(count);
    for (size_t i = 0; i < count; i += 16) {
        uint64_t bits = r.next();
        for (size_t j = i; j < std::min(count, i + 16); ++j, bits >>= 4)
            v[j] = (int)(bits & 15) - 8;
    }
    return v;
}

// round(normal(0, sigma)) clamped to [-8, 7] (decode-style activations).
inline std::vector<int> normal_s4(uint64_t seed, size_t count, double sigma = 2.0)
{
    Rng r(seed);
    std::vector<int> v(count);
    for (size_t i = 0; i < count; i += 2) {
        const double u1 = r.unit(), u2 = r.unit();
        const double rad = std::sqrt(-2.0 * std::log(u1)) * sigma;
        const double z[2] = {rad * std::cos(6.283185307179586 * u2), rad * std::sin(6.283185307179586 * u2)};
        for (size_t j = 0; j < 2 && i + j < count; ++j)
            v[i + j] = (int)std::clamp(std::lrint(z[j]), -8l, 7l);
    }
    return v;
}

struct DeviceBuffer {
    void *p = nullptr;
    size_t bytes = 0;
    explicit DeviceBuffer(size_t n) : bytes(n) { HIP_OK(hipMalloc(&p, n ? n : 1)); }
    ~DeviceBuffer() { (void)hipFree(p); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
};

// rows x k values -> packed words on the device (pack() writes ceil(k/8) words per row).
inline void upload_packed(const std::vector<int> &values, int rows, int k, DeviceBuffer &dst)
{
    std::vector<int> words((size_t)rows * ((k + 7) / 8));
    pack(values.data(), words.data(), rows, k);
    HIP_OK(hipMemcpy(dst.p, words.data(), words.size() * sizeof(int), hipMemcpyHostToDevice));
}

struct Shape {
    int m, n, k;
};

// "MxNxK" or "M,N,K"
inline bool parse_shape(const char *s, Shape &out)
{
    return std::sscanf(s, "%dx%dx%d", &out.m, &out.n, &out.k) == 3 ||
           std::sscanf(s, "%d,%d,%d", &out.m, &out.n, &out.k) == 3;
}

}  // namespace harness
