// What the matrix pipes sustain with nothing else going on: loops of nothing but MFMAs on
// operands held in registers, for the two instructions the library's large-shape kernels issue
// (v_mfma_i32_32x32x32_i8 and v_mfma_f32_32x32x64_f8f6f4 with FP6 E2M3 operands), on operand
// data of several kinds, among them every exact encoding of signed 4-bit values that the FP6 / BF6
// formats offer (the one the FP6 kernel uses, n/8 in E2M3, draws the least power of them).  The rate depends on the data: at the device's power limit the clock
// drops as more operand bits toggle, so "peak" is reached on zeros only.  Each line gives the
// throughput, the shader clock observed while the loop ran (cycle counter against the constant
// 100 MHz counter) and the share of the launch's cycles the matrix pipes were busy (32 cycles
// per MFMA of either kind, two waves per SIMD; launch gaps included).  The figures are what a GEMM kernel's rate can be read
// against; the reference has no counterpart (its README quotes no peak, README.md:57-62).
//
//   mfma_ceiling [--iters N]
//   prints lines:  [MFMA] <int8|fp6|bf6> <data> <TOPS> TOPS <GHz> GHz <busy %>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#define HIP_OK(expr)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            std::exit(2);                                                                             \
        }                                                                                             \
    } while (0)

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ unsigned mix(unsigned x)
{
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

enum Data {
    kZeros = 0, kRandom = 1, kNibbleTimes16 = 2, kSignExtendedS4 = 3,
    // Exact codes of uniform s4 values n: E2M3 n/8 (the FP6 kernel's), n/4, n/2; E3M2 n and n/16.
    kS4Codes = 4, kS4CodesQuarter = 5, kS4CodesHalf = 6, kBf6CodesOne = 7, kBf6CodesSixteenth = 8
};

// The magnitude bits (exponent and mantissa) of |n| = mg in the given exact encoding.
__device__ unsigned s4_magnitude_code(int data, unsigned mg)
{
    if (data == kS4Codes) return mg;                                  // E2M3, n/8: subnormals up to 7/8, then 1.0
    if (data == kS4CodesQuarter) return mg << 1;                       // E2M3, n/4
    if (data == kS4CodesHalf) return mg <= 4 ? mg << 2 : 2 * mg + 8;   // E2M3, n/2
    if (mg == 0) return 0;
    const int lg = 31 - __builtin_clz(mg);                             // mg = 2^lg * 1.ff
    const int ex = lg + 3 + (data == kBf6CodesOne ? 0 : -4);           // E3M2, bias 3
    return ex >= 1 ? ((unsigned)ex << 2) | (((mg << 2) >> lg) & 3u) : mg;   // below 4/16: subnormal mg/16
}

// One dword of int8 operand data of the given kind.
__device__ unsigned int8_word(int data, unsigned r)
{
    if (data == kZeros) return 0;
    if (data == kNibbleTimes16) return r & 0xF0F0F0F0u;   // what the int8 kernel feeds: 16 * s4
    if (data == kSignExtendedS4) {                          // s4 values as plain int8
        const unsigned lo = r & 0x0F0F0F0Fu;
        return lo | (((lo & 0x08080808u) >> 3) * 0xF0u);
    }
    return r;
}

// 32 six-bit values (192 bits) for one lane: random bits, or codes of uniform s4 values
// (sign << 5 | magnitude; kS4Codes is what the FP6 kernel's converter writes).
__device__ v8i fp6_operand(int data, unsigned seed)
{
    unsigned w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (data == kRandom)
        for (int i = 0; i < 6; ++i) w[i] = mix(seed + i);
    if (data >= kS4Codes)
        for (int e = 0; e < 32; ++e) {
            const int n = (int)(mix(seed + 100 + e) & 15u) - 8;
            const unsigned code = (n < 0 ? 32u : 0u) | s4_magnitude_code(data, (unsigned)(n < 0 ? -n : n));
            const int bit = 6 * e;
            w[bit >> 5] |= code << (bit & 31);
            if ((bit & 31) > 26) w[(bit >> 5) + 1] |= code >> (32 - (bit & 31));
        }
    return (v8i){(int)w[0], (int)w[1], (int)w[2], (int)w[3], (int)w[4], (int)w[5], 0, 0};
}

// cycles[0] = shader cycles, cycles[1] = 100 MHz ticks of the loop, as seen by wave 0 of block 0
// FMT: the instruction's operand format field (2 = E2M3, 3 = E3M2)
template <bool FP6, int FMT = 2>
__global__ __launch_bounds__(512) void mfma_loop(int *out, long long *cycles, int iters, int data)
{
    const unsigned seed = (threadIdx.x + blockIdx.x * 512u) * 2654435761u;
    int sum = 0;
    long long c0 = 0, r0 = 0, c1 = 0, r1 = 0;
    if constexpr (FP6) {
        v16f acc[8];
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
        v8i a[4], b[4];
        for (int i = 0; i < 4; ++i) { a[i] = fp6_operand(data, seed + 1000 * i); b[i] = fp6_operand(data, seed + 77 + 1000 * i); }
        c0 = __builtin_readcyclecounter(); r0 = __builtin_amdgcn_s_memrealtime();
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i + (i >> 2)) & 3], acc[i], FMT, FMT, 0, 0, 0, 0);
        }
        c1 = __builtin_readcyclecounter(); r1 = __builtin_amdgcn_s_memrealtime();
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 16; ++j) sum += (int)acc[i][j];
    } else {
        v16i acc[8];
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 16; ++j) acc[i][j] = 0;
        v4i a[4], b[4];
        for (int i = 0; i < 4; ++i) for (int d = 0; d < 4; ++d) {
            a[i][d] = (int)int8_word(data, mix(seed + i * 8 + d));
            b[i][d] = (int)int8_word(data, mix(seed + 1000 + i * 8 + d));
        }
        c0 = __builtin_readcyclecounter(); r0 = __builtin_amdgcn_s_memrealtime();
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[(i + (i >> 2)) & 3], acc[i], 0, 0, 0);
        }
        c1 = __builtin_readcyclecounter(); r1 = __builtin_amdgcn_s_memrealtime();
        for (int i = 0; i < 8; ++i) for (int j = 0; j < 16; ++j) sum += acc[i][j];
    }
    out[blockIdx.x * 512 + threadIdx.x] = sum;
    if (blockIdx.x == 0 && threadIdx.x == 0) { cycles[0] = c1 - c0; cycles[1] = r1 - r0; }
}

template <bool FP6, int FMT = 2>
void run(const char *kind, const char *name, int data, int iters, int cus, int *out, long long *cycles_d)
{
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    const int launches = 20;
    // untimed: lets the clock settle under this load
    for (int l = 0; l < launches; ++l) mfma_loop<FP6, FMT><<<cus, 512>>>(out, cycles_d, iters, data);
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipEventRecord(e0));
    for (int l = 0; l < launches; ++l) mfma_loop<FP6, FMT><<<cus, 512>>>(out, cycles_d, iters, data);
    HIP_OK(hipEventRecord(e1));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    long long cyc[2];
    HIP_OK(hipMemcpy(cyc, cycles_d, sizeof(cyc), hipMemcpyDeviceToHost));
    const double mac_per_mfma = FP6 ? 32.0 * 32 * 64 : 32.0 * 32 * 32;
    const double ops = 2.0 * mac_per_mfma * 8 * iters * 8.0 * cus * launches;  // 8 MFMAs x 8 waves per workgroup
    const double ghz = (double)cyc[0] / ((double)cyc[1] * 10e-9) / 1e9;
    // two waves per SIMD, 8 * iters MFMAs each, 32 cycles per MFMA, over a launch's share of the
    // timed interval at the observed clock (the oldest wave of a SIMD gets the pipe first, so
    // one wave's own loop time says nothing about the SIMD)
    const double busy = 2.0 * 8 * iters * 32.0 / ((double)ms * 1e-3 / launches * ghz * 1e9);
    std::printf("[MFMA] %s %-22s %8.1f TOPS %5.2f GHz %5.1f %% busy\n", kind, name, ops / (ms * 1e-3) / 1e12, ghz, 100.0 * busy);
    std::fflush(stdout);
}

}  // namespace

int main(int argc, char **argv)
{
    int iters = 4000;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--iters") && i + 1 < argc) iters = std::atoi(argv[++i]);
        else { std::fprintf(stderr, "usage: mfma_ceiling [--iters N]\n"); return 2; }
    }
    if (iters < 1) { std::fprintf(stderr, "usage: mfma_ceiling [--iters N]\n"); return 2; }
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    int *out = nullptr;
    long long *cycles = nullptr;
    HIP_OK(hipMalloc(&out, (size_t)cus * 512 * 4));
    HIP_OK(hipMalloc(&cycles, 16));
    run<false>("int8", "zeros", kZeros, iters, cus, out, cycles);
    run<false>("int8", "random-int8", kRandom, iters, cus, out, cycles);
    run<false>("int8", "16x-s4 (kernel's form)", kNibbleTimes16, iters, cus, out, cycles);
    run<false>("int8", "sign-extended-s4", kSignExtendedS4, iters, cus, out, cycles);
    run<true>("fp6", "zeros", kZeros, iters, cus, out, cycles);
    run<true>("fp6", "random-bits", kRandom, iters, cus, out, cycles);
    run<true>("fp6", "s4-codes (kernel's form)", kS4Codes, iters, cus, out, cycles);
    // the other exact encodings of s4 values the instruction offers
    run<true>("fp6", "s4-codes n/4 (E2M3)", kS4CodesQuarter, iters, cus, out, cycles);
    run<true>("fp6", "s4-codes n/2 (E2M3)", kS4CodesHalf, iters, cus, out, cycles);
    run<true, 3>("bf6", "s4-codes n (E3M2)", kBf6CodesOne, iters, cus, out, cycles);
    run<true, 3>("bf6", "s4-codes n/16 (E3M2)", kBf6CodesSixteenth, iters, cus, out, cycles);
    run<false>("int8", "zeros-again", kZeros, iters, cus, out, cycles);
    return 0;
}
