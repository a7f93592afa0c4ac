// Where the time of the int8 GEMM kernel (mfma_gemm_kernel, 256 x 256 tiles) goes: the
// library's own kernel source compiled here with variations of its WholeInt8Kernel description
// that leave single parts out, every build timed on the same packed operands.  The builds with
// parts left out compute nothing useful and their output is never looked at.
//
//   int8_ablation [MxNxK] [--iters I] [--warmup W]       (default 8192x8192x8192, 30, 15)
//
// prints one line per build:  [ABLATION] <build> <us per launch> us <TOPS> TOPS
// and, for two builds with time stamps, when the workgroups of every XCD end ([SPREAD-XCD]).
// Run it under  rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE  for the clock and the
// share of cycles the matrix pipes are busy (the kernels differ in their last template
// argument).
#include "../../int4linear_amd/csrc/kernels_mfma.hip"

#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace {

#define CHECK(x)                                                                         \
    do {                                                                                 \
        hipError_t e_ = (x);                                                             \
        if (e_ != hipSuccess) {                                                          \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            std::exit(1);                                                                \
        }                                                                                \
    } while (0)

__global__ void fill_kernel(uint32_t *p, size_t n, uint32_t seed)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t x = (uint32_t)i * 2654435761u + seed;
        x ^= x >> 15;
        x *= 2246822519u;
        x ^= x >> 13;
        x *= 3266489917u;
        x ^= x >> 16;
        p[i] = x;  // every nibble uniform in [-8, 7]
    }
}

using int4linear::WholeInt8Kernel;
struct NoStores : WholeInt8Kernel { static constexpr bool kStores = false; };
struct NoLdsReads : WholeInt8Kernel { static constexpr bool kLdsReads = false; };
struct NoLoads : WholeInt8Kernel { static constexpr bool kLoads = false; };
struct NoWiden : WholeInt8Kernel { static constexpr bool kWiden = false; };
struct NoStagger : WholeInt8Kernel { static constexpr bool kStagger = false; };
struct NoLoadsNoReads : NoLoads { static constexpr bool kLdsReads = false; };
struct WidenAndMfma : NoLoadsNoReads { static constexpr bool kStores = false; };   // widening, MFMAs, barrier, loop
struct MfmaLoop : WidenAndMfma { static constexpr bool kWiden = false; };           // MFMAs, barrier, loop
struct MfmaLoopNoStagger : MfmaLoop { static constexpr bool kStagger = false; };
// Builds that record when every workgroup starts and ends (the constant 100 MHz clock).
__device__ unsigned long long g_stamps[2][1024];
struct Stamped : WholeInt8Kernel {
    __device__ static void stamp(int workgroup, int which) { g_stamps[which][workgroup & 1023] = wall_clock64(); }
};
struct StampedMfmaLoop : Stamped { static constexpr bool kLoads = false, kLdsReads = false, kStores = false, kWiden = false, kStagger = false; };

template <class Parts>
double time_build(const uint8_t *a, const uint8_t *b, int32_t *y, int m, int n, int k, int cus, int iters, int warmup)
{
    using namespace int4linear;
    using C = CfgLarge;
    auto kern = mfma_gemm_kernel<C, Parts>;
    CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES));
    const int tiles_m = (m + C::BM - 1) / C::BM, tiles_n = (n + C::BN - 1) / C::BN;
    long grid = (long)cus * C::OCC;
    if (grid > (long)tiles_m * tiles_n)
        grid = (long)tiles_m * tiles_n;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < warmup; ++i)
        kern<<<(unsigned)grid, C::THREADS, C::LDS_BYTES, 0>>>(a, b, y, m, n, k, tiles_m, tiles_n, 1, Epilogue{});
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < iters; ++i)
        kern<<<(unsigned)grid, C::THREADS, C::LDS_BYTES, 0>>>(a, b, y, m, n, k, tiles_m, tiles_n, 1, Epilogue{});
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipDeviceSynchronize());
    CHECK(hipGetLastError());
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return (double)ms * 1e3 / iters;
}

// Start and end of every workgroup of the last launch, per XCD (workgroup ids go round the eight XCDs).
void report_spread(const char *name, int workgroups)
{
    static unsigned long long h[2][1024];
    CHECK(hipMemcpyFromSymbol(h, HIP_SYMBOL(g_stamps), sizeof h));
    if (workgroups > 1024)
        workgroups = 1024;
    unsigned long long s0 = ~0ull, e0 = ~0ull, e1 = 0;
    for (int i = 0; i < workgroups; ++i) {
        s0 = h[0][i] < s0 ? h[0][i] : s0;
        e0 = h[1][i] < e0 ? h[1][i] : e0;
        e1 = h[1][i] > e1 ? h[1][i] : e1;
    }
    for (int x = 0; x < 8 && x < workgroups; ++x) {
        unsigned long long lo = ~0ull, hi = 0;
        for (int i = x; i < workgroups; i += 8) {
            lo = h[1][i] < lo ? h[1][i] : lo;
            hi = h[1][i] > hi ? h[1][i] : hi;
        }
        std::printf("[SPREAD-XCD] %-18s xcd %d: ends %7.2f .. %7.2f us after the first start\n", name, x, (double)(lo - s0) / 100.0,
                    (double)(hi - s0) / 100.0);
    }
    std::printf("[SPREAD] %-22s first end to last end %6.2f us, first start to last end %7.2f us\n", name, (double)(e1 - e0) / 100.0,
                (double)(e1 - s0) / 100.0);
    std::fflush(stdout);
}

}  // namespace

int main(int argc, char **argv)
{
    using namespace int4linear;
    int m = 8192, n = 8192, k = 8192, iters = 30, warmup = 15;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--iters") && i + 1 < argc) {
            iters = std::atoi(argv[++i]);
        } else if (!std::strcmp(argv[i], "--warmup") && i + 1 < argc) {
            warmup = std::atoi(argv[++i]);
        } else if (std::sscanf(argv[i], "%dx%dx%d", &m, &n, &k) != 3) {
            std::fprintf(stderr, "usage: %s [MxNxK] [--iters I] [--warmup W]\n", argv[0]);
            return 2;
        }
    }
    if (m < 256 || n < 256 || k < 512 || !mfma_supports(m, n, k) || iters < 1 || warmup < 0) {
        std::fprintf(stderr, "shape not accepted: at least 256 x 256 x 512, K a multiple of 128\n");
        return 2;
    }
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
        std::fprintf(stderr, "no GPU\n");
        return 3;
    }
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;

    uint8_t *a, *b;
    int32_t *y;
    const size_t abytes = (size_t)m * k / 2, bbytes = (size_t)n * k / 2;
    CHECK(hipMalloc(&a, abytes));
    CHECK(hipMalloc(&b, bbytes));
    CHECK(hipMalloc(&y, (size_t)m * n * 4));
    fill_kernel<<<1024, 256>>>((uint32_t *)a, abytes / 4, 1u);
    fill_kernel<<<1024, 256>>>((uint32_t *)b, bbytes / 4, 2u);
    CHECK(hipDeviceSynchronize());

    const double ops = 2.0 * m * n * k;
    auto report = [&](const char *name, double us) {
        std::printf("[ABLATION] %-46s %8.1f us  %7.1f TOPS\n", name, us, ops / us / 1e6);
        std::fflush(stdout);
    };
    // a load on the device before the first timed build, so that all of them meet the same clocks
    time_build<WholeInt8Kernel>(a, b, y, m, n, k, cus, iters, warmup);
    report("whole kernel", time_build<WholeInt8Kernel>(a, b, y, m, n, k, cus, iters, warmup));
    report("no stores", time_build<NoStores>(a, b, y, m, n, k, cus, iters, warmup));
    report("no LDS reads", time_build<NoLdsReads>(a, b, y, m, n, k, cus, iters, warmup));
    report("no global -> LDS loads", time_build<NoLoads>(a, b, y, m, n, k, cus, iters, warmup));
    report("no nibble widening", time_build<NoWiden>(a, b, y, m, n, k, cus, iters, warmup));
    report("no staggered start", time_build<NoStagger>(a, b, y, m, n, k, cus, iters, warmup));
    report("no loads, no LDS reads", time_build<NoLoadsNoReads>(a, b, y, m, n, k, cus, iters, warmup));
    report("widening and MFMAs only", time_build<WidenAndMfma>(a, b, y, m, n, k, cus, iters, warmup));
    report("MFMA loop (nothing else)", time_build<MfmaLoop>(a, b, y, m, n, k, cus, iters, warmup));
    report("MFMA loop, no staggered start", time_build<MfmaLoopNoStagger>(a, b, y, m, n, k, cus, iters, warmup));
    report("whole kernel again", time_build<WholeInt8Kernel>(a, b, y, m, n, k, cus, iters, warmup));
    const int tiles = ((m + CfgLarge::BM - 1) / CfgLarge::BM) * ((n + CfgLarge::BN - 1) / CfgLarge::BN);
    report("whole kernel with time stamps", time_build<Stamped>(a, b, y, m, n, k, cus, iters, warmup));
    report_spread("whole kernel", tiles < cus ? tiles : cus);
    report("MFMA loop, no staggered start, with time stamps", time_build<StampedMfmaLoop>(a, b, y, m, n, k, cus, iters, warmup));
    report_spread("MFMA loop", tiles < cus ? tiles : cus);
    return 0;
}
