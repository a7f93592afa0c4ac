// Where the time of the FP6 GEMM kernel goes: the library's own kernel source compiled here
// with variations of its WholeKernel description that leave single parts out, every build timed
// on the same converted operands.  What remains without stores, without global -> LDS loads and
// without LDS reads is the MFMA loop with its barrier; each part's cost is the difference.  The
// builds with parts left out compute nothing useful and their output is never looked at.  One
// more build keeps everything and records when every workgroup starts and ends, which gives the
// spread of the ends and what the staggered start costs.
//
//   fp6_ablation [MxNxK] [--iters I] [--warmup W]       (default 8192x8192x8192, 40, 20)
//
// prints one line per build:  [ABLATION] <build> <us per launch> us <TOPS> TOPS
// and one [SPREAD] line.  Run it under  rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE
// for the clock and the share of cycles the matrix pipes are busy (the kernels differ in their
// last template argument).
#include "../../int4linear_amd/csrc/kernels_fp6.hip"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

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

using int4linear::WholeKernel;
struct SameTile : WholeKernel { static constexpr bool kOwnTile = false; };
struct NoStores : WholeKernel { static constexpr bool kStores = false; };
struct NoLdsReads : WholeKernel { static constexpr bool kLdsReads = false; };
struct NoLoads : WholeKernel { static constexpr bool kLoads = false; };
struct NoLoadsNoReads : NoLoads { static constexpr bool kLdsReads = false; };
struct MfmaLoop : NoLoadsNoReads { static constexpr bool kStores = false; };            // MFMAs, barrier, loop
struct MfmaLoopNoStagger : MfmaLoop { static constexpr bool kStagger = false; };
struct MfmaLoopNoFences : MfmaLoop { static constexpr bool kFences = false; };
struct MfmaLoopBare : MfmaLoop { static constexpr bool kStagger = false, kFences = false; };
struct NoStagger : WholeKernel { static constexpr bool kStagger = false; };
struct NoFences : WholeKernel { static constexpr bool kFences = false; };
// The whole kernel with time stamps: the epilogue's bias pointer (unused: the launch passes an
// epilogue that the kernel takes for "plain" only because `out` is 0 and the scales are null)
// cannot carry them, so they go to a global the harness reads back.
__device__ unsigned long long g_stamps[2][1024];
struct Stamped : WholeKernel {
    __device__ static void stamp(const int4linear::Epilogue &, int workgroup, int which) { g_stamps[which][workgroup & 1023] = wall_clock64(); }
};
struct StampedNoStagger : Stamped { static constexpr bool kStagger = false; };
struct StampedMfmaLoop : StampedNoStagger { static constexpr bool kLoads = false, kLdsReads = false, kStores = false; };

template <class Parts>
double time_build(const uint8_t *xw, const uint8_t *ww, int32_t *y, int m, int n, int k, int cus, int iters, int warmup)
{
    using namespace int4linear;
    using C = Fp6Cfg;
    auto kern = fp6_gemm_kernel<C, false, Parts>;
    CHECK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
    const int tiles_m = (m + kTileRows - 1) / kTileRows, tiles_n = (n + kTileRows - 1) / kTileRows;
    long grid = (long)cus * C::OCC;
    if (grid > (long)tiles_m * tiles_n)
        grid = (long)tiles_m * tiles_n;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < warmup; ++i)
        kern<<<(unsigned)grid, C::THREADS, kLdsBytes, 0>>>(xw, ww, y, m, n, padded_k(k), tiles_m, tiles_n, 1, Epilogue{});
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < iters; ++i)
        kern<<<(unsigned)grid, C::THREADS, kLdsBytes, 0>>>(xw, ww, y, m, n, padded_k(k), tiles_m, tiles_n, 1, Epilogue{});
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipDeviceSynchronize());
    CHECK(hipGetLastError());
    float ms = 0.f;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return (double)ms * 1e3 / iters;
}

// Start and end of every workgroup of the last launch, from the constant 100 MHz clock.
void report_spread(const char *name, int workgroups)
{
    static unsigned long long h[2][1024];
    CHECK(hipMemcpyFromSymbol(h, HIP_SYMBOL(g_stamps), sizeof h));
    if (workgroups > 1024)
        workgroups = 1024;
    unsigned long long s0 = ~0ull, s1 = 0, e0 = ~0ull, e1 = 0;
    for (int i = 0; i < workgroups; ++i) {
        s0 = h[0][i] < s0 ? h[0][i] : s0;
        s1 = h[0][i] > s1 ? h[0][i] : s1;
        e0 = h[1][i] < e0 ? h[1][i] : e0;
        e1 = h[1][i] > e1 ? h[1][i] : e1;
    }
    // workgroup ids go round the eight XCDs: the ends per XCD show whether the spread is between XCDs or inside them
    for (int x = 0; x < 8 && x < workgroups; ++x) {
        unsigned long long lo = ~0ull, hi = 0, sum = 0;
        int cnt = 0;
        for (int i = x; i < workgroups; i += 8, ++cnt) {
            lo = h[1][i] < lo ? h[1][i] : lo;
            hi = h[1][i] > hi ? h[1][i] : hi;
            sum += h[1][i] - s0;
        }
        std::printf("[SPREAD-XCD] %-18s xcd %d: ends %7.2f .. %7.2f us after the first start (mean %7.2f)\n", name, x, (double)(lo - s0) / 100.0,
                    (double)(hi - s0) / 100.0, (double)sum / cnt / 100.0);
    }
    std::printf("[SPREAD] %-22s first start to last start %6.2f us, first end to last end %6.2f us, first start to last end %7.2f us\n", name,
                (double)(s1 - s0) / 100.0, (double)(e1 - e0) / 100.0, (double)(e1 - s0) / 100.0);
    std::fflush(stdout);
}

}  // namespace

int main(int argc, char **argv)
{
    using namespace int4linear;
    int m = 8192, n = 8192, k = 8192, iters = 40, warmup = 20;
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
    if (m < 256 || n < 256 || k < 512 || k % 128 != 0 || !fp6_supports(m, n, k) || iters < 1 || warmup < 0) {
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

    uint8_t *a, *b, *xw, *ww;
    int32_t *y;
    const size_t abytes = (size_t)m * k / 2, bbytes = (size_t)n * k / 2;
    CHECK(hipMalloc(&a, abytes));
    CHECK(hipMalloc(&b, bbytes));
    CHECK(hipMalloc(&xw, fp6_operand_bytes(m, k)));
    CHECK(hipMalloc(&ww, fp6_operand_bytes(n, k)));
    CHECK(hipMalloc(&y, (size_t)m * n * 4));
    fill_kernel<<<1024, 256>>>((uint32_t *)a, abytes / 4, 1u);
    fill_kernel<<<1024, 256>>>((uint32_t *)b, bbytes / 4, 2u);
    CHECK(launch_fp6_convert(a, xw, m, k, 0));
    CHECK(launch_fp6_convert(b, ww, n, k, 0));
    CHECK(hipDeviceSynchronize());

    const double ops = 2.0 * m * n * k;
    auto report = [&](const char *name, double us) {
        std::printf("[ABLATION] %-46s %8.1f us  %7.1f TOPS\n", name, us, ops / us / 1e6);
        std::fflush(stdout);
    };
    // a load on the device before the first timed build, so that all of them meet the same clocks
    time_build<WholeKernel>(xw, ww, y, m, n, k, cus, iters, warmup);
    report("whole kernel", time_build<WholeKernel>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("every tile reads tile (0, 0)", time_build<SameTile>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("no stores", time_build<NoStores>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("no LDS reads", time_build<NoLdsReads>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("no global -> LDS loads", time_build<NoLoads>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("no loads, no LDS reads", time_build<NoLoadsNoReads>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("no staggered start", time_build<NoStagger>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("no scheduling fences", time_build<NoFences>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("MFMA loop (no loads, LDS reads, stores)", time_build<MfmaLoop>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("MFMA loop, no staggered start", time_build<MfmaLoopNoStagger>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("MFMA loop, no scheduling fences", time_build<MfmaLoopNoFences>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("MFMA loop, neither", time_build<MfmaLoopBare>(xw, ww, y, m, n, k, cus, iters, warmup));
    report("whole kernel again", time_build<WholeKernel>(xw, ww, y, m, n, k, cus, iters, warmup));
    const int tiles = ((m + kTileRows - 1) / kTileRows) * ((n + kTileRows - 1) / kTileRows);
    report("whole kernel with time stamps", time_build<Stamped>(xw, ww, y, m, n, k, cus, iters, warmup));
    report_spread("staggered start", tiles < cus ? tiles : cus);
    report("no staggered start, with time stamps", time_build<StampedNoStagger>(xw, ww, y, m, n, k, cus, iters, warmup));
    report_spread("all at once", tiles < cus ? tiles : cus);
    report("MFMA loop, no staggered start, with time stamps", time_build<StampedMfmaLoop>(xw, ww, y, m, n, k, cus, iters, warmup));
    report_spread("MFMA loop", tiles < cus ? tiles : cus);
    return 0;
}
