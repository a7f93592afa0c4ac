// What the device gives a kernel that only streams: for each MxNxK on the command line, one
// launch reads an N x K/2 byte weight matrix exactly as the library's decode kernel does (one
// workgroup per CU, each wave instruction eight rows x 128 bytes straight into LDS,
// non-temporal, everything issued before anything is waited for) and writes 4*M*N bytes; there
// is no arithmetic and no reduction.  Launches go out back to back over weight buffers that
// rotate through more memory than the caches hold, and the time per launch -- the kernel plus
// the device's fixed cost per launch -- is printed: the ceiling a decode figure can be read
// against.  The reference has no such program (its launcher has no decode path,
// kernels/linear_v21.cu:20-26); timing protocol after test/benchmark.cu:87-107, without the
// per-launch flush, which the rotation replaces.
//
//   stream_ceiling [--steps N] MxNxK ...
//   prints one line per shape:  [CEILING] MxNxK <us per launch> us <GB/s of algorithmic bytes>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define HIP_OK(expr)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (expr);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            std::fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            std::exit(2);                                                                             \
        }                                                                                             \
    } while (0)

namespace {

constexpr int kMaxLds = 160 * 1024;

// 16 bytes per lane from base + lane_off straight to LDS at lds_addr + 16 * lane.
__device__ __forceinline__ void dma16(const void *base, unsigned lane_off, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" : : "v"(lane_off), "s"(base), "s"(lds_addr) : "memory");
}

// A workgroup takes `rows_blk` rows of `rowbytes` bytes; wave w takes the 128-byte column
// tiles w, w + waves, ... of every row, sixteen rows (two instructions) at a time.  `loads`
// instructions per wave; LDS positions wrap, nobody reads them.
__global__ __launch_bounds__(1024) void stream_kernel(const uint8_t *__restrict__ W, int *__restrict__ Y, unsigned rowbytes,
                                                      int rows_blk, int n_rows, int tiles, int y_per_blk)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int row0 = blockIdx.x * rows_blk;
    const int rows = min(rows_blk, n_rows - row0);
    const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) void *)lds + wave * (kMaxLds / 16);
    const unsigned lrow = lane >> 3, chunk = (lane & 7) * 16;
    unsigned slot = 0;
    for (int g = 0; g < rows; g += 16)
        for (int t = wave; t < tiles; t += waves) {
            const uint8_t *base = W + ((size_t)row0 + g) * rowbytes + (size_t)t * 128;
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const unsigned r = min(lrow + 8 * u, (unsigned)(rows - g - 1));
                dma16(base, r * rowbytes + chunk, lds_base + (slot & 7) * 1024);
                ++slot;
            }
        }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): everything has landed
    const int v = *(const int *)(lds + lane * 4);
    for (int i = threadIdx.x; i < y_per_blk; i += blockDim.x)
        Y[(size_t)blockIdx.x * y_per_blk + i] = v;
}

}  // namespace

int main(int argc, char **argv)
{
    int steps = 300;
    std::vector<const char *> shapes;
    for (int i = 1; i < argc; ++i) {
        if (!std::strcmp(argv[i], "--steps") && i + 1 < argc)
            steps = std::atoi(argv[++i]);
        else
            shapes.push_back(argv[i]);
    }
    if (shapes.empty() || steps < 1) {
        std::fprintf(stderr, "usage: stream_ceiling [--steps N] MxNxK ...\n");
        return 2;
    }
    struct Shape { int m, n, k; };
    std::vector<Shape> parsed;
    for (const char *s : shapes) {
        Shape sh{};
        if (std::sscanf(s, "%dx%dx%d", &sh.m, &sh.n, &sh.k) != 3 || sh.m < 1 || sh.n < 1 || sh.k < 256 || sh.k % 256 != 0) {
            std::fprintf(stderr, "bad shape '%s' (MxNxK, K a multiple of 256)\n", s);
            return 2;
        }
        parsed.push_back(sh);
    }
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    HIP_OK(hipFuncSetAttribute((const void *)stream_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kMaxLds));
    const size_t pool = (size_t)1 << 30;  // the weight buffers rotate through 1 GiB
    uint8_t *w = nullptr;
    HIP_OK(hipMalloc(&w, pool));
    HIP_OK(hipMemset(w, 0x5a, pool));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    for (const Shape &sh : parsed) {
        const size_t wbytes = (size_t)sh.n * (size_t)(sh.k / 2);
        if (wbytes > pool) {
            std::fprintf(stderr, "%dx%dx%d: weights larger than the 1 GiB pool\n", sh.m, sh.n, sh.k);
            return 2;
        }
        const int nbuf = (int)(pool / wbytes);
        // rows per workgroup as the decode kernel splits them: evenly over the CUs, in steps of 8
        const int rows_blk = (int)(((sh.n + cus - 1) / cus + 7) / 8 * 8);
        const int grid = (sh.n + rows_blk - 1) / rows_blk;
        const int tiles = sh.k / 256;
        const int waves = tiles < 16 ? tiles : 16;
        const int y_per_blk = (int)(((size_t)sh.m * sh.n + grid - 1) / grid);
        int *y = nullptr;
        HIP_OK(hipMalloc(&y, (size_t)y_per_blk * grid * 4));
        auto launch = [&](int i) {
            stream_kernel<<<grid, waves * 64, kMaxLds>>>(w + (size_t)(i % nbuf) * wbytes, y, (unsigned)(sh.k / 2), rows_blk, sh.n, tiles,
                                                        y_per_blk);
        };
        for (int i = 0; i < nbuf + 20; ++i)
            launch(i);
        HIP_OK(hipDeviceSynchronize());
        float best = 1e30f;
        for (int rep = 0; rep < 3; ++rep) {
            HIP_OK(hipEventRecord(e0));
            for (int i = 0; i < steps; ++i)
                launch(i);
            HIP_OK(hipEventRecord(e1));
            HIP_OK(hipEventSynchronize(e1));
            float ms = 0;
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            if (ms / steps < best)
                best = ms / steps;
        }
        HIP_OK(hipGetLastError());
        const double bytes = (double)sh.m * sh.k / 2 + (double)wbytes + 4.0 * sh.m * sh.n;
        std::printf("[CEILING] %dx%dx%d %.3f us %.1f GB/s\n", sh.m, sh.n, sh.k, best * 1e3, bytes / (best * 1e-3) / 1e9);
        std::fflush(stdout);
        HIP_OK(hipFree(y));
    }
    return 0;
}
