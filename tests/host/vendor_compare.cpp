// Vendor comparison: counterpart of the reference's test/cutlass_benchmark.cu (which times
// CUTLASS's s4 tensor-op GEMM next to the hand-written kernel).  The vendor library on an
// MI355X is hipBLASLt, which has no 4-bit integer GEMM; its closest path is int8 x int8 ->
// int32, so the packed s4 operands are first widened to int8 on the device (one-off, not
// timed) and the same C = A * B^T is run through hipblasLtMatmul.  The result is compared
// bit for bit with this library's, then both are timed with the benchmark harness's
// protocol (5 warm-ups, 50 iterations, cache-cleaning fill, per-launch events, median).
//
//   vendor_compare [--iters I] [--warmup W] [--readme-sweep] MxNxK ...
//
// --readme-sweep adds the two shape families of the reference README's chart (README.md:57-62:
// M = N = K and 2M = 2N = K, 1024 ... 8192) and prints the results once more as one table.
#include <hipblaslt/hipblaslt.h>

#include "harness_common.h"

using namespace harness;

#define BLT_OK(expr)                                                                        \
    do {                                                                                    \
        hipblasStatus_t s_ = (expr);                                                        \
        if (s_ != HIPBLAS_STATUS_SUCCESS) {                                                 \
            std::fprintf(stderr, "%s:%d: %s -> status %d\n", __FILE__, __LINE__, #expr, (int)s_); \
            std::exit(2);                                                                   \
        }                                                                                   \
    } while (0)

// One byte of two nibbles -> two sign-extended int8 values.
__global__ void widen_s4_to_s8(const uint8_t *__restrict__ src, int8_t *__restrict__ dst, size_t bytes)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= bytes)
        return;
    const int b = src[i];
    dst[2 * i] = (int8_t)((int8_t)(b << 4) >> 4);
    dst[2 * i + 1] = (int8_t)((int8_t)(b & 0xF0) >> 4);
}

__global__ void count_mismatches(const int *__restrict__ a, const int *__restrict__ b, size_t count,
                                 unsigned long long *out)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count && a[i] != b[i])
        atomicAdd(out, 1ull);
}

template <class F>
double median_ms(F &&launch, int warmup, int iters, void *fill, size_t fill_bytes)
{
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));
    for (int i = 0; i < warmup; ++i) {
        launch();
        HIP_OK(hipDeviceSynchronize());
    }
    std::vector<float> ms((size_t)iters);
    for (int i = 0; i < iters; ++i) {
        HIP_OK(hipMemsetAsync(fill, i & 0xFF, fill_bytes, nullptr));
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipEventRecord(start, nullptr));
        launch();
        HIP_OK(hipEventRecord(stop, nullptr));
        HIP_OK(hipEventSynchronize(stop));
        HIP_OK(hipEventElapsedTime(&ms[i], start, stop));
    }
    HIP_OK(hipEventDestroy(start));
    HIP_OK(hipEventDestroy(stop));
    std::sort(ms.begin(), ms.end());
    return ms[(size_t)iters / 2];
}

int main(int argc, char **argv)
{
    int iters = 50, warmup = 5;
    bool table = false;
    std::vector<Shape> shapes;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        Shape s;
        if (a == "--iters" && i + 1 < argc) iters = std::atoi(argv[++i]);
        else if (a == "--warmup" && i + 1 < argc) warmup = std::atoi(argv[++i]);
        else if (a == "--readme-sweep") {
            // The two families of the reference README's chart (README.md:57-62): M = N = K and
            // 2M = 2N = K, custom kernel against the vendor library, as one table.
            table = true;
            for (int d : {1024, 2048, 4096, 8192}) shapes.push_back({d, d, d});
            for (int d : {1024, 2048, 4096, 8192}) shapes.push_back({d, d, 2 * d});
        } else if (parse_shape(argv[i], s)) shapes.push_back(s);
        else {
            std::fprintf(stderr, "usage: %s [--iters I] [--warmup W] [--readme-sweep] MxNxK ...\n", argv[0]);
            return 2;
        }
    }
    if (iters < 1)
        return 2;
    if (shapes.empty()) shapes.push_back({8192, 8192, 8192});

    hipblasLtHandle_t handle;
    BLT_OK(hipblasLtCreate(&handle));
    const size_t fill_bytes = 512ull << 20, ws_bytes = 128ull << 20;
    DeviceBuffer fill(fill_bytes), workspace(ws_bytes), mismatches(sizeof(unsigned long long));
    bool all_equal = true;
    std::vector<std::string> rows;

    for (const Shape &s : shapes) {
        const int m = s.m, n = s.n, k = s.k;
        if (k % 8 != 0 || m < 1 || n < 1 || k < 8) {
            std::fprintf(stderr, "[%dx%dx%d] skipped: needs positive sizes and K %% 8 == 0\n", m, n, k);
            continue;
        }
        const size_t packed_k = (size_t)k / 8;
        DeviceBuffer xd(m * packed_k * sizeof(int)), wd(n * packed_k * sizeof(int));
        DeviceBuffer y_lib((size_t)m * n * sizeof(int)), y_vendor((size_t)m * n * sizeof(int));
        DeviceBuffer x8((size_t)m * k), w8((size_t)n * k);
        upload_packed(uniform_s4(21, (size_t)m * k), m, k, xd);
        upload_packed(uniform_s4(22, (size_t)n * k), n, k, wd);
        widen_s4_to_s8<<<(unsigned)((xd.bytes + 255) / 256), 256>>>((const uint8_t *)xd.p, (int8_t *)x8.p, xd.bytes);
        widen_s4_to_s8<<<(unsigned)((wd.bytes + 255) / 256), 256>>>((const uint8_t *)wd.p, (int8_t *)w8.p, wd.bytes);
        HIP_OK(hipDeviceSynchronize());

        // Row-major C[m][n] = sum_l X[m][l] W[n][l] is, in the library's column-major terms,
        // C^T (n x m, ld n) = op_T(W as k x n, ld k) * op_N(X as k x m, ld k).
        hipblasLtMatmulDesc_t desc;
        BLT_OK(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32I, HIP_R_32I));
        const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
        BLT_OK(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)));
        BLT_OK(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)));
        hipblasLtMatrixLayout_t lw, lx, lc;
        BLT_OK(hipblasLtMatrixLayoutCreate(&lw, HIP_R_8I, k, n, k));
        BLT_OK(hipblasLtMatrixLayoutCreate(&lx, HIP_R_8I, k, m, k));
        BLT_OK(hipblasLtMatrixLayoutCreate(&lc, HIP_R_32I, n, m, n));
        hipblasLtMatmulPreference_t pref;
        BLT_OK(hipblasLtMatmulPreferenceCreate(&pref));
        BLT_OK(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws_bytes,
                                                     sizeof(ws_bytes)));
        hipblasLtMatmulHeuristicResult_t heur[4];
        int found = 0;
        const hipblasStatus_t hs = hipblasLtMatmulAlgoGetHeuristic(handle, desc, lw, lx, lc, lc, pref, 4, heur, &found);
        if (hs != HIPBLAS_STATUS_SUCCESS || found == 0) {
            std::printf("[VENDOR] %dx%dx%d hipBLASLt offers no int8 x int8 -> int32 kernel for this shape (status %d)\n",
                        m, n, k, (int)hs);
        } else {
            const int32_t alpha = 1, beta = 0;
            auto vendor = [&]() {
                BLT_OK(hipblasLtMatmul(handle, desc, &alpha, w8.p, lw, x8.p, lx, &beta, y_vendor.p, lc, y_vendor.p, lc,
                                       &heur[0].algo, workspace.p, ws_bytes, nullptr));
            };
            auto ours = [&]() {
                const int st = int4linear_gemm_s4s4s32(xd.p, wd.p, y_lib.p, m, n, k, nullptr);
                if (st != INT4LINEAR_OK) {
                    std::fprintf(stderr, "int4linear_gemm_s4s4s32: %s\n", int4linear_status_string(st));
                    std::exit(2);
                }
            };
            vendor();
            ours();
            HIP_OK(hipMemset(mismatches.p, 0, sizeof(unsigned long long)));
            const size_t count = (size_t)m * n;
            count_mismatches<<<(unsigned)((count + 255) / 256), 256>>>((const int *)y_lib.p, (const int *)y_vendor.p, count,
                                                                        (unsigned long long *)mismatches.p);
            unsigned long long bad = 0;
            HIP_OK(hipMemcpy(&bad, mismatches.p, sizeof(bad), hipMemcpyDeviceToHost));
            all_equal = all_equal && bad == 0;

            const double t_vendor = median_ms(vendor, warmup, iters, fill.p, fill_bytes);
            const double t_ours = median_ms(ours, warmup, iters, fill.p, fill_bytes);
            const double ops = 2.0 * m * (double)n * k;
            std::printf("[VENDOR] %dx%dx%d hipBLASLt int8 %.4f ms %.1f TOPS | int4linear (%s) %.4f ms %.1f TOPS | "
                        "ratio %.2fx | results %s\n",
                        m, n, k, t_vendor, ops / (t_vendor * 1e9), int4linear_kernel_for_shape(m, n, k), t_ours,
                        ops / (t_ours * 1e9), t_vendor / t_ours, bad == 0 ? "identical" : "DIFFER");
            char row[256];
            std::snprintf(row, sizeof(row), "| %d x %d x %d | %s | %.1f | %.0f | %.1f | %.0f | %.2fx | %s |", m, n, k,
                          int4linear_kernel_for_shape(m, n, k), t_ours * 1e3, ops / (t_ours * 1e9), t_vendor * 1e3,
                          ops / (t_vendor * 1e9), t_vendor / t_ours, bad == 0 ? "identical" : "DIFFER");
            rows.push_back(row);
        }
        BLT_OK(hipblasLtMatmulPreferenceDestroy(pref));
        BLT_OK(hipblasLtMatrixLayoutDestroy(lw));
        BLT_OK(hipblasLtMatrixLayoutDestroy(lx));
        BLT_OK(hipblasLtMatrixLayoutDestroy(lc));
        BLT_OK(hipblasLtMatmulDescDestroy(desc));
    }
    BLT_OK(hipblasLtDestroy(handle));
    if (table) {
        std::printf("\n| M x N x K | kernel | int4linear us | TOPS | hipBLASLt int8 us | TOPS | ratio | results |\n"
                    "|---|---|---|---|---|---|---|---|\n");
        for (const std::string &r : rows)
            std::printf("%s\n", r.c_str());
    }
    return all_equal ? 0 : 1;
}
