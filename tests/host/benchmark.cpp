// Benchmark harness: counterpart of the reference's test/benchmark.cu:71-115 -- 5 warm-up
// launches, 50 timed ones, every timed launch preceded by a cache-cleaning fill and bracketed
// by its own event pair, median reported as 2*M*N*K / t in TOPS ("[PERF] ... TOPS").
//
//   benchmark [--kernel auto|simple|mfma|mfma128|mfma256|skinny|fp6] [--epilogue none|bias|f32|f16|bf16]
//             [--entry v0|v1|v2|v10|v11|v20|v21] [--iters I] [--warmup W] [--no-flush] MxNxK ...
//
// --entry times one of the reference's blocking linear_vN_launch entry points instead (each a
// step of this library's kernel history, kernels/linear_v0.h:168 ... linear_v21.h:760): wall
// time of the call between two device synchronisations, which is what the reference's own
// callers see (kernels/linear_v21.cu:37-39), and under rocprofv3 --kernel-trace the kernels of
// that step.
//
// --epilogue bias times int4linear_linear_s32 (bias add fused into the store), f32 times
// int4linear_linear_f32 (bias, per-row and per-column scales, float output), f16 / bf16 the
// same with a half-width output.
//
// The reference cleans twice its L2 (benchmark.cu:77-91); an MI355X also has a 256 MiB
// memory-side cache behind the eight L2s, so the fill here is 512 MiB.  Operand values are
// seeded uniform s4; the harness goes through the asynchronous C ABI so that the events
// bracket the library's device work only.
#include "harness_common.h"

using namespace harness;

namespace {

int kernel_id(const std::string &name)
{
    if (name == "auto") return INT4LINEAR_KERNEL_AUTO;
    if (name == "simple") return INT4LINEAR_KERNEL_SIMPLE;
    if (name == "mfma") return INT4LINEAR_KERNEL_MFMA;
    if (name == "skinny") return INT4LINEAR_KERNEL_SKINNY;
    if (name == "fp6") return INT4LINEAR_KERNEL_FP6;
    if (name == "mfma128") return INT4LINEAR_KERNEL_MFMA_128;
    if (name == "mfma256") return INT4LINEAR_KERNEL_MFMA_256;
    return -1;
}

}  // namespace

int main(int argc, char **argv)
{
    std::string kernel = "auto", epilogue = "none", entry;
    int iters = 50, warmup = 5;
    bool flush = true;
    std::vector<Shape> shapes;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        Shape s;
        if (a == "--kernel" && i + 1 < argc) kernel = argv[++i];
        else if (a == "--epilogue" && i + 1 < argc) epilogue = argv[++i];
        else if (a == "--entry" && i + 1 < argc) entry = argv[++i];
        else if (a == "--iters" && i + 1 < argc) iters = std::atoi(argv[++i]);
        else if (a == "--warmup" && i + 1 < argc) warmup = std::atoi(argv[++i]);
        else if (a == "--no-flush") flush = false;
        else if (parse_shape(argv[i], s)) shapes.push_back(s);
        else {
            std::fprintf(stderr, "usage: %s [--kernel auto|simple|mfma|mfma128|mfma256|skinny|fp6] [--iters I] [--warmup W] "
                                 "[--no-flush] MxNxK ...\n", argv[0]);
            return 2;
        }
    }
    using Launcher = void (*)(void *, void *, void *, int, int, int);
    Launcher entry_fn = nullptr;
    if (!entry.empty()) {
        if (entry == "v0") entry_fn = linear_v0_launch;
        else if (entry == "v1") entry_fn = linear_v1_launch;
        else if (entry == "v2") entry_fn = linear_v2_launch;
        else if (entry == "v10") entry_fn = linear_v10_launch;
        else if (entry == "v11") entry_fn = linear_v11_launch;
        else if (entry == "v20") entry_fn = linear_v20_launch;
        else if (entry == "v21") entry_fn = linear_v21_launch;
        else {
            std::fprintf(stderr, "bad --entry\n");
            return 2;
        }
    }
    const int kid = kernel_id(kernel);
    if (kid < 0 || iters < 1 || (epilogue != "none" && epilogue != "bias" && epilogue != "f32" && epilogue != "f16" && epilogue != "bf16")) {
        std::fprintf(stderr, "bad --kernel, --epilogue or --iters\n");
        return 2;
    }
    if (shapes.empty()) shapes.push_back({8192, 8192, 8192});

    const size_t fill_bytes = 512ull << 20;
    DeviceBuffer fill(flush ? fill_bytes : 16);
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));

    for (const Shape &s : shapes) {
        const int m = s.m, n = s.n, k = s.k;
        const size_t packed_k = (size_t)(k + 7) / 8;
        DeviceBuffer xd(m * packed_k * sizeof(int)), wd(n * packed_k * sizeof(int)), yd((size_t)m * n * sizeof(int));
        upload_packed(uniform_s4(11, (size_t)m * k), m, k, xd);
        upload_packed(uniform_s4(12, (size_t)n * k), n, k, wd);

        DeviceBuffer bias((size_t)n * sizeof(int)), rscale((size_t)m * sizeof(float)), cscale((size_t)n * sizeof(float));
        {
            std::vector<int> b((size_t)n);
            std::vector<float> r((size_t)m), c((size_t)n);
            Rng rng(13);
            for (auto &v : b) v = (int)(rng.next() % 2001) - 1000;
            for (auto &v : r) v = (float)(0.01 + rng.unit());
            for (auto &v : c) v = (float)(0.01 + rng.unit());
            HIP_OK(hipMemcpy(bias.p, b.data(), bias.bytes, hipMemcpyHostToDevice));
            HIP_OK(hipMemcpy(rscale.p, r.data(), rscale.bytes, hipMemcpyHostToDevice));
            HIP_OK(hipMemcpy(cscale.p, c.data(), cscale.bytes, hipMemcpyHostToDevice));
        }
        auto launch = [&]() {
            if (entry_fn) {
                entry_fn(xd.p, wd.p, yd.p, m, n, k);  // blocks until the device is done
                return;
            }
            int st;
            if (epilogue == "bias")
                st = int4linear_linear_s32(xd.p, wd.p, (const int *)bias.p, yd.p, m, n, k, kid, nullptr);
            else if (epilogue == "f32")
                st = int4linear_linear_f32(xd.p, wd.p, (const int *)bias.p, (const float *)rscale.p,
                                           (const float *)cscale.p, (float *)yd.p, m, n, k, kid, nullptr);
            else if (epilogue == "f16")
                st = int4linear_linear_f16(xd.p, wd.p, (const int *)bias.p, (const float *)rscale.p,
                                           (const float *)cscale.p, yd.p, m, n, k, kid, nullptr);
            else if (epilogue == "bf16")
                st = int4linear_linear_bf16(xd.p, wd.p, (const int *)bias.p, (const float *)rscale.p,
                                            (const float *)cscale.p, yd.p, m, n, k, kid, nullptr);
            else
                st = int4linear_gemm_s4s4s32_ex(xd.p, wd.p, yd.p, m, n, k, kid, nullptr);
            if (st != INT4LINEAR_OK) {
                std::fprintf(stderr, "[%dx%dx%d] %s\n", m, n, k, int4linear_status_string(st));
                std::exit(2);
            }
        };
        for (int i = 0; i < warmup; ++i) {
            launch();
            HIP_OK(hipDeviceSynchronize());
        }
        std::vector<float> ms((size_t)iters);
        for (int i = 0; i < iters; ++i) {
            if (flush)
                HIP_OK(hipMemsetAsync(fill.p, i & 0xFF, fill_bytes, nullptr));
            HIP_OK(hipDeviceSynchronize());
            HIP_OK(hipEventRecord(start, nullptr));
            launch();
            HIP_OK(hipEventRecord(stop, nullptr));
            HIP_OK(hipEventSynchronize(stop));
            HIP_OK(hipEventElapsedTime(&ms[i], start, stop));
        }
        std::sort(ms.begin(), ms.end());
        const double median_ms = ms[(size_t)iters / 2];
        const double ops = 2.0 * m * (double)n * k;
        const double bytes = (double)m * k / 2 + (double)n * k / 2 + 4.0 * m * n;
        std::printf("[PERF] %dx%dx%d kernel=%s epilogue=%s median %.4f ms (min %.4f)  %lf TOPS  %.1f GB/s\n", m, n, k,
                    entry_fn ? ("linear_" + entry + "_launch").c_str()
                    : kid == INT4LINEAR_KERNEL_AUTO ? int4linear_kernel_for_shape(m, n, k) : kernel.c_str(),
                    epilogue.c_str(), median_ms, (double)ms[0], ops / (median_ms * 1e9), bytes / (median_ms * 1e6));
    }
    HIP_OK(hipEventDestroy(start));
    HIP_OK(hipEventDestroy(stop));
    return 0;
}
