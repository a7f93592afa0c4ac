// Correctness harness: counterpart of the reference's test/test_correctness.cu:30-80, with the
// comparison that file leaves commented out (:66-76) switched on.
//
//   correctness [--entry v21|v0|...|c] [--dist uniform|normal] [--seed S] [--rows R] MxNxK ...
//
// For each shape: seeded operands -> pack() -> device -> linear_vN_launch (or the C ABI with
// --entry c) -> compare with the CPU reference GEMM, bit for bit.  With --rows R only R seeded
// rows of A (plus the first and last) are checked on the CPU, which keeps 8192^3 affordable.
// Exit status 0 iff every shape passed.
#include "harness_common.h"

// CPU reference GEMM and comparison from the test-side oracle library (plain C).
extern "C" void oracle_linear_ref_mt(const int *x, const int *w, int *y, int m, int n, int k, int threads);
extern "C" int oracle_is_same(const int *a, const int *b, int count);

using namespace harness;

namespace {

typedef void (*launch_fn)(void *, void *, void *, int, int, int);

void launch_c_abi(void *x, void *w, void *y, int m, int n, int k)
{
    const int st = int4linear_gemm_s4s4s32(x, w, y, m, n, k, nullptr);
    if (st != INT4LINEAR_OK) {
        std::fprintf(stderr, "int4linear_gemm_s4s4s32: %s\n", int4linear_status_string(st));
        std::exit(2);
    }
    HIP_OK(hipDeviceSynchronize());
}

launch_fn entry_by_name(const std::string &name)
{
    if (name == "v0") return linear_v0_launch;
    if (name == "v1") return linear_v1_launch;
    if (name == "v2") return linear_v2_launch;
    if (name == "v10") return linear_v10_launch;
    if (name == "v11") return linear_v11_launch;
    if (name == "v20") return linear_v20_launch;
    if (name == "v21") return linear_v21_launch;
    if (name == "c") return launch_c_abi;
    return nullptr;
}

bool run_shape(const Shape &s, launch_fn launch, bool normal_x, uint64_t seed, int sample_rows, int threads)
{
    const int m = s.m, n = s.n, k = s.k;
    const std::vector<int> x = normal_x ? normal_s4(seed, (size_t)m * k) : uniform_s4(seed, (size_t)m * k);
    const std::vector<int> w = uniform_s4(seed + 1, (size_t)n * k);
    const size_t packed_k = (size_t)(k + 7) / 8;
    DeviceBuffer xd(m * packed_k * sizeof(int)), wd(n * packed_k * sizeof(int)), yd((size_t)m * n * sizeof(int));
    upload_packed(x, m, k, xd);
    upload_packed(w, n, k, wd);
    HIP_OK(hipMemset(yd.p, 0x5A, yd.bytes));  // stale contents must not survive

    launch(xd.p, wd.p, yd.p, m, n, k);

    std::vector<int> y((size_t)m * n);
    HIP_OK(hipMemcpy(y.data(), yd.p, yd.bytes, hipMemcpyDeviceToHost));

    // rows to check on the CPU
    std::vector<int> rows;
    if (sample_rows <= 0 || sample_rows >= m) {
        for (int i = 0; i < m; ++i) rows.push_back(i);
    } else {
        Rng r(seed ^ 0xABCDEFull);
        rows = {0, m - 1};
        while ((int)rows.size() < sample_rows) rows.push_back((int)(r.next() % (uint64_t)m));
        std::sort(rows.begin(), rows.end());
        rows.erase(std::unique(rows.begin(), rows.end()), rows.end());
    }
    std::vector<int> xs(rows.size() * (size_t)k), want(rows.size() * (size_t)n), got(rows.size() * (size_t)n);
    for (size_t r = 0; r < rows.size(); ++r) {
        std::memcpy(&xs[r * k], &x[(size_t)rows[r] * k], (size_t)k * sizeof(int));
        std::memcpy(&got[r * n], &y[(size_t)rows[r] * n], (size_t)n * sizeof(int));
    }
    oracle_linear_ref_mt(xs.data(), w.data(), want.data(), (int)rows.size(), n, k, threads);
    const bool ok = oracle_is_same(want.data(), got.data(), (int)want.size()) != 0;
    std::printf("[%dx%dx%d] kernel=%s rows_checked=%zu %s\n", m, n, k, int4linear_kernel_for_shape(m, n, k),
                rows.size(), ok ? "TEST PASSED!" : "TEST FAILED!");
    if (!ok) {
        for (size_t i = 0; i < want.size(); ++i)
            if (want[i] != got[i]) {
                std::printf("  first mismatch: row %d col %zu: got %d want %d\n", rows[i / n], i % n, got[i], want[i]);
                break;
            }
    }
    return ok;
}

}  // namespace

int main(int argc, char **argv)
{
    std::string entry = "v21", dist = "uniform";
    uint64_t seed = 1;
    int sample_rows = 0, threads = 8;
    std::vector<Shape> shapes;
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        Shape s;
        if (a == "--entry" && i + 1 < argc) entry = argv[++i];
        else if (a == "--dist" && i + 1 < argc) dist = argv[++i];
        else if (a == "--seed" && i + 1 < argc) seed = std::strtoull(argv[++i], nullptr, 10);
        else if (a == "--rows" && i + 1 < argc) sample_rows = std::atoi(argv[++i]);
        else if (a == "--threads" && i + 1 < argc) threads = std::atoi(argv[++i]);
        else if (parse_shape(argv[i], s)) shapes.push_back(s);
        else {
            std::fprintf(stderr, "usage: %s [--entry v21|v20|v11|v10|v2|v1|v0|c] [--dist uniform|normal] "
                                 "[--seed S] [--rows R] [--threads T] MxNxK ...\n", argv[0]);
            return 2;
        }
    }
    launch_fn launch = entry_by_name(entry);
    if (!launch || (dist != "uniform" && dist != "normal")) {
        std::fprintf(stderr, "unknown --entry or --dist\n");
        return 2;
    }
    if (shapes.empty()) shapes.push_back({1024, 1024, 1024});
    bool all = true;
    for (const Shape &s : shapes)
        all = run_shape(s, launch, dist == "normal", seed, sample_rows, threads) && all;
    return all ? 0 : 1;
}
