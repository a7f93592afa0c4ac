// C ABI of libint4linear.so, shape dispatch, and the reference's C++-linkage shims.
#include "../../include/int4linear.h"
#include "kernels.h"

#include <atomic>
#include <cstdint>
#include <cstdio>
#include <mutex>

namespace {

using namespace int4linear;

constexpr int kMaxDevices = 64;

// Scratch memory of int4linear_gemm_s4s4s32_static: it stands where the other entry points
// use the workspace they allocate (the FP6 kernel's converted operands, the partial sums of
// the split-K forms).  One copy per device, at its own address on each, for as long as the
// process lives.  In host code the name below is only a handle for hipGetSymbolAddress, not
// a device address: ensure_init() asks for the address once per device and everything else
// uses PerDevice::scratch.
constexpr size_t kStaticScratchBytes = (size_t)INT4LINEAR_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// Arrival counters of the weight-streaming kernel's split over K (kernels.h): two sets, the
// first for calls that keep their partial sums in the internal workspace, the second for
// int4linear_gemm_s4s4s32_static.  Zero when the library is loaded; every launch leaves them
// zero again.
static __device__ __align__(256) unsigned arrivals[2][kSkinnyArrivalWords];

struct PerDevice {
    // Set-up happens once per device, under init_mutex; `ready` is set only when it has
    // succeeded, so a failure (a transient one included) is reported to the caller that
    // met it and tried again by the next call.
    std::mutex init_mutex;
    std::atomic<bool> ready{false};
    DeviceInfo info;
    void *scratch = nullptr;  // this device's copy of `scratch` (kStaticScratchBytes bytes)
    unsigned *arrivals = nullptr;  // this device's copy of `arrivals`
    // Workspace of the FP6 path: grown on demand up to g_workspace_limit, kept until
    // int4linear_release_workspace() or process exit.  `ws_event` marks the end of the
    // last GEMM that used it, so a call on another stream can wait for it.
    std::mutex ws_mutex;
    void *ws = nullptr;
    size_t ws_bytes = 0;
    hipEvent_t ws_event = nullptr;
    hipStream_t ws_stream = nullptr;
    bool ws_used = false;
};

std::atomic<size_t> g_workspace_limit{(size_t)1 << 30};

PerDevice g_devices[kMaxDevices];
thread_local int t_last_hip_error = 0;

int fail_hip(hipError_t e)
{
    t_last_hip_error = (int)e;
    return INT4LINEAR_ERR_HIP;
}

// True while `stream` records into a graph.  Allocating, freeing and recording events on
// other streams are all off limits then, and so is baking the internal workspace's address
// into a graph that may outlive it.  A query that fails counts as capturing.
bool stream_is_capturing(hipStream_t stream)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return status != hipStreamCaptureStatusNone;
}

hipError_t set_up_device(PerDevice &pd, int dev)
{
    hipDeviceProp_t prop;
    hipError_t err = hipGetDeviceProperties(&prop, dev);
    if (err != hipSuccess)
        return err;
    pd.info.cu_count = prop.multiProcessorCount;
    pd.info.lds_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
    err = mfma_init(pd.info);
    if (err == hipSuccess)
        err = fp6_init(pd.info);
    if (err == hipSuccess)
        err = skinny_init(pd.info);
    if (err == hipSuccess)  // `dev` is current here: the addresses are this device's copies
        err = hipGetSymbolAddress((void **)&pd.scratch, HIP_SYMBOL(scratch));
    if (err == hipSuccess)
        err = hipGetSymbolAddress((void **)&pd.arrivals, HIP_SYMBOL(arrivals));
    return err;
}

// Set-up for the device that is current on the calling thread; returns its record.  Set-up
// queries the device, raises the dynamic-LDS limit of some 250 kernels and takes the address
// of the scratch arrays (which loads the device image): none of that belongs inside a graph
// capture, so a first call that arrives with `work_stream` capturing is refused
// (`for_work`: the call is about to enqueue work on work_stream).
int ensure_init(PerDevice **out, bool for_work = false, hipStream_t work_stream = nullptr)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        t_last_hip_error = (int)e;
        return INT4LINEAR_ERR_NO_DEVICE;
    }
    if (dev < 0 || dev >= kMaxDevices)
        return INT4LINEAR_ERR_NO_DEVICE;
    PerDevice &pd = g_devices[dev];
    if (!pd.ready.load(std::memory_order_acquire)) {
        if (for_work && stream_is_capturing(work_stream))
            return INT4LINEAR_ERR_NOT_INITIALISED;
        std::lock_guard<std::mutex> lock(pd.init_mutex);
        if (!pd.ready.load(std::memory_order_relaxed)) {
            e = set_up_device(pd, dev);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return fail_hip(e);
            }
            pd.ready.store(true, std::memory_order_release);
        }
    }
    if (out)
        *out = &pd;
    return INT4LINEAR_OK;
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

// The FP6 path pays off once its 256 x 256 tiles can occupy a good part of the device and K
// is long enough to amortise the converter pass (a fixed cost of about (M + N) * K * 1.25
// bytes of HBM traffic).  Measured against the int8 kernel (tiles, K -> faster kernel):
// 128, 4096 -> tie; 128, 8192 -> FP6 by 8 %; 128, 14336 -> FP6 by 20 %; 144, 3072 -> FP6;
// 256, 2048 -> int8 by 5 %; 512, 2048 -> FP6 by 20 %; 512, 1024 -> FP6 by 3 %; 1024, 1024
// -> tie; 1024, 512 -> int8 by 10 %.  With 64 tiles or fewer the FP6 GEMM splits K, but the
// int8 kernel's small-grid form is as fast or faster there (64 tiles: 62 against 81 us at
// K = 14336, 122 against 131 and 115 against 109 us at K = 28672), so the automatic choice
// leaves those shapes to it.
bool fp6_worthwhile(int m, int n, int k, const DeviceInfo &dev, size_t limit)
{
    const long tiles = (long)((m + 255) / 256) * ((n + 255) / 256);
    const bool pays = (tiles >= 128 && k >= 8192) || (tiles >= 144 && k >= 3072) || (tiles >= 384 && k >= 1024);
    return pays && fp6_supports(m, n, k) && fp6_workspace_bytes(m, n, k, dev) <= limit;
}

// K that is not a multiple of 128 fits neither the int8 nor the weight-streaming kernel,
// but the FP6 converter pads K with zeros: beyond a few million multiply-adds that beats
// the scalar kernel by orders of magnitude even for a handful of rows.
bool fp6_for_ragged_k(int m, int n, int k, const DeviceInfo &dev, size_t limit)
{
    return (k % 128) != 0 && fp6_supports(m, n, k) && (double)m * n * k >= (double)(1 << 22) &&
           fp6_workspace_bytes(m, n, k, dev) <= limit;
}

// The current device's record, set up if it has not been yet; without a usable device an
// all-zero DeviceInfo (the shape-only answers of the queries below).
DeviceInfo current_device_info()
{
    PerDevice *pd = nullptr;
    if (ensure_init(&pd) != INT4LINEAR_OK || !pd)
        return DeviceInfo{};
    return pd->info;
}

// `limit`: the most workspace the chosen kernel may use.
int pick_kernel(int m, int n, int k, const DeviceInfo &dev, size_t limit)
{
    if (skinny_preferred(m, n, k, dev))
        return INT4LINEAR_KERNEL_SKINNY;
    if (fp6_worthwhile(m, n, k, dev, limit))
        return INT4LINEAR_KERNEL_FP6;
    if (mfma_supports(m, n, k))
        return INT4LINEAR_KERNEL_MFMA;
    if (fp6_for_ragged_k(m, n, k, dev, limit))
        return INT4LINEAR_KERNEL_FP6;
    return INT4LINEAR_KERNEL_SIMPLE;
}

// Where a call's workspace comes from.
enum class Workspace {
    Internal,  // the per-device buffer this library allocates and grows (acquire_workspace)
    Static,    // the file-scope `scratch` array: nothing is allocated, the size is fixed
    None       // none: only kernels that need no workspace
};

// Hands out the device's internal workspace with at least `need` bytes for work about to be
// enqueued on `stream` (the caller holds pd->ws_mutex until that work is enqueued).  Calls
// on one stream are ordered by the stream; a call on a different stream than the previous
// user first waits for everything the previous user's stream has been given so far.
int acquire_workspace(PerDevice *pd, size_t need, hipStream_t stream, void **out)
{
    if (need > g_workspace_limit.load())
        return INT4LINEAR_ERR_UNSUPPORTED;
    hipError_t e;
    if (!pd->ws_event) {
        e = hipEventCreateWithFlags(&pd->ws_event, hipEventDisableTiming);
        if (e != hipSuccess)
            return fail_hip(e);
    }
    if (pd->ws_bytes < need) {
        if (pd->ws) {
            e = hipFree(pd->ws);  // waits for the device to be done with it
            pd->ws = nullptr;
            pd->ws_bytes = 0;
            pd->ws_used = false;
            if (e != hipSuccess)
                return fail_hip(e);
        }
        e = hipMalloc(&pd->ws, need);
        if (e != hipSuccess) {
            pd->ws = nullptr;
            return fail_hip(e);
        }
        pd->ws_bytes = need;
    }
    if (pd->ws_used && pd->ws_stream != stream) {
        // The previous user ran on another stream: mark the point its stream has reached
        // now (which is after that user's kernels) and make this stream wait for it.
        // Recording here, only when the stream changes, keeps the common one-stream case
        // free of events.
        e = hipEventRecord(pd->ws_event, pd->ws_stream);
        if (e == hipSuccess) {
            e = hipStreamWaitEvent(stream, pd->ws_event, 0);
        } else {
            // The previous stream no longer exists (destroyed with work possibly still
            // draining): wait for the whole device instead.
            (void)hipGetLastError();
            e = hipDeviceSynchronize();
        }
        if (e != hipSuccess)
            return fail_hip(e);
    }
    pd->ws_stream = stream;
    pd->ws_used = true;
    *out = pd->ws;
    return INT4LINEAR_OK;
}

// The FP6 path: converted operands (and split-K slabs) in the internal workspace or in the
// static scratch array.  `capturing`: the stream records into a graph (Internal only).
int run_fp6(PerDevice *pd, const void *a, const void *b, void *c, int m, int n, int k,
            const Epilogue &ep, Workspace source, bool capturing, hipStream_t stream)
{
    const size_t need = fp6_workspace_bytes(m, n, k, pd->info);
    hipError_t e;
    if (source == Workspace::Static) {
        if (need > kStaticScratchBytes)
            return INT4LINEAR_ERR_SCRATCH;
        e = launch_fp6(a, b, c, m, n, k, pd->scratch, ep, pd->info, stream);
    } else {
        if (source == Workspace::None || capturing)
            return INT4LINEAR_ERR_UNSUPPORTED;
        std::lock_guard<std::mutex> lock(pd->ws_mutex);
        void *ws = nullptr;
        const int st = acquire_workspace(pd, need, stream, &ws);
        if (st != INT4LINEAR_OK)
            return st;
        e = launch_fp6(a, b, c, m, n, k, ws, ep, pd->info, stream);
    }
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

// The int8 kernel under automatic dispatch: split over K when that helps and the workspace
// for the partial sums can be had, otherwise the plain kernel.
int run_mfma_auto(PerDevice *pd, const void *a, const void *b, void *c, int m, int n, int k,
                  const Epilogue &ep, Workspace source, bool capturing, hipStream_t stream)
{
    const size_t need = mfma_workspace_bytes(m, n, k, pd->info);
    hipError_t e;
    if (need == 0 || source == Workspace::None || capturing ||
        (source == Workspace::Static && need > kStaticScratchBytes)) {
        e = launch_mfma(a, b, c, m, n, k, ep, pd->info, stream);
    } else if (source == Workspace::Static) {
        e = launch_mfma_splitk(a, b, c, m, n, k, pd->scratch, ep, pd->info, stream);
    } else {
        std::lock_guard<std::mutex> lock(pd->ws_mutex);
        void *ws = nullptr;
        if (acquire_workspace(pd, need, stream, &ws) != INT4LINEAR_OK)
            ws = nullptr;  // no workspace: the unsplit kernel
        e = launch_mfma_splitk(a, b, c, m, n, k, ws, ep, pd->info, stream);
    }
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

// The weight-streaming kernel under automatic dispatch: the shapes it splits over K across
// workgroups keep their partial sums in the workspace; without one they run unsplit.
int run_skinny_auto(PerDevice *pd, const void *a, const void *b, void *c, int m, int n, int k,
                    const Epilogue &ep, Workspace source, bool capturing, hipStream_t stream)
{
    const size_t need = skinny_workspace_bytes(m, n, k, pd->info);
    hipError_t e;
    if (need == 0 || source == Workspace::None || capturing ||
        (source == Workspace::Static && need > kStaticScratchBytes)) {
        e = launch_skinny(a, b, c, m, n, k, ep, pd->info, stream);
    } else if (source == Workspace::Static) {
        e = launch_skinny_ksplit(a, b, c, m, n, k, pd->scratch, pd->arrivals + kSkinnyArrivalWords, ep, pd->info, stream);
    } else {
        std::lock_guard<std::mutex> lock(pd->ws_mutex);
        void *ws = nullptr;
        if (acquire_workspace(pd, need, stream, &ws) == INT4LINEAR_OK)
            e = launch_skinny_ksplit(a, b, c, m, n, k, ws, pd->arrivals, ep, pd->info, stream);
        else
            e = launch_skinny(a, b, c, m, n, k, ep, pd->info, stream);
    }
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

int gemm_impl(const void *a, const void *b, void *c, int m, int n, int k, int kernel,
              void *stream_v, const Epilogue &ep = Epilogue{}, Workspace source = Workspace::Internal)
{
    if (m < 0 || n < 0 || k < 0 || (k % 8) != 0)
        return INT4LINEAR_ERR_SHAPE;
    if (kernel < INT4LINEAR_KERNEL_AUTO || kernel > INT4LINEAR_KERNEL_MFMA_256)
        return INT4LINEAR_ERR_UNSUPPORTED;
    if (m == 0 || n == 0)
        return INT4LINEAR_OK;
    if (!c)
        return INT4LINEAR_ERR_NULL;
    if (k > 0 && (!a || !b))
        return INT4LINEAR_ERR_NULL;
    if (!aligned16(c) || (k > 0 && (!aligned16(a) || !aligned16(b))))
        return INT4LINEAR_ERR_ALIGN;

    hipStream_t stream = (hipStream_t)stream_v;
    PerDevice *pd = nullptr;
    int st = ensure_init(&pd, true, stream);
    if (st != INT4LINEAR_OK)
        return st;

    const bool plain = !ep.bias && !ep.row_scale && !ep.col_scale && !ep.out;
    if (k == 0 && plain) {
        hipError_t e = launch_zero_i32((int *)c, (size_t)m * (size_t)n, stream);
        return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
    }
    if (k == 0) {  // empty sum with an epilogue: the scalar kernel's loop runs zero times
        hipError_t e = launch_simple(a, b, c, m, n, k, ep, stream);
        return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
    }

    const bool automatic = kernel == INT4LINEAR_KERNEL_AUTO;
    bool capturing = false;
    if (automatic) {
        const size_t limit = source == Workspace::Static ? kStaticScratchBytes : g_workspace_limit.load();
        kernel = pick_kernel(m, n, k, pd->info, limit);
        // A stream under capture gets the kernels that need no workspace.  Whether it is one
        // is asked only when the chosen kernel would touch the internal workspace or its
        // ordering between streams: decode calls with up to 32 rows, a few microseconds
        // long, never pay for the query.
        if (source == Workspace::Internal &&
            (kernel == INT4LINEAR_KERNEL_FP6 ||
             (kernel == INT4LINEAR_KERNEL_MFMA && limit > 0 && mfma_workspace_bytes(m, n, k, pd->info) > 0) ||
             (kernel == INT4LINEAR_KERNEL_SKINNY && limit > 0 && skinny_workspace_bytes(m, n, k, pd->info) > 0))) {
            capturing = stream_is_capturing(stream);
            if (capturing)
                kernel = pick_kernel(m, n, k, pd->info, 0);
        }
        // The static entry point falls back to the kernels without scratch memory when the
        // array is too small; it refuses only what would then be left to the scalar kernel
        // although a fast kernel exists for it (ragged K beyond the array's size).
        if (source == Workspace::Static && kernel == INT4LINEAR_KERNEL_SIMPLE &&
            pick_kernel(m, n, k, pd->info, SIZE_MAX) != INT4LINEAR_KERNEL_SIMPLE)
            return INT4LINEAR_ERR_SCRATCH;
    } else if (kernel == INT4LINEAR_KERNEL_FP6 && source == Workspace::Internal) {
        capturing = stream_is_capturing(stream);
    }
    if (kernel == INT4LINEAR_KERNEL_FP6) {
        if (!fp6_supports(m, n, k))
            return INT4LINEAR_ERR_UNSUPPORTED;
        const int st6 = run_fp6(pd, a, b, c, m, n, k, ep, source, capturing, stream);
        // Under automatic dispatch a workspace that cannot be had falls back to a kernel
        // that needs none.
        if (st6 == INT4LINEAR_OK || !automatic || source == Workspace::Static)
            return st6;
        kernel = mfma_supports(m, n, k) ? INT4LINEAR_KERNEL_MFMA : INT4LINEAR_KERNEL_SIMPLE;
    }

    hipError_t e = hipSuccess;
    switch (kernel) {
    case INT4LINEAR_KERNEL_SIMPLE:
        e = launch_simple(a, b, c, m, n, k, ep, stream);
        break;
    case INT4LINEAR_KERNEL_MFMA:
        if (!mfma_supports(m, n, k))
            return INT4LINEAR_ERR_UNSUPPORTED;
        if (automatic)
            return run_mfma_auto(pd, a, b, c, m, n, k, ep, source, capturing, stream);
        e = launch_mfma(a, b, c, m, n, k, ep, pd->info, stream);
        break;
    case INT4LINEAR_KERNEL_MFMA_128:
    case INT4LINEAR_KERNEL_MFMA_256:
        if (!mfma_supports(m, n, k))
            return INT4LINEAR_ERR_UNSUPPORTED;
        e = launch_mfma_tile(a, b, c, m, n, k, kernel == INT4LINEAR_KERNEL_MFMA_128 ? 128 : 256, ep,
                             pd->info, stream);
        break;
    case INT4LINEAR_KERNEL_SKINNY:
        if (!skinny_supports(m, n, k))
            return INT4LINEAR_ERR_UNSUPPORTED;
        if (automatic)
            return run_skinny_auto(pd, a, b, c, m, n, k, ep, source, capturing, stream);
        e = launch_skinny(a, b, c, m, n, k, ep, pd->info, stream);
        break;
    default:
        return INT4LINEAR_ERR_UNSUPPORTED;
    }
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

// Blocking call in the reference's style: enqueue on the default stream, then wait for
// the device, as kernels/linear_v21.cu:37-39 does.
void launch_blocking(const char *name, void *x, void *w, void *y, int m, int n, int k, int kernel)
{
    int st = gemm_impl(x, w, y, m, n, k, kernel, nullptr);
    if (st == INT4LINEAR_OK) {
        hipError_t e = hipDeviceSynchronize();
        if (e != hipSuccess)
            st = fail_hip(e);
    }
    if (st != INT4LINEAR_OK)
        std::fprintf(stderr, "%s FAILED: %s (hip error %d)\n", name, int4linear_status_string(st),
                     t_last_hip_error);
}

}  // namespace

extern "C" {

int int4linear_init(void) { return ensure_init(nullptr); }

int int4linear_gemm_s4s4s32(const void *a_packed_d, const void *b_packed_d, void *c_d, int m,
                            int n, int k, void *stream)
{
    return gemm_impl(a_packed_d, b_packed_d, c_d, m, n, k, INT4LINEAR_KERNEL_AUTO, stream);
}

int int4linear_gemm_s4s4s32_static(const void *a_packed_d, const void *b_packed_d, void *c_d, int m,
                                   int n, int k, void *stream)
{
    return gemm_impl(a_packed_d, b_packed_d, c_d, m, n, k, INT4LINEAR_KERNEL_AUTO, stream, Epilogue{},
                     Workspace::Static);
}

int int4linear_gemm_s4s4s32_ex(const void *a_packed_d, const void *b_packed_d, void *c_d, int m,
                               int n, int k, int kernel, void *stream)
{
    return gemm_impl(a_packed_d, b_packed_d, c_d, m, n, k, kernel, stream);
}

int int4linear_linear_s32(const void *x_packed_d, const void *w_packed_d, const int *bias_d, void *y_d,
                          int m, int n, int k, int kernel, void *stream)
{
    Epilogue ep;
    ep.bias = bias_d;
    return gemm_impl(x_packed_d, w_packed_d, y_d, m, n, k, kernel, stream, ep);
}

int int4linear_linear_f32(const void *x_packed_d, const void *w_packed_d, const int *bias_d,
                          const float *row_scale_d, const float *col_scale_d, float *y_d, int m, int n,
                          int k, int kernel, void *stream)
{
    Epilogue ep;
    ep.bias = bias_d;
    ep.row_scale = row_scale_d;
    ep.col_scale = col_scale_d;
    ep.out = kOutF32;
    return gemm_impl(x_packed_d, w_packed_d, y_d, m, n, k, kernel, stream, ep);
}

int int4linear_linear_f16(const void *x_packed_d, const void *w_packed_d, const int *bias_d,
                          const float *row_scale_d, const float *col_scale_d, void *y_d, int m, int n,
                          int k, int kernel, void *stream)
{
    Epilogue ep;
    ep.bias = bias_d;
    ep.row_scale = row_scale_d;
    ep.col_scale = col_scale_d;
    ep.out = kOutF16;
    return gemm_impl(x_packed_d, w_packed_d, y_d, m, n, k, kernel, stream, ep);
}

int int4linear_linear_bf16(const void *x_packed_d, const void *w_packed_d, const int *bias_d,
                           const float *row_scale_d, const float *col_scale_d, void *y_d, int m, int n,
                           int k, int kernel, void *stream)
{
    Epilogue ep;
    ep.bias = bias_d;
    ep.row_scale = row_scale_d;
    ep.col_scale = col_scale_d;
    ep.out = kOutBF16;
    return gemm_impl(x_packed_d, w_packed_d, y_d, m, n, k, kernel, stream, ep);
}

int int4linear_pack_s32_to_s4(const int *src_d, int *dst_d, int m, int n, void *stream)
{
    if (m < 0 || n < 0)
        return INT4LINEAR_ERR_SHAPE;
    if (m == 0 || n == 0)
        return INT4LINEAR_OK;
    if (!src_d || !dst_d)
        return INT4LINEAR_ERR_NULL;
    int st = ensure_init(nullptr, true, (hipStream_t)stream);
    if (st != INT4LINEAR_OK)
        return st;
    hipError_t e = launch_pack(src_d, dst_d, m, n, (hipStream_t)stream);
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

int int4linear_unpack_s4_to_s32(const int *src_d, int *dst_d, int m, int n, void *stream)
{
    if (m < 0 || n < 0)
        return INT4LINEAR_ERR_SHAPE;
    if (m == 0 || n == 0)
        return INT4LINEAR_OK;
    if (!src_d || !dst_d)
        return INT4LINEAR_ERR_NULL;
    int st = ensure_init(nullptr, true, (hipStream_t)stream);
    if (st != INT4LINEAR_OK)
        return st;
    hipError_t e = launch_unpack(src_d, dst_d, m, n, (hipStream_t)stream);
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

size_t int4linear_fp6_operand_bytes(int rows, int k)
{
    if (rows <= 0 || !fp6_supports(rows, 1, k))
        return 0;
    return fp6_operand_bytes(rows, k);
}

int int4linear_fp6_convert(const void *packed_d, void *converted_d, int rows, int k, void *stream)
{
    if (rows < 0 || k < 0 || (k % 8) != 0)
        return INT4LINEAR_ERR_SHAPE;
    if (rows == 0)
        return INT4LINEAR_OK;
    if (!fp6_supports(rows, 1, k))
        return INT4LINEAR_ERR_UNSUPPORTED;
    if (!packed_d || !converted_d)
        return INT4LINEAR_ERR_NULL;
    if (!aligned16(packed_d) || ((uintptr_t)converted_d & 255) != 0)
        return INT4LINEAR_ERR_ALIGN;
    int st = ensure_init(nullptr, true, (hipStream_t)stream);
    if (st != INT4LINEAR_OK)
        return st;
    hipError_t e = launch_fp6_convert(packed_d, converted_d, rows, k, (hipStream_t)stream);
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

}  // extern "C"

namespace {

int fp6_converted_impl(const void *a_conv_d, const void *b_conv_d, void *c_d, int m, int n, int k,
                       const Epilogue &ep, void *stream)
{
    if (m < 0 || n < 0 || k < 0 || (k % 8) != 0)
        return INT4LINEAR_ERR_SHAPE;
    if (m == 0 || n == 0)
        return INT4LINEAR_OK;
    if (!fp6_supports(m, n, k))
        return INT4LINEAR_ERR_UNSUPPORTED;
    if (!a_conv_d || !b_conv_d || !c_d)
        return INT4LINEAR_ERR_NULL;
    if (!aligned16(c_d) || ((uintptr_t)a_conv_d & 255) != 0 || ((uintptr_t)b_conv_d & 255) != 0)
        return INT4LINEAR_ERR_ALIGN;
    PerDevice *pd = nullptr;
    int st = ensure_init(&pd, true, (hipStream_t)stream);
    if (st != INT4LINEAR_OK)
        return st;
    hipError_t e = launch_fp6_gemm(a_conv_d, b_conv_d, c_d, m, n, k, ep, pd->info, (hipStream_t)stream);
    return e == hipSuccess ? INT4LINEAR_OK : fail_hip(e);
}

}  // namespace

extern "C" {

int int4linear_gemm_fp6_converted(const void *a_conv_d, const void *b_conv_d, void *c_d, int m, int n,
                                  int k, void *stream)
{
    return fp6_converted_impl(a_conv_d, b_conv_d, c_d, m, n, k, Epilogue{}, stream);
}

int int4linear_linear_fp6_converted(const void *x_conv_d, const void *w_conv_d, const int *bias_d,
                                    const float *row_scale_d, const float *col_scale_d, void *y_d, int out_type,
                                    int m, int n, int k, void *stream)
{
    if (out_type < INT4LINEAR_OUT_S32 || out_type > INT4LINEAR_OUT_BF16)
        return INT4LINEAR_ERR_UNSUPPORTED;
    if (out_type == INT4LINEAR_OUT_S32 && (row_scale_d || col_scale_d))
        return INT4LINEAR_ERR_UNSUPPORTED;  // an int32 output takes a bias only
    Epilogue ep;
    ep.bias = bias_d;
    ep.row_scale = row_scale_d;
    ep.col_scale = col_scale_d;
    ep.out = out_type;  // the INT4LINEAR_OUT_* values are the kernels' OutKind values
    return fp6_converted_impl(x_conv_d, w_conv_d, y_d, m, n, k, ep, stream);
}

const char *int4linear_kernel_for_shape(int m, int n, int k)
{
    if (m < 0 || n < 0 || k < 0 || (k % 8) != 0)
        return "invalid";
    switch (pick_kernel(m, n, k, current_device_info(), g_workspace_limit.load())) {
    case INT4LINEAR_KERNEL_SKINNY:
        return "skinny";
    case INT4LINEAR_KERNEL_FP6:
        return "fp6";
    case INT4LINEAR_KERNEL_MFMA:
        return "mfma";
    default:
        return "simple";
    }
}

const char *int4linear_status_string(int status)
{
    switch (status) {
    case INT4LINEAR_OK:
        return "ok";
    case INT4LINEAR_ERR_SHAPE:
        return "invalid shape (negative dimension or K not a multiple of 8)";
    case INT4LINEAR_ERR_NULL:
        return "null pointer for a non-empty operand";
    case INT4LINEAR_ERR_ALIGN:
        return "operand base pointer is not 16-byte aligned";
    case INT4LINEAR_ERR_HIP:
        return "HIP runtime error";
    case INT4LINEAR_ERR_UNSUPPORTED:
        return "requested kernel does not support this shape";
    case INT4LINEAR_ERR_NO_DEVICE:
        return "no usable HIP device";
    case INT4LINEAR_ERR_NOT_INITIALISED:
        return "first call on this device came while its stream was being captured: call int4linear_init() before the capture";
    case INT4LINEAR_ERR_SCRATCH:
        return "only a kernel with more scratch memory than the static array of int4linear_gemm_s4s4s32_static holds is fast for this shape";
    default:
        return "unknown status";
    }
}

int int4linear_last_hip_error(void) { return t_last_hip_error; }

size_t int4linear_workspace_bytes(int m, int n, int k)
{
    if (m < 1 || n < 1 || k < 8 || (k % 8) != 0)
        return 0;
    const DeviceInfo info = current_device_info();
    const int kernel = pick_kernel(m, n, k, info, g_workspace_limit.load());
    if (kernel == INT4LINEAR_KERNEL_FP6)
        return fp6_workspace_bytes(m, n, k, info);
    if (kernel == INT4LINEAR_KERNEL_MFMA || kernel == INT4LINEAR_KERNEL_SKINNY) {
        // the split-K forms need the device's CU count: unknown only without a device
        if (info.cu_count == 0)
            return 0;
        const size_t need = kernel == INT4LINEAR_KERNEL_MFMA ? mfma_workspace_bytes(m, n, k, info)
                                                             : skinny_workspace_bytes(m, n, k, info);
        return need <= g_workspace_limit.load() ? need : 0;
    }
    return 0;
}

void int4linear_set_workspace_limit(size_t bytes) { g_workspace_limit.store(bytes); }

int int4linear_release_workspace(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return INT4LINEAR_ERR_NO_DEVICE;
    PerDevice &pd = g_devices[dev];
    std::lock_guard<std::mutex> lock(pd.ws_mutex);
    if (pd.ws) {
        hipError_t e = hipFree(pd.ws);
        pd.ws = nullptr;
        pd.ws_bytes = 0;
        pd.ws_used = false;
        if (e != hipSuccess)
            return fail_hip(e);
    }
    return INT4LINEAR_OK;
}

int int4linear_device_cu_count(void)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return 0;
    return g_devices[dev].info.cu_count;
}

}  // extern "C"

// ---- the reference's C++-linkage entry points ------------------------------------------

namespace {

// Kernel of each step of the version history for a shape; a step whose kernel cannot take
// the shape falls back to the step before it.
int version_kernel(int version, int m, int n, int k, const DeviceInfo &info)
{
    const bool int8_ok = mfma_supports(m, n, k);
    switch (version) {
    case 21:
        return INT4LINEAR_KERNEL_AUTO;
    case 20:
        if (fp6_supports(m, n, k) && fp6_workspace_bytes(m, n, k, info) <= g_workspace_limit.load() &&
            !skinny_preferred(m, n, k, info))
            return INT4LINEAR_KERNEL_FP6;
        [[fallthrough]];
    case 11:
        if (skinny_preferred(m, n, k, info))
            return INT4LINEAR_KERNEL_SKINNY;
        [[fallthrough]];
    case 10:
        return int8_ok ? INT4LINEAR_KERNEL_MFMA : INT4LINEAR_KERNEL_SIMPLE;
    case 2:
        return int8_ok ? INT4LINEAR_KERNEL_MFMA_256 : INT4LINEAR_KERNEL_SIMPLE;
    case 1:
        return int8_ok ? INT4LINEAR_KERNEL_MFMA_128 : INT4LINEAR_KERNEL_SIMPLE;
    default:
        return INT4LINEAR_KERNEL_SIMPLE;
    }
}

void launch_version(const char *name, int version, void *x, void *w, void *y, int m, int n, int k)
{
    const bool valid = m >= 0 && n >= 0 && k >= 0 && (k % 8) == 0;
    // The choice may depend on the device; a device that cannot be set up is reported by the launch.
    const DeviceInfo info = current_device_info();
    launch_blocking(name, x, w, y, m, n, k, valid ? version_kernel(version, m, n, k, info) : INT4LINEAR_KERNEL_AUTO);
}

}  // namespace

void linear_v0_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v0_launch", 0, x, w, y, m, n, k);
}
void linear_v1_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v1_launch", 1, x, w, y, m, n, k);
}
void linear_v2_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v2_launch", 2, x, w, y, m, n, k);
}
void linear_v10_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v10_launch", 10, x, w, y, m, n, k);
}
void linear_v11_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v11_launch", 11, x, w, y, m, n, k);
}
void linear_v20_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v20_launch", 20, x, w, y, m, n, k);
}
void linear_v21_launch(void *x, void *w, void *y, int m, int n, int k)
{
    launch_version("linear_v21_launch", 21, x, w, y, m, n, k);
}
