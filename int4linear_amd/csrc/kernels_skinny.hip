// Weight-streaming kernel for skinny M (M <= 64): the decode-shaped linear layer.
//
// The job is HBM-bound: every byte of W (N x K/2) is read exactly once, straight from
// global memory into registers with 16-byte loads, widened to int8 (same 16x trick as
// the big kernel: (w << 4) & 0xF0F0F0F0 and w & 0xF0F0F0F0) and multiplied on
// v_mfma_i32_16x16x64_i8 against X, which is small enough to live in L2.
//
// A workgroup owns 16 consecutive rows of W (16 columns of C) -- one contiguous
// 16 * K/2-byte slab -- and its wavefronts split K between them, interleaved by
// 128-nibble steps so each round of the workgroup reads 64*WAVES contiguous bytes of
// every row.  Partial sums meet in LDS; one pass adds them and stores C.  No atomics,
// no workspace, and the result does not depend on timing.
#include "kernels.h"

namespace int4linear {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kStepK = 128;         // nibbles per wave step
constexpr int kStepBytes = 64;      // bytes per row per step
constexpr int kBatch = 4;           // steps whose loads are issued together

template <int FMX, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void skinny_kernel(
    const uint8_t *__restrict__ X, const uint8_t *__restrict__ W, int32_t *__restrict__ Y,
    int M, int N, int K)
{
    __shared__ v4i partial[WAVES][FMX][64];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int fr = lane & 15;  // operand row inside a 16-row fragment
    const int fg = lane >> 4;  // which 16-byte quarter of the 64-byte step
    const int rowbytes = K >> 1;
    const int KT = K / kStepK;
    const int n0 = blockIdx.x * 16;

    const int wrow = (n0 + fr < N) ? n0 + fr : N - 1;
    const uint8_t *wp = W + (size_t)wrow * rowbytes + fg * 16;
    const uint8_t *xp[FMX];
#pragma unroll
    for (int f = 0; f < FMX; ++f) {
        const int xrow = (f * 16 + fr < M) ? f * 16 + fr : M - 1;
        xp[f] = X + (size_t)xrow * rowbytes + fg * 16;
    }

    const int himask = (int)0xF0F0F0F0u;
    v4i acc[FMX];
#pragma unroll
    for (int f = 0; f < FMX; ++f)
        acc[f] = (v4i){0, 0, 0, 0};

    auto mac = [&](const v4i &w, const v4i (&x)[FMX]) {
        const v4i wlo = (w << 4) & himask;
        const v4i whi = w & himask;
#pragma unroll
        for (int f = 0; f < FMX; ++f) {
            const v4i xlo = (x[f] << 4) & himask;
            const v4i xhi = x[f] & himask;
            acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wlo, xlo, acc[f], 0, 0, 0);
            acc[f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(whi, xhi, acc[f], 0, 0, 0);
        }
    };

    int ks = wave;
    // Full batches: all loads of kBatch steps are in flight before the first use.
    for (; ks + (kBatch - 1) * WAVES < KT; ks += kBatch * WAVES) {
        v4i w[kBatch], x[kBatch][FMX];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
            const size_t off = (size_t)(ks + u * WAVES) * kStepBytes;
            w[u] = __builtin_nontemporal_load((const v4i *)(wp + off));
#pragma unroll
            for (int f = 0; f < FMX; ++f)
                x[u][f] = *(const v4i *)(xp[f] + off);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
            mac(w[u], x[u]);
    }
    for (; ks < KT; ks += WAVES) {
        const size_t off = (size_t)ks * kStepBytes;
        v4i w = __builtin_nontemporal_load((const v4i *)(wp + off));
        v4i x[FMX];
#pragma unroll
        for (int f = 0; f < FMX; ++f)
            x[f] = *(const v4i *)(xp[f] + off);
        mac(w, x);
    }

#pragma unroll
    for (int f = 0; f < FMX; ++f)
        partial[wave][f][lane] = acc[f];
    __syncthreads();

    // Element e = (f, lane): n = n0 + 4*(lane/16) + 0..3, m = f*16 + lane%16.
    for (int e = threadIdx.x; e < FMX * 64; e += WAVES * 64) {
        const int f = e >> 6, l = e & 63;
        v4i s = partial[0][f][l];
#pragma unroll
        for (int wv = 1; wv < WAVES; ++wv)
            s += partial[wv][f][l];
        s = s >> 8;  // both operands carried a factor 16
        const int m = f * 16 + (l & 15);
        const int n = n0 + 4 * (l >> 4);
        if (m < M) {
            int32_t *dst = Y + (size_t)m * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(v4i *)dst = s;
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    if (n + t < N)
                        dst[t] = s[t];
            }
        }
    }
}

template <int FMX, int WAVES>
hipError_t launch_one(const void *a, const void *b, void *c, int m, int n, int k,
                      hipStream_t stream)
{
    const unsigned grid = (unsigned)((n + 15) / 16);
    skinny_kernel<FMX, WAVES><<<grid, WAVES * 64, 0, stream>>>(
        (const uint8_t *)a, (const uint8_t *)b, (int32_t *)c, m, n, k);
    return hipGetLastError();
}

template <int WAVES>
hipError_t launch_fmx(const void *a, const void *b, void *c, int m, int n, int k,
                      hipStream_t stream)
{
    switch ((m + 15) / 16) {
    case 1:
        return launch_one<1, WAVES>(a, b, c, m, n, k, stream);
    case 2:
        return launch_one<2, WAVES>(a, b, c, m, n, k, stream);
    case 3:
        return launch_one<3, WAVES>(a, b, c, m, n, k, stream);
    default:
        return launch_one<4, WAVES>(a, b, c, m, n, k, stream);
    }
}

}  // namespace

bool skinny_supports(int m, int n, int k)
{
    return m >= 1 && m <= 64 && n >= 1 && k >= kStepK && k % kStepK == 0 && k <= 131071 - 127;
}

hipError_t launch_skinny(const void *a, const void *b, void *c, int m, int n, int k,
                         const DeviceInfo &dev, hipStream_t stream)
{
    // Wavefronts per workgroup: enough K-splitting that the grid fills the device with
    // at least ~8 waves per CU, bounded by the number of K steps.
    const long groups = (n + 15) / 16;
    const int steps = k / kStepK;
    const long want_waves = (long)dev.cu_count * 8;
    int waves = 4;
    while (waves < 16 && groups * waves < want_waves && waves * 2 <= steps)
        waves *= 2;
    if (waves > steps)
        waves = steps >= 8 ? 8 : (steps >= 4 ? 4 : (steps >= 2 ? 2 : 1));
    switch (waves) {
    case 1:
        return launch_fmx<1>(a, b, c, m, n, k, stream);
    case 2:
        return launch_fmx<2>(a, b, c, m, n, k, stream);
    case 4:
        return launch_fmx<4>(a, b, c, m, n, k, stream);
    case 8:
        return launch_fmx<8>(a, b, c, m, n, k, stream);
    default:
        return launch_fmx<16>(a, b, c, m, n, k, stream);
    }
}

}  // namespace int4linear
