// Internal launcher interface between the C ABI (api.hip) and the kernel files.
// Every launcher enqueues on `stream` and returns the hipError_t of the launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#if defined(__HIPCC__)
#include <type_traits>
#endif

namespace int4linear {

// Optional work between the accumulator and the store of every output element (i, j):
//   v = acc + bias[j]                                   (bias null: + 0)
//   out == kOutS32: C is int32 and receives v
//   otherwise:      t = (float)v * row_scale[i] * col_scale[j]
//                   (a null scale counts as 1; the two multiplications happen in that order)
//     kOutF32:  C is float and receives t
//     kOutF16:  C is IEEE half and receives t rounded to nearest even
//     kOutBF16: C is bfloat16 and receives t rounded to nearest even
//     (both: t is a float first, so there are two roundings; overflow goes to infinity,
//     denormals are kept, a NaN keeps its sign and upper payload bits and becomes quiet)
// Passed to the kernels by value; an all-zero struct is the plain GEMM.
enum OutKind : int { kOutS32 = 0, kOutF32 = 1, kOutF16 = 2, kOutBF16 = 3 };

struct Epilogue {
    const int32_t *bias = nullptr;
    const float *row_scale = nullptr;
    const float *col_scale = nullptr;
    int out = kOutS32;  // an OutKind
};

#if defined(__HIPCC__)
// The 32 bits stored for one output element of the two full-width kinds.
__device__ __forceinline__ int epilogue_value32(const Epilogue &ep, int acc, int bias_j, float row_scale_i,
                                                float col_scale_j)
{
    const int v = acc + bias_j;
    if (!ep.out)
        return v;
    return __float_as_int(((float)v * row_scale_i) * col_scale_j);
}

// The 16 bits (in the low half) stored for one output element of the two half-width kinds.
__device__ __forceinline__ int epilogue_value16(const Epilogue &ep, int acc, int bias_j, float row_scale_i,
                                                float col_scale_j)
{
    float t = ((float)(acc + bias_j) * row_scale_i) * col_scale_j;
    // The product is rounded to float before it is rounded to 16 bits; with the product in
    // sight the compiler would merge the two into one instruction that rounds once
    // (v_fma_mixlo_f16), which differs at ties.
    asm("" : "+v"(t));
    if (ep.out == kOutF16)
        return (int)(unsigned short)__builtin_bit_cast(unsigned short, (_Float16)t);
    // gfx950 converts in hardware (v_cvt_pk_bf16_f32): round to nearest even, denormals kept,
    // a NaN keeps its sign and its upper payload bits and becomes quiet.
    return (int)__builtin_bit_cast(unsigned short, (__bf16)t);
}

__device__ __forceinline__ bool out_is_half_width(const Epilogue &ep) { return ep.out >= kOutF16; }

// Either of them, by the kind of output.
__device__ __forceinline__ int epilogue_value(const Epilogue &ep, int acc, int bias_j, float row_scale_i,
                                              float col_scale_j)
{
    return out_is_half_width(ep) ? epilogue_value16(ep, acc, bias_j, row_scale_i, col_scale_j)
                                 : epilogue_value32(ep, acc, bias_j, row_scale_i, col_scale_j);
}

// Element `index` of the output array, whichever its width.
__device__ __forceinline__ void store_out(const Epilogue &ep, void *c, size_t index, int bits)
{
    if (out_is_half_width(ep))
        ((unsigned short *)c)[index] = (unsigned short)bits;
    else
        ((int *)c)[index] = bits;
}

// Four consecutive outputs of one row, elements index .. index + 3, of which the first `valid`
// (0 .. 4) exist.  `together`: all four exist and index is a multiple of four elements from a
// 16-byte-aligned base with a row length that is one too, so they go out as one store.
// HALF: the output's elements are 16 bits wide.
typedef int out_v4i __attribute__((ext_vector_type(4)));
typedef int out_v2i __attribute__((ext_vector_type(2)));
template <bool HALF>
__device__ __forceinline__ void store_out4(void *c, size_t index, out_v4i bits, int valid, bool together)
{
    if constexpr (HALF) {
        unsigned short *dst = (unsigned short *)c + index;
        if (together) {
            *(out_v2i *)dst = (out_v2i){bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16)};
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (q < valid)
                    dst[q] = (unsigned short)bits[q];
        }
    } else {
        int *dst = (int *)c + index;
        if (together) {
            *(out_v4i *)dst = bits;
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (q < valid)
                    dst[q] = bits[q];
        }
    }
}

template <bool HALF>
__device__ __forceinline__ int epilogue_value_of(const Epilogue &ep, int acc, int bias_j, float row_scale_i,
                                                 float col_scale_j)
{
    if constexpr (HALF)
        return epilogue_value16(ep, acc, bias_j, row_scale_i, col_scale_j);
    else
        return epilogue_value32(ep, acc, bias_j, row_scale_i, col_scale_j);
}

// f(std::true_type) for the half-width kinds of output, f(std::false_type) for the others:
// the kind is looked at once, not per element.
template <class F>
__device__ __forceinline__ void by_output_width(const Epilogue &ep, F &&f)
{
    if (out_is_half_width(ep))
        f(std::true_type{});
    else
        f(std::false_type{});
}
#endif

struct DeviceInfo {
    int cu_count = 0;      // compute units on the device
    int lds_per_cu = 0;    // bytes of LDS a workgroup may use
};

// One thread per output, scalar nibble decode.  Any M, N >= 1 and K % 8 == 0.
hipError_t launch_simple(const void *a, const void *b, void *c, int m, int n, int k,
                         const Epilogue &ep, hipStream_t stream);

// LDS-pipelined MFMA kernel.  Requires K % 128 == 0, K >= 128.
bool mfma_supports(int m, int n, int k);
hipError_t mfma_init(const DeviceInfo &dev);
hipError_t launch_mfma(const void *a, const void *b, void *c, int m, int n, int k,
                       const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);

// Split-K form for shapes with few tiles and long K: ksplit K-slices per 128 x 128 tile write
// partial sums into `workspace` (mfma_workspace_bytes() bytes, 0 = the shape is not split),
// a second kernel adds them up and applies the epilogue.  With a null workspace it is
// launch_mfma.
size_t mfma_workspace_bytes(int m, int n, int k, const DeviceInfo &dev);
hipError_t launch_mfma_splitk(const void *a, const void *b, void *c, int m, int n, int k, void *workspace,
                              const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);

// The same kernel with the workgroup tile forced to 128 x 128 or 256 x 256 (`tile`).
hipError_t launch_mfma_tile(const void *a, const void *b, void *c, int m, int n, int k, int tile,
                            const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);

// FP6-MFMA path: converts both operands into a workspace of fp6_workspace_bytes() bytes
// (256-byte aligned), then runs the GEMM on it.  Requires K % 8 == 0, K < 2^18.  With few
// output tiles and long K the GEMM is split over K (fp6_ksplit() slices per tile, 1 = not
// split; it depends on the device's CU count and is 1 while that is unknown): the partial
// sums go into slabs in the same workspace and a second kernel adds them up.
bool fp6_supports(int m, int n, int k);
int fp6_ksplit(int m, int n, int k, const DeviceInfo &dev);
size_t fp6_workspace_bytes(int m, int n, int k, const DeviceInfo &dev);
hipError_t fp6_init(const DeviceInfo &dev);
// The two halves of launch_fp6 on caller-owned buffers: an operand of `rows` rows converts
// into fp6_operand_bytes(rows, k) bytes (256-byte aligned); the GEMM runs on two of those.
size_t fp6_operand_bytes(int rows, int k);
hipError_t launch_fp6_convert(const void *src, void *dst, int rows, int k, hipStream_t stream);
hipError_t launch_fp6_gemm(const void *a_conv, const void *b_conv, void *c, int m, int n, int k,
                           const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);
hipError_t launch_fp6(const void *a, const void *b, void *c, int m, int n, int k, void *workspace,
                      const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);

// Weight-streaming kernel for skinny M.  K % 128 == 0; M <= 64, or more (in runs of 64
// rows) when K splits into 128-byte tiles that fit the kernel's plans.  skinny_preferred:
// the shapes for which the automatic dispatch uses it.
bool skinny_supports(int m, int n, int k);
bool skinny_preferred(int m, int n, int k, const DeviceInfo &dev);
hipError_t skinny_init(const DeviceInfo &dev);
hipError_t launch_skinny(const void *a, const void *b, void *c, int m, int n, int k,
                         const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);

// The same kernel split over K across workgroups, for shapes in which a workgroup that owns
// whole rows of W would pull far more of X than of W (more than 16 rows of X, long K, few
// rows of W per CU): a workgroup takes a rectangle (rows of W) x (slice of K), stores its
// partial sums into `workspace` (skinny_workspace_bytes() bytes, 8-byte aligned; 0 = the
// shape is not split) and counts itself in at `arrivals` (kSkinnyArrivalWords words that are
// zero before the launch and zero again after it); the last workgroup of a row block to
// arrive adds the partial sums up, applies the epilogue and stores.  Nobody waits for
// anybody, and integer sums do not depend on the order of arrival.  Launches that share
// `workspace` or `arrivals` must not overlap.
constexpr int kSkinnyArrivalWords = 4096;
size_t skinny_workspace_bytes(int m, int n, int k, const DeviceInfo &dev);
hipError_t launch_skinny_ksplit(const void *a, const void *b, void *c, int m, int n, int k, void *workspace,
                                unsigned *arrivals, const Epilogue &ep, const DeviceInfo &dev, hipStream_t stream);

// Device packer / unpacker, utils/packer.cpp layouts.
hipError_t launch_pack(const int *src, int *dst, int m, int n, hipStream_t stream);
hipError_t launch_unpack(const int *src, int *dst, int m, int n, hipStream_t stream);

// Fill `count` int32 words with zero (a kernel, so callers may capture it in a graph).
hipError_t launch_zero_i32(int *dst, size_t count, hipStream_t stream);

// Second kernel of the split-K forms: c = epilogue(sum of the ksplit slabs of count = m * n
// partial sums each that lie back to back at `slabs`, 16-byte aligned).
hipError_t launch_splitk_reduce(const void *slabs, void *c, size_t count, int ksplit, int n, const Epilogue &ep,
                                hipStream_t stream);

}  // namespace int4linear
