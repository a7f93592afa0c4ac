// Simple kernels: the scalar cross-check GEMM, the device packer/unpacker and a zero
// fill.  None of them is on the performance path; they are written to be obviously
// right and to accept every shape the packed layout allows (K % 8 == 0).
#include "kernels.h"

namespace int4linear {

namespace {

constexpr int kTile = 16;       // outputs per block edge
constexpr int kChunkWords = 16; // 32-bit words (128 nibbles) of K staged per step

// Signed value of nibble `slot` (0..7) of a packed word: utils/packer.cpp:27.
__device__ __forceinline__ int nibble_s4(uint32_t word, int slot)
{
    int v = (int)((word >> (4 * slot)) & 0xFu);
    return (v & 8) ? v - 16 : v;
}

// C[i][j] = sum_l A[i][l] * B[j][l]; one thread per output, operands staged through
// LDS one 128-nibble chunk at a time.  test/test_correctness.cu:12-19 semantics.
__global__ __launch_bounds__(kTile *kTile) void simple_gemm_kernel(
    const uint32_t *__restrict__ a, const uint32_t *__restrict__ b, int32_t *__restrict__ c,
    int m, int n, int k_words, unsigned tile_row0, Epilogue ep)
{
    __shared__ uint32_t a_lds[kTile][kChunkWords + 1];
    __shared__ uint32_t b_lds[kTile][kChunkWords + 1];

    const int tx = threadIdx.x % kTile;  // column of C inside the tile
    const int ty = threadIdx.x / kTile;  // row of C inside the tile
    const long tile_row = (long)tile_row0 + blockIdx.y;  // a launch covers at most 65535 tile rows
    const long row = tile_row * kTile + ty;
    const long col = (long)blockIdx.x * kTile + tx;

    int acc = 0;
    for (int w0 = 0; w0 < k_words; w0 += kChunkWords) {
        // Thread (ty, tx) stages word tx of row ty of each operand tile.
        const int w = w0 + tx;
        const long a_row = tile_row * kTile + ty;
        const long b_row = (long)blockIdx.x * kTile + ty;
        a_lds[ty][tx] = (a_row < m && w < k_words) ? a[a_row * k_words + w] : 0u;
        b_lds[ty][tx] = (b_row < n && w < k_words) ? b[b_row * k_words + w] : 0u;
        __syncthreads();
        for (int ww = 0; ww < kChunkWords; ++ww) {
            const uint32_t aw = a_lds[ty][ww];
            const uint32_t bw = b_lds[tx][ww];
            for (int s = 0; s < 8; ++s)
                acc += nibble_s4(aw, s) * nibble_s4(bw, s);
        }
        __syncthreads();
    }
    if (row < m && col < n)
        store_out(ep, c, (size_t)(row * n + col),
                  epilogue_value(ep, acc, ep.bias ? ep.bias[col] : 0, ep.row_scale ? ep.row_scale[row] : 1.f,
                                 ep.col_scale ? ep.col_scale[col] : 1.f));
}

// utils/packer.cpp:3-18 on device arrays: one thread per destination word.
__global__ void pack_kernel(const int *__restrict__ src, int *__restrict__ dst, int m, int n,
                            int words)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)m * words)
        return;
    const long row = idx / words;
    const int w = (int)(idx % words);
    uint32_t word = 0;
    for (int s = 0; s < 8; ++s) {
        const int col = w * 8 + s;
        if (col < n)
            word |= ((uint32_t)src[row * n + col] & 0xFu) << (4 * s);
    }
    dst[idx] = (int)word;
}

// utils/packer.cpp:20-31 on device arrays: one thread per destination element.
__global__ void unpack_kernel(const int *__restrict__ src, int *__restrict__ dst, int m,
                              int n, int words)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)m * n)
        return;
    const long row = idx / n;
    const int col = (int)(idx % n);
    dst[idx] = nibble_s4((uint32_t)src[row * words + col / 8], col % 8);
}

__global__ void zero_i32_kernel(int4 *__restrict__ dst4, int *__restrict__ dst, size_t vec_count,
                                size_t count)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (size_t v = i; v < vec_count; v += stride)
        dst4[v] = make_int4(0, 0, 0, 0);
    for (size_t t = vec_count * 4 + i; t < count; t += stride)
        dst[t] = 0;
}

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));

// Second kernel of the split-K forms: Y = epilogue(sum of the ksplit slabs), four outputs of
// one row per thread (VEC: n % 4 == 0) or one.
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const int32_t *__restrict__ partial,
                                                                int32_t *__restrict__ Y, size_t count, int ksplit,
                                                                int N, Epilogue ep)
{
    constexpr int kPer = VEC ? 4 : 1;
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * kPer;
    if (i >= count)
        return;
    int sum[kPer] = {};
    for (int s = 0; s < ksplit; ++s) {
        const int32_t *src = partial + (size_t)s * count + i;
        if constexpr (VEC) {
            const v4i v = __builtin_nontemporal_load((const v4i *)src);
#pragma unroll
            for (int q = 0; q < 4; ++q)
                sum[q] += v[q];
        } else {
            sum[0] += *src;
        }
    }
    const size_t row = i / (size_t)N;
    const int col = (int)(i - row * (size_t)N);
    const float rs = ep.row_scale ? ep.row_scale[row] : 1.f;
    by_output_width(ep, [&](auto half) {
#pragma unroll
        for (int q = 0; q < kPer; ++q)
            sum[q] = epilogue_value_of<half()>(ep, sum[q], ep.bias ? ep.bias[col + q] : 0, rs,
                                               ep.col_scale ? ep.col_scale[col + q] : 1.f);
        if constexpr (half() && VEC)  // i % 4 == 0: four half-width outputs are eight aligned bytes
            *(v2i *)((unsigned short *)Y + i) = (v2i){sum[0] | (sum[1] << 16), sum[2] | (sum[3] << 16)};
        else if constexpr (half())
            ((unsigned short *)Y)[i] = (unsigned short)sum[0];
        else if constexpr (VEC)
            *(v4i *)(Y + i) = (v4i){sum[0], sum[1], sum[2], sum[3]};
        else
            Y[i] = sum[0];
    });
}

}  // namespace

hipError_t launch_simple(const void *a, const void *b, void *c, int m, int n, int k,
                         const Epilogue &ep, hipStream_t stream)
{
    // The grid's y extent ends at 65535: more tile rows than that go out as several launches.
    const unsigned tile_rows = (unsigned)((m + kTile - 1) / kTile);
    for (unsigned row0 = 0; row0 < tile_rows; row0 += 65535u) {
        const unsigned rows = tile_rows - row0 < 65535u ? tile_rows - row0 : 65535u;
        const dim3 grid((n + kTile - 1) / kTile, rows);
        simple_gemm_kernel<<<grid, kTile * kTile, 0, stream>>>(
            (const uint32_t *)a, (const uint32_t *)b, (int32_t *)c, m, n, k / 8, row0, ep);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess)
            return e;
    }
    return hipSuccess;
}

hipError_t launch_pack(const int *src, int *dst, int m, int n, hipStream_t stream)
{
    const int words = (n + 7) / 8;
    const long total = (long)m * words;
    if (total == 0)
        return hipSuccess;
    const int block = 256;
    pack_kernel<<<(unsigned)((total + block - 1) / block), block, 0, stream>>>(src, dst, m, n,
                                                                                words);
    return hipGetLastError();
}

hipError_t launch_unpack(const int *src, int *dst, int m, int n, hipStream_t stream)
{
    const int words = (n + 7) / 8;
    const long total = (long)m * n;
    if (total == 0)
        return hipSuccess;
    const int block = 256;
    unpack_kernel<<<(unsigned)((total + block - 1) / block), block, 0, stream>>>(src, dst, m, n,
                                                                                  words);
    return hipGetLastError();
}

hipError_t launch_zero_i32(int *dst, size_t count, hipStream_t stream)
{
    if (count == 0)
        return hipSuccess;
    // dst is 16-byte aligned (checked by the API layer), so the bulk goes out as int4.
    const size_t vec_count = count / 4;
    const int block = 256;
    size_t want = (vec_count + block - 1) / block;
    unsigned grid = (unsigned)(want < 1 ? 1 : (want > 8192 ? 8192 : want));
    zero_i32_kernel<<<grid, block, 0, stream>>>((int4 *)dst, dst, vec_count, count);
    return hipGetLastError();
}

hipError_t launch_splitk_reduce(const void *slabs, void *c, size_t count, int ksplit, int n, const Epilogue &ep,
                                hipStream_t stream)
{
    if (count == 0)
        return hipSuccess;
    if (n % 4 == 0)
        splitk_reduce_kernel<true><<<(unsigned)((count / 4 + 255) / 256), 256, 0, stream>>>(
            (const int32_t *)slabs, (int32_t *)c, count, ksplit, n, ep);
    else
        splitk_reduce_kernel<false><<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(
            (const int32_t *)slabs, (int32_t *)c, count, ksplit, n, ep);
    return hipGetLastError();
}

}  // namespace int4linear
