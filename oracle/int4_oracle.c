/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the packed signed-int4 linear layer.
 *
 * This file restates, in plain C, the host-side algorithm of the reference
 * (myeongs-song/Int4Linear).  It is the checker that the GPU library is compared
 * against; it is never the thing that is shipped or measured as the product.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference tree).  How each one is pinned (none is "parity unpinned"):
 *   oracle_pack        - known-answer words derived from utils/packer.cpp:11, a
 *                        byte-view closed form, and a bit-for-bit diff against the
 *                        reference's own packer.cpp compiled into oracle/_ref/.
 *   oracle_unpack      - round trip through pack for every nibble value and ragged
 *                        widths, nibble sign table, and the same diff against _ref.
 *   oracle_linear_ref  - an independent float64 BLAS product (exact below 2^53),
 *                        closed forms (all -8 => 64*K, one-hot rows, ones),
 *                        algebraic invariants (linearity, K-permutation,
 *                        transposition) and pure-Python brute force on tiny shapes.
 *   oracle_is_same     - trivial; checked on equal / one-element-different arrays.
 *   oracle_epilogue    - not in the reference's code (its README.md:72 names the bias
 *                        add as future work); the definition is this library's own
 *                        header.  Pinned against numpy: int32 wrap-around add for the
 *                        bias, float32 astype / multiply (IEEE round-to-nearest, same
 *                        order) for the scaled output, plus the identities
 *                        "no operands == the plain product" and "scales of 1 == cast".
 *                        The two half-width outputs (oracle_f32_to_f16_bits,
 *                        oracle_f32_to_bf16_bits: one more rounding to nearest even) are
 *                        pinned against numpy's float16 conversion over every float16 value,
 *                        every halfway point between neighbours and random floats, and
 *                        against torch's bfloat16 conversion likewise; quiet NaNs (sign
 *                        and upper payload bits kept) against numpy for the half and
 *                        against the closed form (upper 16 bits, quiet bit set) for
 *                        bfloat16.
 */
#include <stddef.h>
#include <stdint.h>

/* utils/packer.cpp:3-18.  src holds one value per int (any int, only the low four
 * bits are kept); dst holds ceil(n/8) 32-bit words per row; element 8j+k of a row
 * goes to bits [4k, 4k+4) of word j; positions past n stay zero. */
void oracle_pack(const int *src, int *dst, int m, int n)
{
    int words = (n + 7) / 8;
    for (int row = 0; row < m; ++row) {
        for (int w = 0; w < words; ++w) {
            uint32_t word = 0;
            for (int slot = 0; slot < 8; ++slot) {
                int col = w * 8 + slot;
                if (col < n) {
                    uint32_t nib = (uint32_t)src[(size_t)row * n + col] & 0xFu;
                    word |= nib << (4 * slot);
                }
            }
            dst[(size_t)row * words + w] = (int)word;
        }
    }
}

/* utils/packer.cpp:20-31.  Inverse of pack; a nibble with bit 3 set is negative. */
void oracle_unpack(const int *src, int *dst, int m, int n)
{
    int words = (n + 7) / 8;
    for (int row = 0; row < m; ++row) {
        for (int col = 0; col < n; ++col) {
            uint32_t word = (uint32_t)src[(size_t)row * words + col / 8];
            int nib = (int)((word >> (4 * (col % 8))) & 0xFu);
            dst[(size_t)row * n + col] = (nib >= 8) ? nib - 16 : nib;
        }
    }
}

/* test/test_correctness.cu:12-19.  y[i][j] = sum_l x[i][l] * w[j][l] over UNPACKED
 * int-per-element arrays, int32 accumulation, i-j-l loop order. */
void oracle_linear_ref(const int *x, const int *w, int *y, int m, int n, int k)
{
    for (int i = 0; i < m; ++i) {
        const int *xr = x + (size_t)i * k;
        for (int j = 0; j < n; ++j) {
            const int *wr = w + (size_t)j * k;
            int acc = 0;
            for (int l = 0; l < k; ++l)
                acc += xr[l] * wr[l];
            y[(size_t)i * n + j] = acc;
        }
    }
}

/* Same loop nest as oracle_linear_ref with the outer (row) loop spread over
 * `threads` OpenMP threads.  Used for the "all host cores" CPU baseline and to keep
 * full-matrix checks of mid-sized shapes within seconds.  Integer sums make the
 * result independent of the thread count. */
void oracle_linear_ref_mt(const int *x, const int *w, int *y, int m, int n, int k,
                          int threads)
{
    if (threads < 1)
        threads = 1;
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1)
    for (int i = 0; i < m; ++i) {
        const int *xr = x + (size_t)i * k;
        for (int j = 0; j < n; ++j) {
            const int *wr = w + (size_t)j * k;
            int acc = 0;
            for (int l = 0; l < k; ++l)
                acc += xr[l] * wr[l];
            y[(size_t)i * n + j] = acc;
        }
    }
}

/* test/test_correctness.cu:22-27.  1 when the first `count` ints agree, else 0. */
int oracle_is_same(const int *a, const int *b, int count)
{
    for (int i = 0; i < count; ++i)
        if (a[i] != b[i])
            return 0;
    return 1;
}

/* float -> IEEE half, round to nearest even; beyond the largest half it is infinity, a NaN
 * keeps its sign and the upper nine payload bits and becomes quiet. */
unsigned oracle_f32_to_f16_bits(float f)
{
    union { float f; uint32_t u; } v;
    v.f = f;
    const uint32_t sign = (v.u >> 16) & 0x8000u;
    const uint32_t x = v.u & 0x7fffffffu;
    if (x > 0x7f800000u) /* a NaN keeps its sign and upper payload bits and becomes quiet */
        return sign | 0x7e00u | ((x >> 13) & 0x1ffu);
    if (x >= 0x47800000u) /* 65536 and up, infinity included */
        return sign | 0x7c00u;
    if (x >= 0x38800000u) { /* at least 2^-14: a normal half unless the rounding carries into infinity */
        uint32_t h = (((x >> 23) - 112u) << 10) | ((x & 0x7fffffu) >> 13);
        const uint32_t rem = x & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u)))
            ++h;
        return sign | h;
    }
    if (x < 0x33000000u) /* below 2^-25: nearer to zero than to the smallest subnormal (2^-25 itself ties to even) */
        return sign;
    {
        const uint32_t mant = (x & 0x7fffffu) | 0x800000u;
        const unsigned shift = 126u - (x >> 23); /* 14 .. 24: the result counts units of 2^-24 */
        uint32_t h = mant >> shift;
        const uint32_t rem = mant & ((1u << shift) - 1u), halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (h & 1u)))
            ++h;
        return sign | h;
    }
}

/* float -> bfloat16 (the upper half of the float), round to nearest even; a NaN keeps its
 * upper half and becomes quiet. */
unsigned oracle_f32_to_bf16_bits(float f)
{
    union { float f; uint32_t u; } v;
    v.f = f;
    if ((v.u & 0x7fffffffu) > 0x7f800000u)
        return (v.u >> 16) | 0x0040u;
    return (v.u + 0x7fffu + ((v.u >> 16) & 1u)) >> 16;
}

/* n floats to half (kind 2) or bfloat16 (kind 3) bit patterns. */
void oracle_convert_f32(const float *src, unsigned short *dst, size_t n, int kind)
{
    for (size_t i = 0; i < n; ++i)
        dst[i] = (unsigned short)(kind == 2 ? oracle_f32_to_f16_bits(src[i]) : oracle_f32_to_bf16_bits(src[i]));
}

/* The epilogue of int4linear_linear_s32 / _f32 / _f16 / _bf16, applied in place to a finished
 * int32 product y (m x n): v = y[i][j] + bias[j] (two's-complement wrap), and for out != 0
 * t = ((float)v * row_scale[i]) * col_scale[j].  Null operands count as 0 / 1.
 * Compiled without floating-point contraction; the two products round separately.
 * `out`: 0 int32 (v), 1 float32 (the bits of t), 2 half, 3 bfloat16 (t rounded once more; the
 * 16 bits in the low half of the int). */
void oracle_epilogue(int *y, int m, int n, const int *bias, const float *row_scale,
                     const float *col_scale, int out)
{
    for (int i = 0; i < m; ++i) {
        const float rs = row_scale ? row_scale[i] : 1.0f;
        for (int j = 0; j < n; ++j) {
            const uint32_t sum = (uint32_t)y[(size_t)i * n + j] + (uint32_t)(bias ? bias[j] : 0);
            int v = (int)sum;
            if (out) {
                volatile float a = (float)v * rs;  /* volatile: no fused or reassociated product */
                const float f = a * (col_scale ? col_scale[j] : 1.0f);
                union { float f; int i; } u;
                u.f = f;
                v = out == 2 ? (int)oracle_f32_to_f16_bits(f) : out == 3 ? (int)oracle_f32_to_bf16_bits(f) : u.i;
            }
            y[(size_t)i * n + j] = v;
        }
    }
}
