// Host packer with the reference's signatures and layout (utils/packer.h:5-6,
// utils/packer.cpp:3-31): host arrays in, host arrays out.  This is the same host-side
// role the reference gives it -- preparing operands before they are copied to the
// device -- not a CPU stand-in for any device kernel.
#include "../../include/int4linear.h"

#include <cstddef>
#include <cstdint>

// Eight source ints per destination word; slot s of a word sits in bits [4s, 4s+4);
// a row of n values takes ceil(n/8) words and the unused slots of the last word are 0.
void pack(const int *src, int *dst, const int m, const int n)
{
    const int words = (n + 7) / 8;
    const int full = n / 8;
    for (int row = 0; row < m; ++row) {
        const int *s = src + (size_t)row * n;
        int *d = dst + (size_t)row * words;
        for (int w = 0; w < full; ++w, s += 8) {
            uint32_t v = 0;
            for (int t = 7; t >= 0; --t)
                v = (v << 4) | ((uint32_t)s[t] & 0xFu);
            d[w] = (int)v;
        }
        if (full < words) {
            uint32_t v = 0;
            for (int t = n - full * 8 - 1; t >= 0; --t)
                v = (v << 4) | ((uint32_t)s[t] & 0xFu);
            d[full] = (int)v;
        }
    }
}

// Inverse of pack: slot value 8..15 means -8..-1.
void unpack(const int *src, int *dst, const int m, const int n)
{
    const int words = (n + 7) / 8;
    for (int row = 0; row < m; ++row) {
        const int *s = src + (size_t)row * words;
        int *d = dst + (size_t)row * n;
        for (int col = 0; col < n; ++col) {
            const uint32_t v = (uint32_t)s[col >> 3] >> (4 * (col & 7));
            d[col] = (int)((v & 0xFu) ^ 8u) - 8;
        }
    }
}
