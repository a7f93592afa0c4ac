"""Writes tests/golden/int4_gemm_golden.npz: small seeded inputs with expected outputs.

The expected values come from implementations that share no code with the oracle or
the GPU library: pure-Python integer arithmetic for the packer words and the GEMM of the
tiny cases, numpy int64 einsum for the larger ones.  The reference repository holds no
fixtures of its own for this path, so these are the committed known-answer vectors.

Run from the repository root:  python tests/golden/make_golden.py
"""
from pathlib import Path

import numpy as np

OUT = Path(__file__).resolve().parent / "int4_gemm_golden.npz"

# (m, n, k, seed) -- k % 8 == 0 everywhere; some k % 128 == 0 so every GPU kernel is hit.
CASES = [
    (1, 1, 8, 11),
    (3, 5, 16, 12),
    (7, 9, 40, 13),
    (16, 16, 128, 14),
    (17, 33, 128, 15),
    (5, 70, 256, 16),
    (33, 18, 384, 17),
    (64, 48, 512, 18),
    (1, 40, 1024, 19),
    (130, 70, 128, 20),
]


def py_pack_words(row):
    """Word j of a row = OR_k (row[8j+k] & 0xF) << 4k, missing slots zero."""
    words = []
    for j in range((len(row) + 7) // 8):
        w = 0
        for s in range(8):
            if 8 * j + s < len(row):
                w |= (int(row[8 * j + s]) & 0xF) << (4 * s)
        words.append(w - (1 << 32) if w >= (1 << 31) else w)
    return words


def main():
    out = {}
    shapes = []
    for idx, (m, n, k, seed) in enumerate(CASES):
        rng = np.random.default_rng(seed)
        x = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
        w = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
        if m * n * k <= 20000:
            y = np.array([[sum(int(a) * int(b) for a, b in zip(x[i], w[j])) for j in range(n)]
                          for i in range(m)], dtype=np.int64)
        else:
            y = np.einsum("ik,jk->ij", x.astype(np.int64), w.astype(np.int64))
        assert np.abs(y).max() < 2 ** 31
        out[f"x{idx}"] = x
        out[f"w{idx}"] = w
        out[f"y{idx}"] = y.astype(np.int32)
        out[f"xwords{idx}"] = np.array([py_pack_words(r) for r in x], dtype=np.int32)
        shapes.append((m, n, k))
    out["shapes"] = np.array(shapes, dtype=np.int32)
    # Ragged packer vectors (n not a multiple of 8), including every nibble value.
    rag = np.array([[-8, -7, -6, -5, -4, -3, -2, -1, 0, 1], [2, 3, 4, 5, 6, 7, -1, -8, 7, -8]],
                   dtype=np.int32)
    out["ragged_values"] = rag
    out["ragged_words"] = np.array([py_pack_words(r) for r in rag], dtype=np.int32)
    np.savez_compressed(OUT, **out)
    print(OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
