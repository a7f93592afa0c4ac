"""Pins oracle_pack / oracle_unpack (restating utils/packer.cpp:3-31) without running any
GPU code: known-answer words, the byte-view closed form, round trips, the committed
golden words, and a bit-for-bit diff against the reference's own packer.cpp where
oracle/_ref has been built."""
import numpy as np
import pytest

from oracle import loader as oracle
from tests import helpers

GOLDEN = np.load(helpers.__file__.replace("helpers.py", "golden/int4_gemm_golden.npz"))


def u32(words):
    return [int(w) & 0xFFFFFFFF for w in np.asarray(words).ravel()]


@pytest.mark.parametrize("values, word", [
    ([0, 1, 2, 3, 4, 5, 6, 7], 0x76543210),           # slot k lands in bits [4k, 4k+4)
    ([-1] * 8, 0xFFFFFFFF),
    ([-8, 7, -8, 7, -8, 7, -8, 7], 0x78787878),
    ([-8] * 8, 0x88888888),
    ([1, 0, 0, 0, 0, 0, 0, 0], 0x00000001),           # element 0 is the LOW nibble
    ([0, 0, 0, 0, 0, 0, 0, -1], 0xF0000000),          # element 7 is the HIGH nibble
    ([16 + 3, -16 + 5, 0, 0, 0, 0, 0, 0], 0x00000053),  # only the low 4 bits are kept
])
def test_pack_known_words(values, word):
    assert u32(oracle.pack(np.array([values]))) == [word]


def test_pack_ragged_tail_is_zero_padded():
    # n = 10: the second word holds two nibbles and 24 zero bits (packer.cpp:10).
    words = oracle.pack(np.array([[1, 2, 3, 4, 5, 6, 7, -8, -1, -2]]))
    assert u32(words) == [0x87654321, 0x000000EF]


def test_pack_matches_committed_golden_words():
    for idx in range(len(GOLDEN["shapes"])):
        assert np.array_equal(oracle.pack(GOLDEN[f"x{idx}"]), GOLDEN[f"xwords{idx}"])
    assert np.array_equal(oracle.pack(GOLDEN["ragged_values"]), GOLDEN["ragged_words"])
    assert np.array_equal(oracle.unpack(GOLDEN["ragged_words"], 10), GOLDEN["ragged_values"])


@pytest.mark.parametrize("m, n", [(1, 8), (3, 64), (5, 128), (2, 24)])
def test_pack_byte_view(m, n):
    # byte e/2 = (v[e] & 0xF) | (v[e+1] & 0xF) << 4 on a little-endian host.
    v = helpers.uniform_s4(7, m, n)
    by = oracle.pack(v).view(np.uint8).reshape(m, -1)
    for i in range(m):
        for b in range(n // 2):
            assert by[i, b] == (int(v[i, 2 * b]) & 0xF) | ((int(v[i, 2 * b + 1]) & 0xF) << 4)
    assert np.array_equal(by, helpers.pack_bytes(v))


def test_unpack_sign_table():
    # nibble 0x0..0x7 -> 0..7, 0x8..0xF -> -8..-1 (packer.cpp:27)
    words = np.array([[0x76543210, 0xFEDCBA98 - (1 << 32)]], dtype=np.int64).astype(np.int32)
    got = oracle.unpack(words, 16)
    assert got.tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1]]


@pytest.mark.parametrize("n", [1, 2, 7, 8, 9, 15, 16, 17, 63, 64, 65, 130])
def test_roundtrip_all_values(n):
    m = 16
    v = (np.arange(m * n).reshape(m, n) * 5 + np.arange(m)[:, None]) % 16 - 8
    assert np.array_equal(oracle.unpack(oracle.pack(v), n), v)


@pytest.mark.parametrize("m, n, seed", [(1, 1, 1), (4, 8, 2), (5, 13, 3), (9, 100, 4), (33, 257, 5)])
def test_against_reference_packer(m, n, seed):
    ref = oracle.ref_packer()
    if ref is None:
        pytest.skip("oracle/_ref/libpacker_ref.so not built (reference tree absent)")
    rng = np.random.default_rng(seed)
    # arbitrary ints: the reference masks with 0xF, so must the oracle
    v = rng.integers(-1000, 1000, size=(m, n), dtype=np.int32)
    words = (n + 7) // 8
    ref_words = np.empty((m, words), dtype=np.int32)
    ref._Z4packPKiPiii(v.ctypes.data, ref_words.ctypes.data, m, n)
    assert np.array_equal(oracle.pack(v), ref_words)
    ref_vals = np.empty((m, n), dtype=np.int32)
    ref._Z6unpackPKiPiii(ref_words.ctypes.data, ref_vals.ctypes.data, m, n)
    assert np.array_equal(oracle.unpack(ref_words, n), ref_vals)
