"""Pins oracle_linear_ref (restating test/test_correctness.cu:12-19) and oracle_is_same
(:22-27) with checks that do not retype its formula: committed golden products, an
independent float64 BLAS product, closed forms, algebraic invariants and a pure-Python
brute force.  A dropped term, a wrong sign or index, or a transposed operand fails at
least one of them."""
import numpy as np
import pytest

from oracle import loader as oracle
from tests import helpers

GOLDEN = np.load(helpers.__file__.replace("helpers.py", "golden/int4_gemm_golden.npz"))


def test_golden_products():
    for idx, (m, n, k) in enumerate(GOLDEN["shapes"]):
        y = oracle.linear_ref(GOLDEN[f"x{idx}"], GOLDEN[f"w{idx}"])
        assert y.shape == (m, n)
        assert np.array_equal(y, GOLDEN[f"y{idx}"]), f"case {idx} {(m, n, k)}"


@pytest.mark.parametrize("m, n, k, seed", [(64, 96, 256, 1), (37, 53, 1000, 2), (128, 128, 1024, 3)])
def test_against_blas_float64(m, n, k, seed):
    x = helpers.uniform_s4(seed, m, k)
    w = helpers.uniform_s4(seed + 100, n, k)
    assert np.array_equal(oracle.linear_ref(x, w), helpers.exact_matmul(x, w))


def test_threaded_variant_matches_single_thread():
    x = helpers.uniform_s4(5, 50, 512)
    w = helpers.uniform_s4(6, 70, 512)
    assert np.array_equal(oracle.linear_ref(x, w, threads=4), oracle.linear_ref(x, w))


@pytest.mark.parametrize("a, b, per_k", [(-8, -8, 64), (7, 7, 49), (-8, 7, -56), (1, -1, -1)])
def test_constant_operands(a, b, per_k):
    m, n, k = 5, 6, 4096
    y = oracle.linear_ref(np.full((m, k), a), np.full((n, k), b))
    assert np.all(y == per_k * k)


def test_all_minus_eight_at_k_8192_is_524288():
    y = oracle.linear_ref(np.full((2, 8192), -8), np.full((3, 8192), -8))
    assert np.all(y == 524288)


def test_one_hot_rows_select_columns():
    # W[j] = delta(l, k_j)  =>  C[i][j] = A[i][k_j]; pins the k index and the B-row index.
    m, n, k = 9, 11, 64
    x = helpers.uniform_s4(8, m, k).astype(np.int32)
    kj = (np.arange(n) * 7 + 3) % k
    w = np.zeros((n, k), dtype=np.int32)
    w[np.arange(n), kj] = 1
    assert np.array_equal(oracle.linear_ref(x, w), x[:, kj])


def test_ones_give_row_sums():
    n, k = 13, 200
    w = helpers.uniform_s4(9, n, k).astype(np.int32)
    y = oracle.linear_ref(np.ones((4, k), dtype=np.int32), w)
    assert np.array_equal(y, np.tile(w.sum(axis=1), (4, 1)))


def test_invariants():
    m, n, k = 12, 10, 96
    x = helpers.uniform_s4(10, m, k).astype(np.int32)
    x2 = helpers.uniform_s4(11, m, k).astype(np.int32)
    w = helpers.uniform_s4(12, n, k).astype(np.int32)
    y = oracle.linear_ref(x, w)
    # linear in A
    assert np.array_equal(oracle.linear_ref(x + x2, w), y + oracle.linear_ref(x2, w))
    # the same K permutation on both operands changes nothing
    perm = np.random.default_rng(13).permutation(k)
    assert np.array_equal(oracle.linear_ref(x[:, perm], w[:, perm]), y)
    # swapping operands transposes the result
    assert np.array_equal(oracle.linear_ref(w, x), y.T)
    # permuting rows of A / rows of B permutes rows / columns of C
    pr, pc = np.random.default_rng(14).permutation(m), np.random.default_rng(15).permutation(n)
    assert np.array_equal(oracle.linear_ref(x[pr], w[pc]), y[pr][:, pc])


@pytest.mark.parametrize("m, n, k", [(1, 1, 8), (2, 3, 8), (3, 2, 24), (4, 4, 32)])
def test_brute_force_python(m, n, k):
    x = helpers.uniform_s4(20 + m, m, k)
    w = helpers.uniform_s4(30 + n, n, k)
    want = [[sum(int(x[i, l]) * int(w[j, l]) for l in range(k)) for j in range(n)] for i in range(m)]
    assert oracle.linear_ref(x, w).tolist() == want


def test_empty_k_gives_zeros():
    y = oracle.linear_ref(np.zeros((3, 0), dtype=np.int32), np.zeros((4, 0), dtype=np.int32))
    assert y.shape == (3, 4) and not y.any()


def test_is_same():
    a = np.arange(100, dtype=np.int32)
    b = a.copy()
    assert oracle.is_same(a, b)
    b[99] += 1
    assert not oracle.is_same(a, b)
    b[99] -= 1
    b[0] -= 1
    assert not oracle.is_same(a, b)


# ---- the linear layer's epilogue ---------------------------------------------------------

def test_epilogue_identities():
    rng = np.random.default_rng(11)
    y = rng.integers(-2**20, 2**20, size=(7, 13), dtype=np.int32)
    assert np.array_equal(oracle.epilogue(y), y)                                  # no operands: unchanged
    assert np.array_equal(oracle.epilogue(y, f32=True), y.astype(np.float32))    # scales of 1: the cast
    ones_r, ones_c = np.ones(7, np.float32), np.ones(13, np.float32)
    assert np.array_equal(oracle.epilogue(y, None, ones_r, ones_c, f32=True), y.astype(np.float32))


def test_epilogue_against_numpy():
    rng = np.random.default_rng(12)
    m, n = 33, 50
    y = rng.integers(-2**30, 2**30, size=(m, n), dtype=np.int32)
    bias = rng.integers(-2**30, 2**30, size=n, dtype=np.int32)
    # int32 bias add wraps like two's-complement hardware
    want = (y.astype(np.int64) + bias.astype(np.int64)).astype(np.uint64).astype(np.uint32).view(np.int32) \
        if False else ((y.astype(np.int64) + bias[None, :].astype(np.int64)) & 0xFFFFFFFF).astype(np.uint32).view(np.int32)
    assert np.array_equal(oracle.epilogue(y, bias), want.reshape(m, n))
    # scaled float output: cast rounds once, each product rounds once, row scale first
    rs = rng.uniform(0.001, 3.0, size=m).astype(np.float32)
    cs = rng.uniform(0.001, 3.0, size=n).astype(np.float32)
    v = want.reshape(m, n).astype(np.float32)
    wantf = (v * rs[:, None]) * cs[None, :]
    got = oracle.epilogue(y, bias, rs, cs, f32=True)
    assert got.dtype == np.float32 and np.array_equal(got.view(np.int32), wantf.view(np.int32))
    # only one of the scales
    assert np.array_equal(oracle.epilogue(y, None, rs, None, f32=True), y.astype(np.float32) * rs[:, None])
    assert np.array_equal(oracle.epilogue(y, None, None, cs, f32=True), y.astype(np.float32) * cs[None, :])


def _interesting_floats(rng):
    """Every float16 value as a float, every midpoint between float16 neighbours, the floats
    next to those midpoints, and random bit patterns (NaNs left out)."""
    h = np.arange(0x10000, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h)]
    hs = np.sort(np.unique(h))
    mid = ((hs[:-1].astype(np.float64) + hs[1:].astype(np.float64)) / 2).astype(np.float32)  # exact in float32
    near = np.concatenate([np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    big = np.array([65504.0, 65519.99, 65520.0, 65520.01, 65536.0, 1e6, 3.4e38, np.inf, 2.0**-24, 2.0**-25,
                    np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-26, 0.0], dtype=np.float32)
    big = np.concatenate([big, -big])
    rnd = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    rnd = rnd[~np.isnan(rnd)]
    return np.concatenate([h, mid, near, big, rnd])


def test_half_conversion_against_numpy():
    """float -> half as the epilogue rounds it: numpy's conversion (round to nearest even,
    overflow to infinity, gradual underflow) is the independent implementation."""
    v = _interesting_floats(np.random.default_rng(21))
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)
    got = oracle.convert_f32(v, "f16")
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:5]
    # quiet NaNs: sign and upper payload kept (numpy's rule as well)
    q = helpers.special_floats(24)
    q = q[np.isnan(q) & ((q.view(np.uint32) & 0x00400000) != 0)]
    assert len(q) > 100
    assert np.array_equal(oracle.convert_f32(q, "f16"), q.astype(np.float16).view(np.uint16))
    assert oracle.convert_f32(np.array([0x7F800001], np.uint32).view(np.float32), "f16")[0] == 0x7E00  # a signalling NaN comes out quiet


def test_bfloat16_conversion_against_torch():
    """float -> bfloat16: torch's CPU conversion is the independent implementation; the closed
    form (exactly representable values, ties to even on the 17th bit) is checked as well."""
    import torch

    v = _interesting_floats(np.random.default_rng(22))
    bits = v.view(np.uint32)
    ties = ((bits & 0xFFFF0000) | 0x8000).view(np.float32)       # exact halfway points
    v = np.concatenate([v, ties[np.isfinite(ties)]])
    want = torch.from_numpy(v.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.convert_f32(v, "bf16")
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:5]
    exact = (np.arange(0x7F80, dtype=np.uint32) << 16).view(np.float32)   # every finite bfloat16 value
    assert np.array_equal(oracle.convert_f32(exact, "bf16"), np.arange(0x7F80, dtype=np.uint16))
    # NaNs: the upper half with the quiet bit set
    q = helpers.special_floats(25)
    q = q[np.isnan(q)]
    assert np.array_equal(oracle.convert_f32(q, "bf16"), ((q.view(np.uint32) >> 16) | 0x40).astype(np.uint16))
    assert oracle.convert_f32(np.array([1.00390625], np.float32), "bf16")[0] == 0x3F80       # 1 + 2^-8 ties down to even
    assert oracle.convert_f32(np.array([1.01171875], np.float32), "bf16")[0] == 0x3F82       # 1 + 3 * 2^-8 ties up to even


def test_epilogue_half_width_outputs():
    rng = np.random.default_rng(23)
    m, n = 19, 37
    y = rng.integers(-2**22, 2**22, size=(m, n), dtype=np.int32)
    bias = rng.integers(-2**10, 2**10, size=n, dtype=np.int32)
    rs = rng.uniform(0.0001, 0.01, size=m).astype(np.float32)
    cs = rng.uniform(0.001, 3.0, size=n).astype(np.float32)
    f = oracle.epilogue(y, bias, rs, cs, out="f32")
    for kind in ("f16", "bf16"):
        got = oracle.epilogue(y, bias, rs, cs, out=kind)
        assert got.dtype == np.uint16 and got.shape == (m, n)
        assert np.array_equal(got, oracle.convert_f32(f, kind))
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.epilogue(y, bias, rs, cs, out="f16"), f.astype(np.float16).view(np.uint16))
