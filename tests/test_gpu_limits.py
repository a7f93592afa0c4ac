"""GPU tests at the edges of what the library advertises: the largest K each kernel's
arithmetic is exact for, and operands and outputs beyond 2^31 bytes / elements.

Expected values are closed forms (constant operands: per-output sum = a * b * K), the CPU
oracle (test/test_correctness.cu:12-19 restated: int32 accumulation is the contract), or the
scalar kernel on the device, which indexes in 64 bits and accumulates in int32."""
import numpy as np
import pytest

from oracle import loader as oracle
from tests import helpers

pytestmark = pytest.mark.gpu

FP6_MAX_K = (1 << 18) - 128      # fp6_supports: |sum| <= 64 * K stays below 2^24
INT8_MAX_K = 131071 - 127        # mfma_supports / skinny_supports: 256 * |sum| stays below 2^31


def _const_packed(rows, k, value):
    byte = (value & 0xF) | ((value & 0xF) << 4)
    return np.full((rows, k // 2), byte, dtype=np.uint8)


# ---- exactness at the largest K ---------------------------------------------------------

@pytest.mark.parametrize("a, b", [(-8, -8), (-8, 7), (7, 7)])
def test_fp6_exact_at_largest_k_constants(gpu, a, b):
    """fp32 accumulation of multiples of 1/64: the largest sums the kernel accepts
    (64 * 262016 = 16 769 024 = 2^24 - 8192)."""
    m = n = 256
    k = FP6_MAX_K
    print(f"fp6 constants a={a} b={b} K={k}", flush=True)
    got = helpers.run_gemm(_const_packed(m, k, a), _const_packed(n, k, b), m, n, k, kernel="fp6")
    assert int(got.min()) == a * b * k and int(got.max()) == a * b * k, (got.min(), got.max(), a * b * k)


@pytest.mark.parametrize("big_first", [True, False])
def test_fp6_small_addends_next_to_a_large_accumulator(gpu, host_threads, big_first):
    """Most of K contributes 64 per element (both operands -8), the rest products of every
    size down to 1: the 1/64 addends meet an accumulator of about 2^18 (big part first) or the
    large partial sums meet a small odd accumulator (big part last).  Checked against the CPU
    oracle and the scalar kernel."""
    import torch

    m = n = 256
    k = FP6_MAX_K
    small = 1536
    rng = np.random.default_rng(77 + big_first)
    x = np.full((m, k), -8, dtype=np.int8)
    w = np.full((n, k), -8, dtype=np.int8)
    xs = rng.integers(-8, 8, size=(m, small), dtype=np.int8)
    ws = rng.integers(-8, 8, size=(n, small), dtype=np.int8)
    xs[:, :256] = 1          # a run of 1 * (-1, 0, 1): the smallest addends
    ws[:, :256] = rng.integers(-1, 2, size=(n, 256), dtype=np.int8)
    if big_first:
        x[:, k - small:], w[:, k - small:] = xs, ws
    else:
        x[:, :small], w[:, :small] = xs, ws
    want = oracle.linear_ref(x, w, threads=host_threads)
    assert np.array_equal(want, 64 * (k - small) + oracle.linear_ref(xs, ws, threads=host_threads))
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    print(f"fp6 mixed magnitudes big_first={big_first} K={k}", flush=True)
    got = helpers.run_gemm(xp, wp, m, n, k, kernel="fp6")
    assert np.array_equal(got, want)
    ref = helpers.run_gemm(xp, wp, m, n, k, kernel="simple")
    assert np.array_equal(ref, want)


def test_fp6_random_long_k(gpu):
    """Random data at K = 131072 (sums of either sign, partial sums wandering through many
    binades) against the scalar kernel on the device."""
    import torch

    m, n, k = 384, 512, 131072
    g = torch.Generator(device="cuda:0")
    g.manual_seed(131072)
    x = torch.randint(0, 256, (m * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
    w = torch.randint(0, 256, (n * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
    import int4linear_amd as lib

    got = torch.full((m, n), 0x5A5A5A5A, dtype=torch.int32, device="cuda:0")
    ref = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
    print("fp6 random K=131072", flush=True)
    lib.gemm_s4s4s32(x, w, got, m, n, k, kernel="fp6")
    lib.gemm_s4s4s32(x, w, ref, m, n, k, kernel="simple")
    torch.cuda.synchronize()
    assert torch.equal(got, ref)


@pytest.mark.parametrize("kernel, m, k", [
    ("mfma", 256, INT8_MAX_K), ("mfma", 2048, INT8_MAX_K), ("mfma128", 300, INT8_MAX_K),
    ("mfma256", 300, INT8_MAX_K), ("auto", 256, INT8_MAX_K), ("auto", 16, INT8_MAX_K),
    # the weight-streaming kernel: K in 128-byte tiles (511 of them, a ragged split in eight
    # passes) and the largest K, which is not (its fallback form)
    ("skinny", 16, INT8_MAX_K - 128), ("skinny", 64, INT8_MAX_K - 128), ("skinny", 16, INT8_MAX_K),
    ("skinny", 64, INT8_MAX_K),
])
def test_int8_exact_at_largest_k(gpu, kernel, m, k):
    """The int8 kernels accumulate 256 * sum: all -8 at K = 130944 gives 8 380 416 per output,
    2 145 386 496 in the accumulator -- the largest value the kernels accept; A = -8, B = 7 is
    the most negative one."""
    n = 384
    for a, b in ((-8, -8), (-8, 7)):
        print(f"int8 constants kernel={kernel} m={m} a={a} b={b} K={k}", flush=True)
        got = helpers.run_gemm(_const_packed(m, k, a), _const_packed(n, k, b), m, n, k, kernel=kernel)
        assert int(got.min()) == a * b * k and int(got.max()) == a * b * k, (kernel, got.min(), got.max())


def test_k_beyond_the_fast_kernels(gpu):
    """Past those bounds an explicit request is refused and the automatic dispatch still
    answers (on the scalar kernel, exact for as long as the sum fits int32)."""
    import int4linear_amd as lib

    m, n = 16, 32
    k = FP6_MAX_K + 128
    xp, wp = _const_packed(m, k, -8), _const_packed(n, k, 7)
    for kern in ("fp6", "mfma", "skinny"):
        with pytest.raises(lib.Int4LinearError) as err:
            helpers.run_gemm(xp, wp, m, n, k, kernel=kern)
        assert err.value.status == 5, kern
    assert lib.kernel_for_shape(m, n, k) == "simple"
    got = helpers.run_gemm(xp, wp, m, n, k, kernel="auto")
    assert int(got.min()) == -56 * k and int(got.max()) == -56 * k


# ---- beyond 2^31 ------------------------------------------------------------------------

def _device_pair(torch, lib, m, n, k, seed, kernels):
    """Random operands made on the device; every kernel's whole output against the scalar
    kernel's, compared on the device."""
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    x = torch.randint(0, 256, (m * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
    w = torch.randint(0, 256, ((n * k) // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
    ref = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
    print(f"reference (scalar kernel) {(m, n, k)}", flush=True)
    lib.gemm_s4s4s32(x, w, ref, m, n, k, kernel="simple")
    torch.cuda.synchronize()
    for kern in kernels:
        got = torch.full((m, n), 0x5A5A5A5A, dtype=torch.int32, device="cuda:0")
        print(f"kernel {kern} {(m, n, k)}", flush=True)
        lib.gemm_s4s4s32(x, w, got, m, n, k, kernel=kern)
        torch.cuda.synchronize()
        assert torch.equal(got, ref), f"{kern} {(m, n, k)}"
        del got
    del ref, x, w
    torch.cuda.empty_cache()


def test_weights_larger_than_2_gib_streaming_form(gpu):
    """Decode against 2.29 GiB of weights: the resident-workgroup form of the weight-streaming
    kernel, whose lanes address W with unsigned 32-bit byte offsets."""
    import torch

    import int4linear_amd as lib

    m, n, k = 16, 300000, 16384
    assert n * (k // 2) > 2 ** 31
    assert lib.kernel_for_shape(m, n, k) == "skinny"
    _device_pair(torch, lib, m, n, k, seed=31, kernels=("auto", "skinny"))


def test_weights_larger_than_4_gib(gpu):
    """4.6 GiB of weights: past the 32-bit lane offsets of the resident form, so the first form
    of the weight-streaming kernel (64-bit base per workgroup) takes it; also 33 rows of X."""
    import torch

    import int4linear_amd as lib

    n, k = 600000, 16384
    assert n * (k // 2) > 2 ** 32
    for m in (16, 33):
        assert lib.kernel_for_shape(m, n, k) == "skinny"
        _device_pair(torch, lib, m, n, k, seed=32 + m, kernels=("auto",))


def test_output_larger_than_2_31_elements(gpu):
    """C with 2.15 * 10^9 elements (8.6 GB): every MFMA kernel's store addressing."""
    import torch

    import int4linear_amd as lib

    m = n = 46400
    k = 128
    assert m * n > 2 ** 31
    _device_pair(torch, lib, m, n, k, seed=33, kernels=("auto", "mfma", "mfma128", "mfma256", "fp6"))


def test_more_rows_than_one_grid_of_the_scalar_kernel(gpu):
    """M beyond 65535 * 16 rows: the scalar kernel runs as several launches."""
    m, n, k = 65535 * 16 + 40, 24, 8
    got = helpers.run_gemm(_const_packed(m, k, -8), _const_packed(n, k, 7), m, n, k, kernel="simple")
    assert got.shape == (m, n) and int(got.min()) == -56 * k and int(got.max()) == -56 * k
    got = helpers.run_gemm(_const_packed(m, k, 3), _const_packed(n, k, 5), m, n, k, kernel="auto")
    assert int(got.min()) == 15 * k and int(got.max()) == 15 * k
