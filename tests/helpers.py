"""Shared test helpers: seeded inputs, packing, and the C-ABI call wrapper."""
from __future__ import annotations

import numpy as np

from oracle import loader as oracle


def uniform_s4(seed: int, rows: int, cols: int) -> np.ndarray:
    """Uniform integers in [-8, 7], int8, from a fixed seed."""
    rng = np.random.default_rng(seed)
    return rng.integers(-8, 8, size=(rows, cols), dtype=np.int8)


def normal_s4(seed: int, rows: int, cols: int, sigma: float = 2.0) -> np.ndarray:
    """normal(0, sigma) rounded to nearest and clamped to [-8, 7] (decode activations)."""
    rng = np.random.default_rng(seed)
    v = np.rint(rng.normal(0.0, sigma, size=(rows, cols)))
    return np.clip(v, -8, 7).astype(np.int8)


def pack_bytes(values: np.ndarray) -> np.ndarray:
    """(m, k) int8/int32 in [-8,7] with k % 2 == 0 -> (m, k/2) uint8, low nibble = even k.
    Vectorised numpy restatement of the byte view of the packer; checked against the
    oracle's pack in the CPU tests."""
    v = values.astype(np.uint8) & 0xF
    return (v[:, 0::2] | (v[:, 1::2] << 4)).astype(np.uint8)


def pack_words_as_bytes(values: np.ndarray) -> np.ndarray:
    """Same bytes via the oracle's word packer (little-endian host)."""
    return oracle.pack(values.astype(np.int32)).view(np.uint8)


def exact_matmul(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """Independent implementation: float64 BLAS product, exact while |sum| < 2^53."""
    y = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.all(np.abs(y) < 2.0 ** 31)
    return y.astype(np.int64).astype(np.int32)


GUARD_WORDS = 16384  # int32 words of poison kept before and after C


def run_gemm(xp: np.ndarray, wp: np.ndarray, m: int, n: int, k: int, kernel: str = "auto",
             poison: int = 0x5A5A5A5A, keep_on_device: bool = False):
    """Copy packed operands to the device, run the C-ABI GEMM, return C as numpy int32
    (or the device tensor).  C sits between two guard zones and everything is pre-filled
    with a poison value, so untouched outputs and out-of-bounds writes are both caught."""
    import torch

    import int4linear_amd as lib

    dev = torch.device("cuda:0")
    xd = torch.from_numpy(np.ascontiguousarray(xp).view(np.uint8).reshape(-1)).to(dev)
    wd = torch.from_numpy(np.ascontiguousarray(wp).view(np.uint8).reshape(-1)).to(dev)
    buf = torch.full((2 * GUARD_WORDS + m * n,), poison, dtype=torch.int32, device=dev)
    yd = buf[GUARD_WORDS:GUARD_WORDS + m * n].view(m, n)
    lib.gemm_s4s4s32(xd, wd, yd, m, n, k, kernel=kernel)
    torch.cuda.synchronize()
    assert bool((buf[:GUARD_WORDS] == poison).all()), "write before the start of C"
    assert bool((buf[GUARD_WORDS + m * n:] == poison).all()), "write past the end of C"
    if keep_on_device:
        return yd
    return yd.cpu().numpy()


def to_device_bytes(packed: np.ndarray):
    import torch

    return torch.from_numpy(np.ascontiguousarray(packed).view(np.uint8).reshape(-1)).to("cuda:0")


def check_half_width_outputs(xd, wd, want: np.ndarray, bias: np.ndarray, rs: np.ndarray, cs: np.ndarray,
                             m: int, n: int, k: int, kernel: str = "auto") -> None:
    """linear_f16 / linear_bf16 on device operands against the oracle's epilogue of the int32
    product `want`, bit for bit, with the row scales shrunk so that most outputs stay inside
    the half range; the elements behind the m x n outputs must stay untouched."""
    import torch

    import int4linear_amd as lib

    rs_small = (rs * np.float32(2.0 ** -9)).astype(np.float32)
    bd, rd, cd = (torch.from_numpy(a).to("cuda:0") for a in (bias, rs_small, cs))
    for kind, fn in (("f16", lib.linear_f16), ("bf16", lib.linear_bf16)):
        y16 = torch.full((m * n + 256,), 0x7BAD, dtype=torch.int16, device="cuda:0")
        fn(xd, wd, bd, rd, cd, y16, m, n, k, kernel=kernel)
        got = y16.cpu().numpy().view(np.uint16)
        assert np.array_equal(got[:m * n].reshape(m, n), oracle.epilogue(want, bias, rs_small, cs, out=kind)), f"{kind} {kernel}"
        assert np.all(got[m * n:] == 0x7BAD), f"{kind} {kernel}: wrote past the output"


def special_floats(seed: int) -> np.ndarray:
    """Floats on which a conversion to half or bfloat16 is most likely to go wrong: every half
    value, the midpoints between neighbouring halves and bfloat16s and the floats next to them,
    the ends of both ranges, denormals, infinities, NaNs of both signs with several payloads,
    and random bit patterns."""
    rng = np.random.default_rng(seed)
    h = np.arange(0x10000, dtype=np.uint16).view(np.float16).astype(np.float32)
    hs = np.sort(np.unique(h[np.isfinite(h)]))
    mid = ((hs[:-1].astype(np.float64) + hs[1:].astype(np.float64)) / 2).astype(np.float32)
    near = np.concatenate([np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])
    b = (np.arange(0x10000, dtype=np.uint32) << 16)
    bf_ties = b | 0x8000
    bf_near = np.concatenate([b | 0x7FFF, b | 0x8001, b | 0xFFFF, b | 0x0001])
    edge = np.array([65504.0, 65519.99, 65520.0, 65520.01, 65536.0, 1e6, 3.4e38, np.inf, 2.0**-24, 2.0**-25,
                     np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-26, 0.0], dtype=np.float32)
    nans = np.array([0x7FC00000, 0xFFC00000, 0x7FC12345, 0xFFC54321, 0x7FE00000, 0x7FFFFFFF, 0xFFFFFFFF], dtype=np.uint32)
    rnd = rng.integers(0, 2**32, size=100000, dtype=np.uint64).astype(np.uint32)
    return np.concatenate([h, mid, near, bf_ties.view(np.float32), bf_near.view(np.float32), edge, -edge,
                           nans.view(np.float32), rnd.view(np.float32)])
