"""int4linear_gemm_s4s4s32_static: the entry point that allocates nothing.

Its scratch memory is a fixed array inside the library's device image; these tests call it
through the C ABI and compare its output bit for bit with int4linear_gemm_s4s4s32 (the
entry point it is a variant of, which allocates its workspace) on calls in a row that
reuse the array, the second always with a smaller input than the first.
"""
from __future__ import annotations

import ctypes

import numpy as np
import pytest

from tests.helpers import pack_bytes, to_device_bytes, uniform_s4

pytestmark = pytest.mark.gpu

POISON = 0x5A5A5A5A


def _run_pair(lib, torch, m, n, k, seed):
    """The same problem through both entry points; returns the two results (device)."""
    xd = to_device_bytes(pack_bytes(uniform_s4(seed, m, k)))
    wd = to_device_bytes(pack_bytes(uniform_s4(seed + 1, n, k)))
    want = torch.full((m, n), POISON, dtype=torch.int32, device="cuda:0")
    got = torch.full((m, n), POISON, dtype=torch.int32, device="cuda:0")
    lib.gemm_s4s4s32(xd, wd, want, m, n, k)
    lib.gemm_s4s4s32_static(xd, wd, got, m, n, k)
    torch.cuda.synchronize()
    return got, want


# (first call, second smaller call): both of a pair use the scratch array.
#   FP6 kernel: converted operands (and split-K slabs) live in the scratch array;
#   int8 split-K forms: partial sums live there.
PAIRS = [
    ("fp6 then smaller fp6", (4096, 4096, 4096), "fp6", (2304, 4096, 3072), "fp6"),
    ("fp6 then int8 split-K", (2048, 8192, 8192), "fp6", (128, 4096, 14336), "mfma"),
    ("int8 split-K, 128^2 then 64^2 slices", (512, 4096, 14336), "mfma", (200, 136, 16384), "mfma"),
    ("fp6 with ragged K then a tiny one", (1000, 3000, 4104), "fp6", (40, 56, 4104), "fp6"),
    ("decode split over K, then a smaller one", (64, 4096, 14336), "skinny", (40, 2000, 16384), "skinny"),
]


@pytest.mark.parametrize("name,first,first_kernel,second,second_kernel", PAIRS, ids=[p[0] for p in PAIRS])
def test_static_matches_allocating_entry(gpu, name, first, first_kernel, second, second_kernel):
    import torch

    import int4linear_amd as lib

    for i, (shape, kernel) in enumerate(((first, first_kernel), (second, second_kernel))):
        m, n, k = shape
        assert lib.kernel_for_shape(m, n, k) == kernel, (shape, lib.kernel_for_shape(m, n, k))
        if kernel == "mfma":  # only the split-K forms of the int8 kernel use scratch memory
            assert lib.workspace_bytes(m, n, k) > 0, shape
        assert 0 < lib.workspace_bytes(m, n, k) <= lib.api.STATIC_SCRATCH_BYTES, shape
        print(f"static entry call {i}: shape {shape} kernel {kernel}", flush=True)
        got, want = _run_pair(lib, torch, m, n, k, seed=100 + 10 * i)
        assert not bool((want == POISON).all())
        assert torch.equal(got, want), f"{name}: call {i} {shape} differs from int4linear_gemm_s4s4s32"


def test_static_kernels_without_scratch(gpu):
    """Shapes whose kernel needs no scratch run through the same entry point."""
    import torch

    import int4linear_amd as lib

    for shape in ((16, 4096, 4096), (300, 520, 512), (33, 70, 40), (5, 7, 0)):
        m, n, k = shape
        print(f"static entry, no scratch: shape {shape}", flush=True)
        got, want = _run_pair(lib, torch, m, n, k, seed=7)
        assert torch.equal(got, want), shape


def test_static_falls_back_or_rejects_oversize(gpu):
    """A shape whose fast kernel would need more scratch than the array holds runs on the
    kernels that need none (as under graph capture); only when that would leave a large
    problem to the scalar kernel (K not a multiple of 128) is it refused, with status 7, before
    anything is enqueued and with the output left alone."""
    import torch

    import int4linear_amd as lib
    from int4linear_amd import _lib

    m, n, k = 12288, 12288, 8192  # FP6 operands: 144 MiB
    assert lib.kernel_for_shape(m, n, k) == "fp6"
    assert lib.workspace_bytes(m, n, k) > lib.api.STATIC_SCRATCH_BYTES
    g = torch.Generator(device="cuda:0")
    g.manual_seed(77)
    xd = torch.randint(0, 256, (m * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
    wd = torch.randint(0, 256, (n * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
    want = torch.full((m, n), POISON, dtype=torch.int32, device="cuda:0")
    got = torch.full((m, n), POISON, dtype=torch.int32, device="cuda:0")
    lib.gemm_s4s4s32(xd, wd, want, m, n, k)
    lib.gemm_s4s4s32_static(xd, wd, got, m, n, k)   # the int8 kernel: no scratch
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    del want, got

    k = 8200  # K % 128 != 0: only the FP6 kernel is fast, and its operands do not fit
    assert lib.kernel_for_shape(m, n, k) == "fp6"
    assert lib.workspace_bytes(m, n, k) > lib.api.STATIC_SCRATCH_BYTES
    xd = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda:0")
    wd = torch.zeros(n * k // 2, dtype=torch.uint8, device="cuda:0")
    yd = torch.full((m, n), POISON, dtype=torch.int32, device="cuda:0")
    raw = _lib.load()
    st = raw.int4linear_gemm_s4s4s32_static(xd.data_ptr(), wd.data_ptr(), yd.data_ptr(), m, n, k,
                                            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert st == 7, st
    assert b"scratch" in raw.int4linear_status_string(st)
    assert bool((yd == POISON).all())
    with pytest.raises(lib.Int4LinearError):
        lib.gemm_s4s4s32_static(xd, wd, yd, m, n, k)


def test_static_entry_in_a_graph(gpu):
    """What the entry point is for: captured in a HIP graph and replayed three times with new
    operand contents and eager work between the replays, each replay checked against the
    eager result of the allocating entry point."""
    import torch

    import int4linear_amd as lib

    shapes = [(2304, 4096, 3072), (128, 4096, 14336), (64, 4096, 14336)]  # FP6 kernel; int8 split over K; decode split over K
    lib.init()  # set-up does not belong inside a capture (a first call there is refused)
    bufs = []
    for (m, n, k) in shapes:
        bufs.append((torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda:0"),
                     torch.zeros(n * k // 2, dtype=torch.uint8, device="cuda:0"),
                     torch.zeros((m, n), dtype=torch.int32, device="cuda:0"),
                     torch.zeros((m, n), dtype=torch.int32, device="cuda:0")))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for (m, n, k), (xd, wd, yd, _) in zip(shapes, bufs):
            lib.gemm_s4s4s32_static(xd, wd, yd, m, n, k)
    g = torch.Generator(device="cuda:0")
    for rep in range(3):
        g.manual_seed(900 + rep)
        for (m, n, k), (xd, wd, yd, ref) in zip(shapes, bufs):
            xd.copy_(torch.randint(0, 256, xd.shape, dtype=torch.uint8, device="cuda:0", generator=g))
            wd.copy_(torch.randint(0, 256, wd.shape, dtype=torch.uint8, device="cuda:0", generator=g))
            yd.fill_(POISON)
            lib.gemm_s4s4s32(xd, wd, ref, m, n, k)
        torch.cuda.synchronize()
        print(f"static entry, graph replay {rep}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        for shape, (_, _, yd, ref) in zip(shapes, bufs):
            assert torch.equal(yd, ref), f"{shape}, replay {rep}"
