"""GPU parity tests: every kernel of the library, called through the C ABI, against the
CPU oracle on identical seeded inputs -- bit-exact int32.  Covers the five benchmark
configurations, the committed golden vectors, ragged and degenerate shapes, and
size-independent properties at full size."""
import numpy as np
import pytest

from oracle import loader as oracle
from tests import helpers

pytestmark = pytest.mark.gpu

GOLDEN = np.load(helpers.__file__.replace("helpers.py", "golden/int4_gemm_golden.npz"))


def kernels_for(m, n, k):
    ks = ["auto", "simple"]
    if k >= 8:
        ks.append("fp6")  # any K % 8 == 0: the converter pads K
    if k >= 128 and k % 128 == 0:
        ks += ["mfma", "mfma128", "mfma256"]
        if m <= 64:
            ks.append("skinny")
    return ks


def check_all_kernels(x, w, want=None, threads=1, kernels=None):
    m, k = x.shape
    n = w.shape[0]
    if want is None:
        want = oracle.linear_ref(x, w, threads=threads)
    xp, wp = helpers.pack_words_as_bytes(x), helpers.pack_words_as_bytes(w)
    for kern in kernels or kernels_for(m, n, k):
        got = helpers.run_gemm(xp, wp, m, n, k, kernel=kern)
        bad = np.argwhere(got != want)
        assert bad.size == 0, (f"kernel={kern} shape={(m, n, k)}: {len(bad)} mismatches, first at "
                               f"{tuple(bad[0])}: got {got[tuple(bad[0])]} want {want[tuple(bad[0])]}")


# ---- committed golden vectors ----------------------------------------------------------

@pytest.mark.parametrize("idx", range(len(GOLDEN["shapes"])))
def test_golden_vectors(gpu, idx):
    x, w, y = GOLDEN[f"x{idx}"], GOLDEN[f"w{idx}"], GOLDEN[f"y{idx}"]
    check_all_kernels(x, w, want=y)


# ---- configuration 1: 1024^3, full compare ---------------------------------------------

def test_cfg1_1024_cubed(gpu, host_threads):
    x = helpers.uniform_s4(1, 1024, 1024)
    w = helpers.uniform_s4(2, 1024, 1024)
    check_all_kernels(x, w, threads=host_threads)


# ---- configurations 2 and 3: large squares and the 2M = 2N = K family ------------------

@pytest.mark.parametrize("m, n, k", [
    (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 8192),
    (1024, 1024, 2048), (2048, 2048, 4096), (4096, 4096, 8192),
])
def test_cfg2_cfg3_large(gpu, host_threads, m, n, k):
    import torch

    x = helpers.uniform_s4(100 + m, m, k)
    w = helpers.uniform_s4(200 + k, n, k)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    got_d = helpers.run_gemm(xp, wp, m, n, k, kernel="auto", keep_on_device=True)
    # sampled rows against the CPU oracle
    rows = np.unique(np.concatenate([[0, 1, m - 1, 255, 256], np.random.default_rng(m + k).integers(0, m, 27)]))
    want = oracle.linear_ref(x[rows], w, threads=host_threads)
    got_rows = got_d[torch.from_numpy(rows).to(got_d.device)].cpu().numpy()
    assert np.array_equal(got_rows, want)
    # the whole matrix against the independent scalar kernel, on the device
    ref_d = helpers.run_gemm(xp, wp, m, n, k, kernel="simple", keep_on_device=True)
    assert torch.equal(got_d, ref_d)
    del got_d
    for kern in ("mfma", "fp6"):
        other = helpers.run_gemm(xp, wp, m, n, k, kernel=kern, keep_on_device=True)
        assert torch.equal(other, ref_d), kern
        del other


# ---- configuration 4: decode shapes ------------------------------------------------------

@pytest.mark.parametrize("n, k", [(4096, 4096), (14336, 4096), (4096, 14336)])
@pytest.mark.parametrize("m", [1, 16, 64])
def test_cfg4_decode(gpu, host_threads, m, n, k):
    x = helpers.normal_s4(300 + m, m, k)           # activations: normal(0, 2) -> [-8, 7]
    w = helpers.uniform_s4(400 + n + k, n, k)      # weights: uniform [-8, 7]
    want = oracle.linear_ref(x, w, threads=host_threads)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    for kern in ("auto", "skinny", "mfma", "fp6"):
        got = helpers.run_gemm(xp, wp, m, n, k, kernel=kern)
        assert np.array_equal(got, want), f"kernel={kern}"


# Every plan family of the weight-streaming kernel: tiles per wave 1..4, 1/2/4 row groups
# per workgroup (chosen from N against the CU count), 1..4 sixteen-row groups of X, the
# register-X variant (K = 14336), the fallback for K % 256 != 0 and for very long K.
@pytest.mark.parametrize("m, n, k", [
    (1, 5, 256), (7, 100, 512), (16, 4099, 768), (17, 7000, 1024), (33, 6600, 2048), (48, 333, 4096),
    (64, 4096, 8192), (16, 13200, 8192), (5, 6560, 12288), (32, 6556, 12288), (64, 1030, 16384),
    (16, 13112, 14336), (32, 6562, 14336), (40, 515, 14336), (9, 1000, 1920), (64, 200, 20480),
    (16, 14336, 4096 + 256), (3, 16, 4096),
    # more than 16 rows of X with several row groups per workgroup (X in registers)
    (64, 14336, 4096), (48, 14300, 4096), (32, 14336, 4096), (64, 4096, 2048), (33, 9000, 1024), (64, 14336, 512),
    (40, 14336, 6144), (64, 3000, 8192),
    # K covered in several passes
    (64, 4096, 14336), (32, 4100, 14336), (16, 14336, 14336), (64, 500, 20480), (8, 700, 32768), (48, 1000, 12288),
    # ... with several row groups of W and of X (later groups issued one ahead, in every pass)
    (32, 8200, 32768), (64, 8200, 20480), (48, 14336, 12288),
    # 33 to 64 rows of X, few rows of W per CU, long K: split four ways over K across workgroups under
    # automatic dispatch (whole row blocks, a ragged last one, fewer row blocks than a quarter of the CUs)
    (48, 4096, 14336), (33, 4000, 14336), (64, 3000, 14336), (64, 2048, 28672), (40, 2000, 16384), (50, 2100, 57344),
    # more than 64 rows of X: runs of 64, one launch each (only when the kernel is asked for by name)
    (65, 4096, 4096), (128, 14336, 4096), (100, 3000, 2048), (96, 14336, 512), (128, 600, 14336),
    (200, 520, 1024), (130, 20000, 4096),
    # K whose 128-byte tiles do not split evenly over the waves (43, 17, 74, 19, 23, 61, 5 tiles)
    (16, 4096, 11008), (64, 4096, 11008), (1, 300, 4352), (33, 3584, 18944), (48, 1000, 4864),
    (16, 14336, 5888), (64, 700, 15616), (100, 4096, 11008), (8, 50, 1280),
    # at most 16 rows of X against more than 64 rows of W per CU: the form whose workgroups stay on
    # their CU and stream W through wave-private rings (2 to 8 tiles for each of 7 to 16 waves)
    (16, 20480, 4096), (5, 21001, 3584), (16, 20480, 14336), (16, 33000, 5120), (3, 40001, 7168),
    (1, 21000, 6144), (9, 20481, 8192), (16, 20500, 28672), (2, 20490, 32768),
    # ... the same with 17 to 64 rows of X (seven or eight waves, widened X kept where it fits)
    (64, 32800, 4096), (33, 32768, 8192), (48, 33000, 3584), (17, 32770, 7168), (32, 32768, 14336),
    # ... and shapes with as many rows of W whose K does not qualify
    (16, 20500, 256), (7, 20481, 1024), (3, 40001, 2048), (64, 32768, 14336), (40, 33000, 5120),
])
def test_skinny_plans(gpu, host_threads, m, n, k):
    x = helpers.normal_s4(500 + m + k, m, k)
    w = helpers.uniform_s4(600 + n + k, n, k)
    want = oracle.linear_ref(x, w, threads=host_threads)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    for kern in ("skinny", "auto"):
        got = helpers.run_gemm(xp, wp, m, n, k, kernel=kern)
        bad = np.argwhere(got != want)
        assert bad.size == 0, f"kernel={kern}: {len(bad)} mismatches, first at {tuple(bad[0])}"


def test_decode_split_over_k_across_workgroups(gpu, host_threads):
    """The shapes of the weight-streaming kernel whose workgroups take a slice of K each and
    exchange partial sums through the workspace: two shapes in turn, new data every call (the
    arrival counters must be back at zero after every launch), on alternating streams without
    host synchronisation (the library orders users of the workspace), and under graph capture
    (no workspace there: the unsplit form, same result)."""
    import torch

    import int4linear_amd as lib

    shapes = [(64, 4096, 14336), (40, 2000, 16384)]
    for (m, n, k) in shapes:
        assert lib.kernel_for_shape(m, n, k) == "skinny" and lib.workspace_bytes(m, n, k) > 0, (m, n, k)
    assert lib.workspace_bytes(16, 4096, 14336) == 0 and lib.workspace_bytes(64, 4096, 8192) == 0
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    cases = []
    for i in range(6):
        m, n, k = shapes[i % 2]
        x = helpers.normal_s4(2100 + i, m, k)
        w = helpers.uniform_s4(2200 + i, n, k)
        cases.append((m, n, k, helpers.to_device_bytes(helpers.pack_bytes(x)), helpers.to_device_bytes(helpers.pack_bytes(w)),
                      torch.full((m, n), -1, dtype=torch.int32, device="cuda:0"), oracle.linear_ref(x, w, threads=host_threads)))
    torch.cuda.synchronize()
    for rep in range(3):
        for i, (m, n, k, xd, wd, yd, _) in enumerate(cases):
            lib.gemm_s4s4s32(xd, wd, yd, m, n, k, stream=streams[(i + rep) % 2].cuda_stream)
    torch.cuda.synchronize()
    for i, (m, n, k, _, _, yd, want) in enumerate(cases):
        assert np.array_equal(yd.cpu().numpy(), want), f"case {i} {(m, n, k)}"
    # captured: automatic dispatch must not touch the workspace
    m, n, k, xd, wd, yd, want = cases[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lib.gemm_s4s4s32(xd, wd, yd, m, n, k)
    for rep in range(2):
        yd.fill_(-1)
        lib.release_workspace()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(yd.cpu().numpy(), want), f"captured, replay {rep}"


@pytest.mark.parametrize("m, n, k", [(1024, 2048, 4096), (777, 33, 1152), (300, 520, 512)])
def test_epilogue_on_fp6_converted_operands(gpu, host_threads, m, n, k):
    """int4linear_linear_fp6_converted: the bias add and the scaled float / half / bfloat16
    outputs on caller-owned converted operands, bit for bit against the oracle's epilogue."""
    import torch

    import int4linear_amd as lib

    rng = np.random.default_rng(m * 7 + n)
    x = helpers.normal_s4(2300 + m, m, k)
    w = helpers.uniform_s4(2400 + n, n, k)
    prod = oracle.linear_ref(x, w, threads=host_threads)
    bias = rng.integers(-100000, 100000, size=n, dtype=np.int32)
    rs = (rng.uniform(0.01, 2.0, size=m) * 2.0 ** -9).astype(np.float32)
    cs = rng.uniform(0.01, 2.0, size=n).astype(np.float32)
    xd = helpers.to_device_bytes(helpers.pack_bytes(x))
    wd = helpers.to_device_bytes(helpers.pack_bytes(w))
    xc = torch.empty(lib.fp6_operand_bytes(m, k), dtype=torch.uint8, device="cuda:0")
    wc = torch.empty(lib.fp6_operand_bytes(n, k), dtype=torch.uint8, device="cuda:0")
    lib.fp6_convert(xd, xc, m, k)
    lib.fp6_convert(wd, wc, n, k)
    bd, rd, cd = (torch.from_numpy(a).to("cuda:0") for a in (bias, rs, cs))
    y = torch.full((m, n), 0x7BADBAD, dtype=torch.int32, device="cuda:0")
    lib.linear_fp6_converted(xc, wc, bd, None, None, y, "s32", m, n, k)
    assert np.array_equal(y.cpu().numpy(), oracle.epilogue(prod, bias)), "s32"
    lib.linear_fp6_converted(xc, wc, None, None, None, y, "s32", m, n, k)
    assert np.array_equal(y.cpu().numpy(), prod), "s32 without bias"
    yf = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    lib.linear_fp6_converted(xc, wc, bd, rd, cd, yf, "f32", m, n, k)
    assert np.array_equal(yf.cpu().numpy().view(np.int32), oracle.epilogue(prod, bias, rs, cs, f32=True).view(np.int32)), "f32"
    lib.linear_fp6_converted(xc, wc, None, rd, None, yf, "f32", m, n, k)
    assert np.array_equal(yf.cpu().numpy().view(np.int32), oracle.epilogue(prod, None, rs, None, f32=True).view(np.int32)), "f32 row scale"
    for kind in ("f16", "bf16"):
        y16 = torch.full((m * n + 256,), 0x7BAD, dtype=torch.int16, device="cuda:0")
        lib.linear_fp6_converted(xc, wc, bd, rd, cd, y16, kind, m, n, k)
        got = y16.cpu().numpy().view(np.uint16)
        assert np.array_equal(got[:m * n].reshape(m, n), oracle.epilogue(prod, bias, rs, cs, out=kind)), kind
        assert np.all(got[m * n:] == 0x7BAD), f"{kind}: wrote past the output"
    # an int32 output takes no scales; an unknown output type is refused
    with pytest.raises(lib.Int4LinearError) as refused:
        lib.linear_fp6_converted(xc, wc, bd, rd, None, y, "s32", m, n, k)
    assert refused.value.status == 5
    from int4linear_amd import _lib
    assert _lib.load().int4linear_linear_fp6_converted(xc.data_ptr(), wc.data_ptr(), None, None, None, y.data_ptr(), 4, m, n, k, None) == 5


def test_first_call_inside_a_capture_is_refused(gpu):
    """Set-up must not happen inside a graph capture: a process whose first library call comes
    while its stream is capturing gets INT4LINEAR_ERR_NOT_INITIALISED (and may call again after
    int4linear_init()).  Needs a process of its own: this one has set the device up long ago."""
    import subprocess
    import sys
    from pathlib import Path

    code = (
        "import sys, ctypes, torch\n"
        "sys.path.insert(0, %r)\n"
        "from int4linear_amd import _lib\n"
        "L = _lib.load()\n"
        "x = torch.zeros(16 * 512, dtype=torch.uint8, device='cuda:0'); w = torch.zeros(1024 * 512, dtype=torch.uint8, device='cuda:0')\n"
        "y = torch.zeros((16, 1024), dtype=torch.int32, device='cuda:0')\n"
        "torch.cuda.synchronize()\n"
        "s = torch.cuda.Stream()\n"
        "g = torch.cuda.CUDAGraph()\n"
        "with torch.cuda.graph(g, stream=s):\n"
        "    st = L.int4linear_gemm_s4s4s32(x.data_ptr(), w.data_ptr(), y.data_ptr(), 16, 1024, 1024, ctypes.c_void_p(s.cuda_stream))\n"
        "print('captured call:', st, L.int4linear_status_string(st).decode())\n"
        "assert st == 8, st\n"
        "assert L.int4linear_init() == 0\n"
        "g2 = torch.cuda.CUDAGraph()\n"
        "with torch.cuda.graph(g2, stream=s):\n"
        "    st = L.int4linear_gemm_s4s4s32(x.data_ptr(), w.data_ptr(), y.data_ptr(), 16, 1024, 1024, ctypes.c_void_p(s.cuda_stream))\n"
        "assert st == 0, st\n"
        "y.fill_(-1); g2.replay(); torch.cuda.synchronize()\n"
        "assert int(y.abs().sum()) == 0\n"
        "print('ok')\n"
    ) % str(Path(__file__).resolve().parent.parent)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "ok" in r.stdout, r.stdout + r.stderr


@pytest.mark.parametrize("m, n, k", [(300, 520, 512), (1, 1, 128), (1024, 2048, 4096), (777, 33, 1152)])
def test_fp6_converted_operands(gpu, host_threads, m, n, k):
    """Weights converted once, activations per call, GEMM on caller-owned buffers."""
    import torch

    import int4linear_amd as lib

    x = helpers.normal_s4(700 + m, m, k)
    w = helpers.uniform_s4(800 + n, n, k)
    want = oracle.linear_ref(x, w, threads=host_threads)
    xd = helpers.to_device_bytes(helpers.pack_bytes(x))
    wd = helpers.to_device_bytes(helpers.pack_bytes(w))
    xc = torch.full((lib.fp6_operand_bytes(m, k),), 0xA5, dtype=torch.uint8, device="cuda")
    wc = torch.full((lib.fp6_operand_bytes(n, k),), 0x5A, dtype=torch.uint8, device="cuda")
    y = torch.full((m, n), 0x7BADBAD, dtype=torch.int32, device="cuda")
    lib.fp6_convert(wd, wc, n, k)
    for _ in range(2):  # the converted weights are reused across calls
        lib.fp6_convert(xd, xc, m, k)
        lib.gemm_fp6_converted(xc, wc, y, m, n, k)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy(), want)
        y.fill_(-1)


@pytest.mark.parametrize("m, n, k", [(1000, 3000, 4104), (16, 4096, 4104), (300, 300, 1000), (257, 513, 40),
                                     (64, 2048, 2040), (512, 512, 136)])
def test_ragged_k_runs_on_the_fp6_kernel(gpu, host_threads, m, n, k):
    """K % 128 != 0 (K % 8 == 0): automatic dispatch pads K in the FP6 converter instead of
    falling back to the scalar kernel."""
    import int4linear_amd as lib

    x = helpers.uniform_s4(1000 + m, m, k)
    w = helpers.uniform_s4(1100 + n, n, k)
    want = oracle.linear_ref(x, w, threads=host_threads)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    assert lib.kernel_for_shape(m, n, k) == "fp6"
    for kern in ("auto", "fp6"):
        got = helpers.run_gemm(xp, wp, m, n, k, kernel=kern)
        assert np.array_equal(got, want), kern


# ---- epilogue: bias add and scaled float output, fused into every kernel's store ----------

@pytest.mark.parametrize("m, n, k, kernels", [
    (300, 520, 512, ("auto", "simple", "mfma128", "mfma256", "fp6")),
    (16, 1024, 1024, ("auto", "skinny", "mfma", "fp6")),
    (40, 515, 14336, ("skinny",)),
    (100, 4100, 4096, ("auto", "skinny")),   # two runs of rows of X: the row scales move with them
    (13, 20600, 4096, ("auto", "skinny")),   # the form for very many rows of W
    (50, 32790, 4096, ("auto", "skinny")),   # ... with several row groups of X
    (33, 70, 72, ("auto", "simple", "fp6")),
    (9, 1000, 1920, ("skinny",)),           # the fallback streaming kernel
    (2048, 2304, 1024, ("auto", "mfma")),   # 72 tiles of 256 x 256, several per workgroup
    (64, 4096, 14336, ("auto",)),           # decode split over K across workgroups: the last arrival applies the epilogue
    (40, 3000, 14336, ("auto", "skinny")),  # ... with a ragged last row block, against the unsplit form
])
def test_linear_with_epilogue(gpu, host_threads, m, n, k, kernels):
    import torch

    import int4linear_amd as lib

    rng = np.random.default_rng(m + n + k)
    x = helpers.normal_s4(1200 + m, m, k)
    w = helpers.uniform_s4(1300 + n, n, k)
    bias = rng.integers(-100000, 100000, size=n, dtype=np.int32)
    rs = rng.uniform(0.01, 2.0, size=m).astype(np.float32)
    cs = rng.uniform(0.01, 2.0, size=n).astype(np.float32)
    prod = oracle.linear_ref(x, w, threads=host_threads)
    want_s32 = oracle.epilogue(prod, bias)
    want_f32 = oracle.epilogue(prod, bias, rs, cs, f32=True)
    want_f32_nobias = oracle.epilogue(prod, None, rs, None, f32=True)
    xd = helpers.to_device_bytes(helpers.pack_bytes(x))
    wd = helpers.to_device_bytes(helpers.pack_bytes(w))
    bd, rd, cd = (torch.from_numpy(a).to("cuda:0") for a in (bias, rs, cs))
    rs_small = (rs * np.float32(2.0 ** -9)).astype(np.float32)   # keeps most outputs inside the half range
    rd_small = torch.from_numpy(rs_small).to("cuda:0")
    want_16 = {kind: oracle.epilogue(prod, bias, rs_small, cs, out=kind) for kind in ("f16", "bf16")}
    plain_16 = {kind: oracle.epilogue(prod, None, None, None, out=kind) for kind in ("f16", "bf16")}
    for kern in kernels:
        y = torch.full((m, n), 0x7BADBAD, dtype=torch.int32, device="cuda:0")
        lib.linear_s32(xd, wd, bd, y, m, n, k, kernel=kern)
        assert np.array_equal(y.cpu().numpy(), want_s32), f"s32 {kern}"
        lib.linear_s32(xd, wd, None, y, m, n, k, kernel=kern)
        assert np.array_equal(y.cpu().numpy(), prod), f"s32 without bias {kern}"
        yf = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
        lib.linear_f32(xd, wd, bd, rd, cd, yf, m, n, k, kernel=kern)
        # bit-exact: one rounding in the cast, one per product, same order as the oracle
        assert np.array_equal(yf.cpu().numpy().view(np.int32), want_f32.view(np.int32)), f"f32 {kern}"
        lib.linear_f32(xd, wd, None, rd, None, yf, m, n, k, kernel=kern)
        assert np.array_equal(yf.cpu().numpy().view(np.int32), want_f32_nobias.view(np.int32)), f"f32 row scale {kern}"
        # half-width outputs: the same value rounded once more; the elements behind the m x n
        # outputs stay untouched (a store of the wrong width would reach them)
        for kind, fn in (("f16", lib.linear_f16), ("bf16", lib.linear_bf16)):
            y16 = torch.full((m * n + 256,), 0x7BAD, dtype=torch.int16, device="cuda:0")
            fn(xd, wd, bd, rd_small, cd, y16, m, n, k, kernel=kern)
            got = y16.cpu().numpy().view(np.uint16)
            assert np.array_equal(got[:m * n].reshape(m, n), want_16[kind]), f"{kind} {kern}"
            assert np.all(got[m * n:] == 0x7BAD), f"{kind} {kern}: wrote past the output"
            fn(xd, wd, None, None, None, y16, m, n, k, kernel=kern)
            assert np.array_equal(y16.cpu().numpy().view(np.uint16)[:m * n].reshape(m, n), plain_16[kind]), f"{kind} plain {kern}"


@pytest.mark.parametrize("kernel", ["auto", "simple", "mfma", "fp6", "skinny"])
def test_half_width_outputs_of_special_values(gpu, kernel):
    """Every accumulator is 1 (one nonzero nibble per row), so output (i, j) is the conversion
    of row_scale[i] * col_scale[j]: the hardware's float -> half and float -> bfloat16 against
    the oracle's on halves, ties, range ends, denormals, infinities and quiet NaNs."""
    import torch

    import int4linear_amd as lib

    v = helpers.special_floats(31)
    snan = (v.view(np.uint32) & 0x7FC00000) == 0x7F800000
    snan &= (v.view(np.uint32) & 0x003FFFFF) != 0
    v = v[~snan]    # a signalling NaN is quieted by the multiplication: left to the quiet ones
    rows = 16384 if kernel != "skinny" else 64
    n, k = 16, 128
    cs = np.array([1, 0.5, 2, 1, 0.75, 3, 1, 0.125, 1, 1, 1.5, 1, 4, 1, 1, 0.25], dtype=np.float32)
    x = np.zeros((rows, k), dtype=np.int8)
    x[:, 5] = 1
    w = np.zeros((n, k), dtype=np.int8)
    w[:, 5] = 1
    xd = helpers.to_device_bytes(helpers.pack_bytes(x))
    wd = helpers.to_device_bytes(helpers.pack_bytes(w))
    ones = np.ones((rows, n), dtype=np.int32)
    y = torch.zeros((rows, n), dtype=torch.int32, device="cuda:0")
    lib.linear_s32(xd, wd, None, y, rows, n, k, kernel=kernel)
    assert np.array_equal(y.cpu().numpy(), ones)
    cd = torch.from_numpy(cs).to("cuda:0")
    if kernel not in ("auto", "simple"):   # those go through all of them, the others through a sample with the range ends and NaNs
        pick = np.random.default_rng(32).choice(len(v), max(4 * rows, 4096) - 40, replace=False)
        v = np.concatenate([v[pick], v[len(v) - 100040:len(v) - 100000]])
    for first in range(0, len(v), rows):
        rs = np.resize(v[first:first + rows], rows).astype(np.float32)
        rd = torch.from_numpy(rs).to("cuda:0")
        for kind, fn in (("f16", lib.linear_f16), ("bf16", lib.linear_bf16)):
            y16 = torch.zeros((rows, n), dtype=torch.int16, device="cuda:0")
            fn(xd, wd, None, rd, cd, y16, rows, n, k, kernel=kernel)
            got = y16.cpu().numpy().view(np.uint16)
            want = oracle.epilogue(ones, None, rs, cs, out=kind)
            bad = np.argwhere(got != want)
            assert bad.size == 0, (kind, kernel, first, bad[:3], [hex(int(rs.view(np.uint32)[i])) for i, _ in bad[:3]])


def test_internal_workspace_shared_between_streams(gpu, host_threads):
    """Calls that use the FP6 workspace from alternating streams, without any host
    synchronisation in between: the library orders them itself."""
    import torch

    import int4linear_amd as lib

    m, n, k = 512, 768, 1024
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    cases = []
    for i in range(6):
        x = helpers.uniform_s4(1400 + i, m, k)
        w = helpers.uniform_s4(1500 + i, n, k)
        cases.append((helpers.to_device_bytes(helpers.pack_bytes(x)), helpers.to_device_bytes(helpers.pack_bytes(w)),
                      torch.full((m, n), -1, dtype=torch.int32, device="cuda:0"),
                      oracle.linear_ref(x, w, threads=host_threads)))
    torch.cuda.synchronize()
    for rep in range(3):
        for i, (xd, wd, yd, _) in enumerate(cases):
            s = streams[i % 2]
            lib.gemm_s4s4s32(xd, wd, yd, m, n, k, kernel="fp6", stream=s.cuda_stream)
    torch.cuda.synchronize()
    for i, (_, _, yd, want) in enumerate(cases):
        assert np.array_equal(yd.cpu().numpy(), want), f"case {i}"


@pytest.mark.parametrize("m, n, k", [(128, 128, 128), (1, 1, 128), (129, 257, 384), (1000, 3000, 1024), (2048, 2048, 256),
                                     (777, 1531, 2048), (2048, 4096, 512), (160, 4096, 4096), (300, 520, 4096), (65, 63, 1024)])
def test_small_grid_form_of_the_int8_kernel(gpu, host_threads, m, n, k):
    """Up to two 128 x 128 tiles per CU the int8 kernel runs in the form whose two waves per
    SIMD split every stage's K and merge their sums through LDS (with 64 x 64 tiles when the
    larger ones would leave half of the CUs idle): plain and with every epilogue, ragged
    edges in both directions, one to many stages."""
    import torch

    import int4linear_amd as lib

    x = helpers.uniform_s4(4200 + m, m, k)
    w = helpers.uniform_s4(4300 + n, n, k)
    want = oracle.linear_ref(x, w, threads=host_threads)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    assert np.array_equal(helpers.run_gemm(xp, wp, m, n, k, kernel="mfma"), want)
    rng = np.random.default_rng(m + n + k)
    bias = rng.integers(-1000, 1000, size=n, dtype=np.int32)
    rs = rng.uniform(0.1, 2.0, size=m).astype(np.float32)
    cs = rng.uniform(0.1, 2.0, size=n).astype(np.float32)
    xd, wd = helpers.to_device_bytes(xp), helpers.to_device_bytes(wp)
    bd, rd, cd = (torch.from_numpy(a).to("cuda:0") for a in (bias, rs, cs))
    y = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
    lib.linear_s32(xd, wd, bd, y, m, n, k, kernel="mfma")
    assert np.array_equal(y.cpu().numpy(), oracle.epilogue(want, bias))
    yf = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    lib.linear_f32(xd, wd, bd, rd, cd, yf, m, n, k, kernel="mfma")
    assert np.array_equal(yf.cpu().numpy().view(np.int32), oracle.epilogue(want, bias, rs, cs, f32=True).view(np.int32))
    lib.linear_f32(xd, wd, None, rd, None, yf, m, n, k, kernel="mfma")
    assert np.array_equal(yf.cpu().numpy().view(np.int32), oracle.epilogue(want, None, rs, None, f32=True).view(np.int32))
    helpers.check_half_width_outputs(xd, wd, want, bias, rs, cs, m, n, k, kernel="mfma")


@pytest.mark.parametrize("m, n, k", [(300, 2049, 8192), (257, 1000, 4096), (512, 1024, 14336), (300, 520, 16392),
                                     (1024, 4096, 14336)])
def test_split_k_form_of_the_fp6_kernel(gpu, host_threads, m, n, k):
    """64 tiles of 256 x 256 or fewer and long K: the FP6 GEMM runs K-slices of every tile on
    their own CUs (partial sums in slabs behind the converted operands in the internal
    workspace), a second kernel adds them up and applies the epilogue."""
    import torch

    import int4linear_amd as lib

    x = helpers.uniform_s4(3200 + m, m, k)
    w = helpers.uniform_s4(3300 + n, n, k)
    want = oracle.linear_ref(x, w, threads=host_threads)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    lib.init()
    operands = lib.fp6_operand_bytes(m, k) + lib.fp6_operand_bytes(n, k)
    if lib.kernel_for_shape(m, n, k) == "fp6":
        slabs = lib.workspace_bytes(m, n, k) - operands
        assert slabs >= 2 * m * n * 4 and slabs % (m * n * 4) == 0
    assert np.array_equal(helpers.run_gemm(xp, wp, m, n, k, kernel="fp6"), want)
    rng = np.random.default_rng(m + k)
    bias = rng.integers(-1000, 1000, size=n, dtype=np.int32)
    rs = rng.uniform(0.1, 2.0, size=m).astype(np.float32)
    cs = rng.uniform(0.1, 2.0, size=n).astype(np.float32)
    xd, wd = helpers.to_device_bytes(xp), helpers.to_device_bytes(wp)
    bd, rd, cd = (torch.from_numpy(a).to("cuda:0") for a in (bias, rs, cs))
    y = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
    lib.linear_s32(xd, wd, bd, y, m, n, k, kernel="fp6")
    assert np.array_equal(y.cpu().numpy(), oracle.epilogue(want, bias))
    yf = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    lib.linear_f32(xd, wd, bd, rd, cd, yf, m, n, k, kernel="fp6")
    assert np.array_equal(yf.cpu().numpy().view(np.int32), oracle.epilogue(want, bias, rs, cs, f32=True).view(np.int32))
    helpers.check_half_width_outputs(xd, wd, want, bias, rs, cs, m, n, k, kernel="fp6")


@pytest.mark.parametrize("m, n, k", [(128, 4096, 14336), (300, 520, 12288), (1024, 512, 14336), (100, 300, 8192),
                                     (140, 1000, 12288), (200, 136, 16384)])
def test_split_k_form_of_the_int8_kernel(gpu, host_threads, m, n, k):
    """Few tiles and long K: automatic dispatch splits K over workgroups (partial sums in the
    internal workspace, a second kernel adds them and applies the epilogue)."""
    import torch

    import int4linear_amd as lib

    x = helpers.uniform_s4(2200 + m, m, k)
    w = helpers.uniform_s4(2300 + n, n, k)
    want = oracle.linear_ref(x, w, threads=host_threads)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    assert lib.kernel_for_shape(m, n, k) == "mfma"
    lib.init()
    assert lib.workspace_bytes(m, n, k) > 0 and lib.workspace_bytes(m, n, k) % (m * n * 4) == 0
    assert np.array_equal(helpers.run_gemm(xp, wp, m, n, k, kernel="auto"), want)
    # the epilogue moves into the second kernel
    rng = np.random.default_rng(m + k)
    bias = rng.integers(-1000, 1000, size=n, dtype=np.int32)
    rs = rng.uniform(0.1, 2.0, size=m).astype(np.float32)
    cs = rng.uniform(0.1, 2.0, size=n).astype(np.float32)
    xd, wd = helpers.to_device_bytes(xp), helpers.to_device_bytes(wp)
    bd, rd, cd = (torch.from_numpy(a).to("cuda:0") for a in (bias, rs, cs))
    y = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
    lib.linear_s32(xd, wd, bd, y, m, n, k)
    assert np.array_equal(y.cpu().numpy(), oracle.epilogue(want, bias))
    yf = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda:0")
    lib.linear_f32(xd, wd, bd, rd, cd, yf, m, n, k)
    assert np.array_equal(yf.cpu().numpy().view(np.int32), oracle.epilogue(want, bias, rs, cs, f32=True).view(np.int32))
    helpers.check_half_width_outputs(xd, wd, want, bias, rs, cs, m, n, k)
    # without a workspace the same call runs unsplit
    lib.set_workspace_limit(0)
    try:
        assert lib.workspace_bytes(m, n, k) == 0
        assert np.array_equal(helpers.run_gemm(xp, wp, m, n, k, kernel="auto"), want)
    finally:
        lib.set_workspace_limit(1 << 30)


def test_concurrent_host_threads(gpu, host_threads):
    """Four host threads, each with its own stream, mixing kernels that share the internal
    workspace with kernels that do not: the library serialises what has to be serialised."""
    import threading

    import torch

    import int4linear_amd as lib

    shapes = [(512, 768, 1024, "fp6"), (16, 2048, 1024, "auto"), (300, 520, 512, "mfma"), (640, 512, 384, "fp6")]
    cases = []
    for i, (m, n, k, kern) in enumerate(shapes):
        x = helpers.uniform_s4(2000 + i, m, k)
        w = helpers.uniform_s4(2100 + i, n, k)
        cases.append((m, n, k, kern, helpers.to_device_bytes(helpers.pack_bytes(x)),
                      helpers.to_device_bytes(helpers.pack_bytes(w)),
                      torch.full((m, n), -1, dtype=torch.int32, device="cuda:0"),
                      oracle.linear_ref(x, w, threads=host_threads)))
    torch.cuda.synchronize()
    errors = []

    def worker(case):
        m, n, k, kern, xd, wd, yd, want = case
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            for _ in range(25):
                lib.gemm_s4s4s32(xd, wd, yd, m, n, k, kernel=kern, stream=stream.cuda_stream)
            stream.synchronize()
            if not np.array_equal(yd.cpu().numpy(), want):
                errors.append(f"mismatch {(m, n, k, kern)}")
        except Exception as exc:  # surfaced in the main thread below
            errors.append(repr(exc))

    threads = [threading.Thread(target=worker, args=(c,)) for c in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors


def test_hip_graph_capture_and_replay(gpu, host_threads):
    """The allocation-free entry points are plain kernel launches, so a caller may capture them
    in a HIP graph: caller-owned FP6 operands, the int8 kernel and the streaming kernel, replayed
    three times with new operand contents and eager work in between."""
    import torch

    import int4linear_amd as lib

    m, n, k = 320, 768, 512
    ms, ns, ks = 16, 2048, 1024
    xd = torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda:0")
    wd = torch.zeros(n * k // 2, dtype=torch.uint8, device="cuda:0")
    xs = torch.zeros(ms * ks // 2, dtype=torch.uint8, device="cuda:0")
    ws = torch.zeros(ns * ks // 2, dtype=torch.uint8, device="cuda:0")
    xc = torch.zeros(lib.fp6_operand_bytes(m, k), dtype=torch.uint8, device="cuda:0")
    wc = torch.zeros(lib.fp6_operand_bytes(n, k), dtype=torch.uint8, device="cuda:0")
    y6 = torch.zeros((m, n), dtype=torch.int32, device="cuda:0")
    y8 = torch.zeros((m, n), dtype=torch.int32, device="cuda:0")
    ysk = torch.zeros((ms, ns), dtype=torch.int32, device="cuda:0")
    lib.init()
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        lib.fp6_convert(xd, xc, m, k)
        lib.fp6_convert(wd, wc, n, k)
        lib.gemm_fp6_converted(xc, wc, y6, m, n, k)
        lib.gemm_s4s4s32(xd, wd, y8, m, n, k, kernel="mfma")
        lib.gemm_s4s4s32(xs, ws, ysk, ms, ns, ks, kernel="skinny")

    for rep in range(3):
        x = helpers.uniform_s4(1600 + rep, m, k)
        w = helpers.uniform_s4(1700 + rep, n, k)
        x2 = helpers.normal_s4(1800 + rep, ms, ks)
        w2 = helpers.uniform_s4(1900 + rep, ns, ks)
        xd.copy_(helpers.to_device_bytes(helpers.pack_bytes(x)))
        wd.copy_(helpers.to_device_bytes(helpers.pack_bytes(w)))
        xs.copy_(helpers.to_device_bytes(helpers.pack_bytes(x2)))
        ws.copy_(helpers.to_device_bytes(helpers.pack_bytes(w2)))
        for y in (y6, y8, ysk):
            y.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle.linear_ref(x, w, threads=host_threads)
        assert np.array_equal(y6.cpu().numpy(), want), f"fp6, replay {rep}"
        assert np.array_equal(y8.cpu().numpy(), want), f"int8, replay {rep}"
        assert np.array_equal(ysk.cpu().numpy(), oracle.linear_ref(x2, w2, threads=host_threads)), f"skinny, replay {rep}"


def test_automatic_dispatch_under_graph_capture(gpu):
    """A call with automatic dispatch on a stream that is being captured must not touch the
    internal workspace (no allocation, no free, no events on other streams, no workspace
    address baked into the graph): shapes that would take the FP6 kernel or a split-K form
    run on kernels that need none, and an explicit FP6 request is refused.  The workspace is
    released between the replays, which would invalidate any pointer a graph had kept."""
    import torch

    import int4linear_amd as lib

    shapes = [(2304, 4096, 3072), (128, 4096, 14336), (40, 56, 4104)]  # fp6, int8 split-K, fp6 (ragged K)
    assert [lib.kernel_for_shape(*s) for s in shapes] == ["fp6", "mfma", "fp6"]
    assert all(lib.workspace_bytes(*s) > 0 for s in shapes)
    bufs = []
    for (m, n, k) in shapes:
        bufs.append((torch.zeros(m * k // 2, dtype=torch.uint8, device="cuda:0"),
                     torch.zeros(n * k // 2, dtype=torch.uint8, device="cuda:0"),
                     torch.zeros((m, n), dtype=torch.int32, device="cuda:0"),
                     torch.zeros((m, n), dtype=torch.int32, device="cuda:0")))
    lib.release_workspace()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for (m, n, k), (xd, wd, yd, _) in zip(shapes, bufs):
            lib.gemm_s4s4s32(xd, wd, yd, m, n, k)
        with pytest.raises(lib.Int4LinearError) as refused:
            lib.gemm_s4s4s32(bufs[0][0], bufs[0][1], bufs[0][2], *shapes[0], kernel="fp6")
    assert refused.value.status == 5
    g = torch.Generator(device="cuda:0")
    for rep in range(3):
        g.manual_seed(4200 + rep)
        for (xd, wd, yd, ref) in bufs:
            xd.copy_(torch.randint(0, 256, xd.shape, dtype=torch.uint8, device="cuda:0", generator=g))
            wd.copy_(torch.randint(0, 256, wd.shape, dtype=torch.uint8, device="cuda:0", generator=g))
            yd.fill_(-1)
        # eager calls of the same shapes in between: these do use (and regrow) the workspace
        for (m, n, k), (xd, wd, _, ref) in zip(shapes, bufs):
            lib.gemm_s4s4s32(xd, wd, ref, m, n, k)
        torch.cuda.synchronize()
        lib.release_workspace()
        graph.replay()
        torch.cuda.synchronize()
        for shape, (_, _, yd, ref) in zip(shapes, bufs):
            assert torch.equal(yd, ref), f"{shape}, replay {rep}"


def _random_shapes(count, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        m = int(rng.integers(1, 65)) if rng.random() < 0.5 else int(rng.integers(65, 700))
        n = int(rng.integers(1, 6000))
        r = rng.random()
        if r < 0.4:
            k = 256 * int(rng.integers(1, 40))
        elif r < 0.7:
            k = 128 * int(rng.integers(1, 80))
        else:
            k = 8 * int(rng.integers(1, 600))
        shapes.append((m, n, k))
    return shapes


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_random_shapes_against_the_scalar_kernel(gpu, seed):
    """Forty random shapes per seed through the automatic dispatch, whole outputs compared on
    the device with the scalar kernel (itself checked against the oracle above): exercises the
    plan search of the streaming kernel, tile edges and K padding on shapes nobody picked."""
    import torch

    import int4linear_amd as lib

    g = torch.Generator(device="cuda:0")
    for (m, n, k) in _random_shapes(40, seed):
        g.manual_seed(m * 1000003 + n * 101 + k)
        x = torch.randint(0, 256, (m * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
        w = torch.randint(0, 256, (n * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
        got = torch.full((m, n), 0x5A5A5A5A, dtype=torch.int32, device="cuda:0")
        ref = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
        lib.gemm_s4s4s32(x, w, got, m, n, k)
        lib.gemm_s4s4s32(x, w, ref, m, n, k, kernel="simple")
        torch.cuda.synchronize()
        assert torch.equal(got, ref), f"shape {(m, n, k)} kernel {lib.kernel_for_shape(m, n, k)}"


def test_random_decode_split_shapes_against_the_scalar_kernel(gpu):
    """Random shapes in and around the regime in which the weight-streaming kernel splits K across
    workgroups (33 to 64 rows of X, long K, up to 64 rows of W per quarter of the CUs), every
    shape twice in a row (the arrival counters must be back at zero), whole outputs compared on
    the device with the scalar kernel."""
    import torch

    import int4linear_amd as lib

    rng = np.random.default_rng(20261)
    g = torch.Generator(device="cuda:0")
    split = 0
    for _ in range(24):
        m = int(rng.integers(30, 65))
        n = int(rng.integers(200, 4300))
        k = int(rng.choice([14336, 15360, 16384, 20480, 28672, 12288, 14336 + 256]))
        split += lib.workspace_bytes(m, n, k) > 0
        g.manual_seed(m * 1000003 + n * 101 + k)
        x = torch.randint(0, 256, (m * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
        w = torch.randint(0, 256, (n * k // 2,), dtype=torch.uint8, device="cuda:0", generator=g)
        ref = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
        lib.gemm_s4s4s32(x, w, ref, m, n, k, kernel="simple")
        for rep in range(2):
            got = torch.full((m, n), 0x5A5A5A5A, dtype=torch.int32, device="cuda:0")
            lib.gemm_s4s4s32(x, w, got, m, n, k)
            torch.cuda.synchronize()
            assert torch.equal(got, ref), f"shape {(m, n, k)} call {rep} workspace {lib.workspace_bytes(m, n, k)}"
    assert split >= 8, split  # the draw must actually reach the split form


# ---- configuration 5: adversarial ---------------------------------------------------------

def test_cfg5_all_minus_eight_full_size(gpu):
    import torch

    m, n, k = 8192, 28672, 8192
    xp = np.full((m, k // 2), 0x88, dtype=np.uint8)
    wp = np.full((n, k // 2), 0x88, dtype=np.uint8)
    for kern in ("auto", "mfma", "fp6"):
        got = helpers.run_gemm(xp, wp, m, n, k, kernel=kern, keep_on_device=True)
        assert int(got.min()) == 524288 and int(got.max()) == 524288, kern
        del got
        torch.cuda.empty_cache()


def test_cfg5_ragged_1000_3000_4096(gpu, host_threads):
    x = helpers.uniform_s4(51, 1000, 4096)
    w = helpers.uniform_s4(52, 3000, 4096)
    check_all_kernels(x, w, threads=host_threads, kernels=["auto", "mfma", "fp6", "simple"])


@pytest.mark.parametrize("a, b, per_k", [(-8, -8, 64), (7, 7, 49), (-8, 7, -56), (7, -8, -56)])
def test_extreme_constants(gpu, a, b, per_k):
    m, n, k = 300, 260, 8192
    x = np.full((m, k), a, dtype=np.int8)
    w = np.full((n, k), b, dtype=np.int8)
    check_all_kernels(x, w, want=np.full((m, n), per_k * k, dtype=np.int32))


# ---- edges ------------------------------------------------------------------------------------

@pytest.mark.parametrize("m, n, k", [
    (1, 1, 128), (15, 17, 128), (16, 16, 256), (65, 3, 384), (257, 255, 128), (256, 256, 512),
    (129, 130, 640), (300, 515, 256), (513, 257, 1024), (70, 1000, 1152), (2, 2, 8), (9, 7, 24),
    (31, 33, 72), (64, 64, 64), (100, 100, 200),
])
def test_ragged_shapes(gpu, m, n, k):
    x = helpers.uniform_s4(m * 7 + n, m, k)
    w = helpers.uniform_s4(k * 3 + n, n, k)
    check_all_kernels(x, w, threads=4)


def test_one_hot_rows_pin_nibble_and_k_order(gpu):
    # W[j] = delta(l, k_j)  =>  C[i][j] = A[i][k_j], for every k position of several stages.
    m, k = 40, 512
    n = k
    x = helpers.uniform_s4(61, m, k)
    w = np.zeros((n, k), dtype=np.int8)
    w[np.arange(n), np.arange(n)] = 1
    check_all_kernels(x, w, want=x.astype(np.int32))


def test_degenerate_sizes(gpu):
    import torch

    import int4linear_amd as lib

    dev = torch.device("cuda:0")
    y = torch.full((8, 12), 77, dtype=torch.int32, device=dev)
    a = torch.zeros(64, dtype=torch.uint8, device=dev)
    lib.gemm_s4s4s32(a, a, y, 8, 12, 0)             # K == 0: C is zero-filled
    torch.cuda.synchronize()
    assert not bool(y.any())
    y.fill_(77)
    lib.gemm_s4s4s32(a, a, y, 0, 12, 128)           # M == 0: nothing happens
    lib.gemm_s4s4s32(a, a, y, 8, 0, 128)            # N == 0: nothing happens
    torch.cuda.synchronize()
    assert bool((y == 77).all())
    with pytest.raises(lib.Int4LinearError):
        lib.gemm_s4s4s32(a, a, y, 8, 12, 64, kernel="mfma")   # K below one stage
    with pytest.raises(lib.Int4LinearError):
        lib.gemm_s4s4s32(a, a, y, 65, 12, 128, kernel="skinny")  # more than 64 rows need K in 128-byte tiles


# ---- properties that hold at any size -------------------------------------------------------

def test_properties_at_4096(gpu):
    import torch

    m = n = k = 4096
    x = helpers.uniform_s4(71, m, k)
    w = helpers.uniform_s4(72, n, k)
    xp, wp = helpers.pack_bytes(x), helpers.pack_bytes(w)
    y = helpers.run_gemm(xp, wp, m, n, k, keep_on_device=True)
    # swapping the operands transposes the result
    yt = helpers.run_gemm(wp, xp, n, m, k, keep_on_device=True)
    assert torch.equal(yt, y.t())
    # the same byte permutation along K on both operands changes nothing
    perm = np.random.default_rng(73).permutation(k // 2)
    yp = helpers.run_gemm(xp[:, perm], wp[:, perm], m, n, k, keep_on_device=True)
    assert torch.equal(yp, y)
    # negating A (values in [-7, 7] so -A is representable) negates C
    x7 = np.clip(x, -7, 7)
    y7 = helpers.run_gemm(helpers.pack_bytes(x7), wp, m, n, k, keep_on_device=True)
    yn = helpers.run_gemm(helpers.pack_bytes(-x7), wp, m, n, k, keep_on_device=True)
    assert torch.equal(yn, -y7)
    # row sums: A = ones  =>  C[i][j] = sum_l W[j][l]
    ones = helpers.pack_bytes(np.ones((64, k), dtype=np.int8))
    ys = helpers.run_gemm(ones, wp, 64, n, k)
    assert np.array_equal(ys, np.tile(w.astype(np.int32).sum(axis=1), (64, 1)))


# ---- the reference's blocking entry points ------------------------------------------------------

@pytest.mark.parametrize("shape", [(300, 520, 512), (16, 1024, 1024), (33, 70, 72), (2048, 2304, 256)])
@pytest.mark.parametrize("version", [0, 1, 2, 10, 11, 20, 21])
def test_every_version_takes_every_shape(gpu, version, shape):
    """v0..v21 are different kernels (scalar, int8 128/256 tile, +skinny, +fp6, automatic);
    a version whose kernel cannot run a shape falls back, so all of them agree everywhere."""
    import torch

    import int4linear_amd as lib

    m, n, k = shape
    x = helpers.uniform_s4(900 + version, m, k)
    w = helpers.uniform_s4(901 + version, n, k)
    want = oracle.linear_ref(x, w, threads=4)
    xd = helpers.to_device_bytes(helpers.pack_words_as_bytes(x))
    wd = helpers.to_device_bytes(helpers.pack_words_as_bytes(w))
    yd = torch.full((m, n), 0x5A5A5A5A, dtype=torch.int32, device="cuda:0")
    getattr(lib, f"linear_v{version}_launch")(xd, wd, yd, m, n, k)
    assert np.array_equal(yd.cpu().numpy(), want)


@pytest.mark.parametrize("version", [0, 1, 2, 10, 11, 20, 21])
def test_reference_entry_points(gpu, version):
    import torch

    import int4linear_amd as lib

    m, n, k = 260, 136, 256
    x = helpers.uniform_s4(80 + version, m, k)
    w = helpers.uniform_s4(90 + version, n, k)
    want = oracle.linear_ref(x, w)
    # operands packed by the library's own host packer, as the reference's harness does
    xd = helpers.to_device_bytes(lib.pack_rows(x))
    wd = helpers.to_device_bytes(lib.pack_rows(w))
    yd = torch.full((m, n), -1, dtype=torch.int32, device="cuda:0")
    getattr(lib, f"linear_v{version}_launch")(xd, wd, yd, m, n, k)
    # blocking call: the result is complete on return, no synchronisation here
    assert oracle.is_same(yd.cpu().numpy(), want)


# ---- device packer / unpacker ----------------------------------------------------------------------

@pytest.mark.parametrize("m, n", [(1, 8), (5, 13), (64, 4096), (33, 1001), (1000, 64)])
def test_device_packer(gpu, m, n):
    import torch

    import int4linear_amd as lib

    v = np.random.default_rng(m + n).integers(-100, 100, size=(m, n), dtype=np.int32)
    words = (n + 7) // 8
    src = torch.from_numpy(v).to("cuda:0")
    dst = torch.full((m, words), -1, dtype=torch.int32, device="cuda:0")
    lib.pack_device(src, dst, m, n)
    back = torch.full((m, n), 99, dtype=torch.int32, device="cuda:0")
    lib.unpack_device(dst, back, m, n)
    torch.cuda.synchronize()
    want_words = oracle.pack(v)
    assert np.array_equal(dst.cpu().numpy(), want_words)
    assert np.array_equal(back.cpu().numpy(), oracle.unpack(want_words, n))
