"""CPU-side checks of the product library: the C ABI loads and exports every symbol the
header declares, the host packer agrees with the oracle, and argument validation that
needs no device behaves as documented.  No compute call is made here."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

import int4linear_amd as lib
from int4linear_amd import _lib
from oracle import loader as oracle
from tests import helpers

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "int4linear.h").read_text()
GOLDEN = np.load(ROOT / "tests" / "golden" / "int4_gemm_golden.npz")


def declared_c_symbols():
    body = HEADER.split('extern "C" {', 1)[1].split('} /* extern "C" */', 1)[0]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    return sorted(set(re.findall(r"\b(int4linear_\w+)\s*\(", body)))


def test_header_symbols_all_exported():
    names = declared_c_symbols()
    assert len(names) >= 9
    cdll = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in names:
        assert hasattr(cdll, name), name
    # and the binding table covers exactly the header
    assert sorted(n for n, _, _ in _lib.C_ABI) == names


def test_reference_cxx_entry_points_exported():
    cdll = ctypes.CDLL(str(_lib.LIB_PATH))
    for version in (0, 1, 2, 10, 11, 20, 21):
        name = f"linear_v{version}_launch"
        assert f"void {name}(void *x_packed_d" in HEADER
        assert hasattr(cdll, f"_Z{len(name)}{name}PvS_S_iii"), name
    assert hasattr(cdll, "_Z4packPKiPiii") and hasattr(cdll, "_Z6unpackPKiPiii")


def test_status_strings():
    L = _lib.load()
    seen = {L.int4linear_status_string(s).decode() for s in range(0, 9)}
    assert len(seen) == 9 and "ok" in seen and "unknown status" not in seen
    assert L.int4linear_status_string(99).decode() == "unknown status"


@pytest.mark.parametrize("m, n, k", [(-1, 4, 8), (4, -1, 8), (4, 4, -8), (4, 4, 12), (4, 4, 7)])
def test_bad_shapes_are_rejected_before_touching_the_device(m, n, k):
    L = _lib.load()
    st = L.int4linear_gemm_s4s4s32(None, None, None, m, n, k, None)
    assert st == 1  # INT4LINEAR_ERR_SHAPE
    with pytest.raises(lib.Int4LinearError):
        _lib.check(st)


def test_empty_output_is_a_noop_without_a_device():
    L = _lib.load()
    assert L.int4linear_gemm_s4s4s32(None, None, None, 0, 5, 8, None) == 0
    assert L.int4linear_gemm_s4s4s32(None, None, None, 5, 0, 8, None) == 0


def test_null_and_alignment_checks():
    L = _lib.load()
    assert L.int4linear_gemm_s4s4s32(None, None, None, 4, 4, 8, None) == 2      # null C
    assert L.int4linear_gemm_s4s4s32(None, 16, 16, 4, 4, 8, None) == 2          # null A
    assert L.int4linear_gemm_s4s4s32(16, 16, 24, 4, 4, 8, None) == 3            # C misaligned
    assert L.int4linear_gemm_s4s4s32(8, 16, 16, 4, 4, 8, None) == 3             # A misaligned
    assert L.int4linear_gemm_s4s4s32_ex(16, 16, 16, 4, 4, 8, 9, None) == 5      # unknown kernel
    assert L.int4linear_gemm_s4s4s32_ex(16, 16, 16, 4, 4, 8, -1, None) == 5


def test_kernel_dispatch_table():
    assert lib.kernel_for_shape(8192, 8192, 8192) == "fp6"
    assert lib.kernel_for_shape(4096, 4096, 4096) == "fp6"
    assert lib.kernel_for_shape(2048, 2048, 2048) == "mfma"   # too few 256 x 256 tiles
    assert lib.kernel_for_shape(1024, 1024, 1024) == "mfma"
    assert lib.kernel_for_shape(1000, 3000, 4096) == "mfma"
    assert lib.kernel_for_shape(16, 4096, 4096) == "skinny"
    assert lib.kernel_for_shape(1, 14336, 4096) == "skinny"
    assert lib.kernel_for_shape(64, 4096, 14336) == "skinny"
    # from 65 rows on the int8 kernel's small-grid forms are faster than runs of 64 rows
    assert lib.kernel_for_shape(65, 4096, 4096) == "mfma"
    assert lib.kernel_for_shape(129, 4096, 4096) == "mfma"
    assert lib.kernel_for_shape(128, 128, 64) == "simple"     # K below one pipeline stage
    assert lib.kernel_for_shape(128, 128, 200) == "simple"    # K % 128 != 0, tiny
    assert lib.kernel_for_shape(1000, 3000, 4104) == "fp6"    # K % 128 != 0: padded by the converter
    assert lib.kernel_for_shape(16, 4096, 4104) == "fp6"
    assert lib.kernel_for_shape(4, 4, 12) == "invalid"


def test_workspace_accounting():
    # FP6 workspace: both operands, rows padded to 256, 0.75 byte per element
    assert lib.workspace_bytes(8192, 8192, 8192) == 2 * 8192 * 8192 * 3 // 4
    assert lib.workspace_bytes(4000, 8192, 4096) == (4096 + 8192) * 4096 * 3 // 4
    assert lib.workspace_bytes(16, 4096, 4096) == 0      # skinny kernel: none
    assert lib.workspace_bytes(1024, 1024, 1024) == 0    # int8 kernel: none
    # K % 128 != 0 runs on the FP6 kernel: rows padded to 256, K to 128
    assert lib.workspace_bytes(1000, 3000, 4104) == (1024 + 3072) * 4224 * 3 // 4
    assert lib.workspace_bytes(0, 3000, 4096) == 0 and lib.workspace_bytes(8192, 8192, 12) == 0
    lib.set_workspace_limit(0)
    try:
        assert lib.workspace_bytes(8192, 8192, 8192) == 0
        assert lib.kernel_for_shape(8192, 8192, 8192) == "mfma"
    finally:
        lib.set_workspace_limit(1 << 30)
    assert lib.kernel_for_shape(8192, 8192, 8192) == "fp6"
    # caller-owned converted operands: rows padded to 256, 0.75 byte per element
    assert lib.fp6_operand_bytes(8192, 8192) == 8192 * 8192 * 3 // 4
    assert lib.fp6_operand_bytes(1, 128) == 256 * 128 * 3 // 4
    assert lib.fp6_operand_bytes(16, 200) == 256 * 256 * 3 // 4   # K padded to 256
    assert lib.fp6_operand_bytes(16, 12) == 0             # K % 8 != 0
    assert lib.fp6_operand_bytes(16, 1 << 18) == 0        # beyond the exact range


@pytest.mark.parametrize("m, n, seed", [(1, 8, 1), (3, 10, 2), (16, 64, 3), (7, 129, 4), (64, 4096, 5)])
def test_host_packer_matches_oracle(m, n, seed):
    v = np.random.default_rng(seed).integers(-8, 8, size=(m, n), dtype=np.int32)
    words = lib.pack_rows(v)
    assert np.array_equal(words, oracle.pack(v))
    back = np.empty((m, n), dtype=np.int32)
    lib.unpack(words, back, m, n)
    assert np.array_equal(back, v)


def test_host_packer_masks_wide_values_and_pads_with_zero():
    v = np.array([[19, -11, 7, -8, 100, -100, 0, 1, 2, 255]], dtype=np.int32)
    assert np.array_equal(lib.pack_rows(v), oracle.pack(v))
    assert (int(lib.pack_rows(v)[0, 1]) & 0xFFFFFF00) == 0


def test_host_packer_golden_words():
    for idx in range(len(GOLDEN["shapes"])):
        assert np.array_equal(lib.pack_rows(GOLDEN[f"x{idx}"]), GOLDEN[f"xwords{idx}"])
    assert np.array_equal(lib.pack_rows(GOLDEN["ragged_values"]), GOLDEN["ragged_words"])


def test_numpy_byte_packer_used_by_large_gpu_tests():
    v = helpers.uniform_s4(3, 33, 256)
    assert np.array_equal(helpers.pack_bytes(v), helpers.pack_words_as_bytes(v).reshape(33, -1))


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parent.parent
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""
