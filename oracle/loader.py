"""ctypes loader of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import c_int, c_void_p
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ORACLE_SO = HERE / "liboracle.so"
REF_PACKER_SO = HERE / "_ref" / "libpacker_ref.so"

_oracle = None
_ref = None


def build() -> None:
    """Compile liboracle.so (and _ref/libpacker_ref.so when the reference is mounted)."""
    subprocess.run(["make", "-C", str(HERE), "-B", "all"], check=True, stdout=subprocess.DEVNULL)


def oracle() -> ctypes.CDLL:
    global _oracle
    if _oracle is None:
        if not ORACLE_SO.exists():
            build()
        lib = ctypes.CDLL(str(ORACLE_SO))
        lib.oracle_pack.argtypes = [c_void_p, c_void_p, c_int, c_int]
        lib.oracle_unpack.argtypes = [c_void_p, c_void_p, c_int, c_int]
        lib.oracle_linear_ref.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]
        lib.oracle_linear_ref_mt.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int]
        lib.oracle_is_same.argtypes = [c_void_p, c_void_p, c_int]
        lib.oracle_is_same.restype = c_int
        for f in (lib.oracle_pack, lib.oracle_unpack, lib.oracle_linear_ref, lib.oracle_linear_ref_mt):
            f.restype = None
        _oracle = lib
    return _oracle


def ref_packer():
    """The reference's own packer.cpp compiled into oracle/_ref/, or None if not built."""
    global _ref
    if _ref is None and REF_PACKER_SO.exists():
        lib = ctypes.CDLL(str(REF_PACKER_SO))
        for name in ("_Z4packPKiPiii", "_Z6unpackPKiPiii"):
            fn = getattr(lib, name)
            fn.argtypes = [c_void_p, c_void_p, c_int, c_int]
            fn.restype = None
        _ref = lib
    return _ref


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def pack(values: np.ndarray) -> np.ndarray:
    """values: (m, n) ints -> (m, ceil(n/8)) int32 words."""
    v = _i32(values)
    m, n = v.shape
    out = np.empty((m, (n + 7) // 8), dtype=np.int32)
    oracle().oracle_pack(v.ctypes.data, out.ctypes.data, m, n)
    return out


def unpack(words: np.ndarray, n: int) -> np.ndarray:
    w = _i32(words)
    m = w.shape[0]
    out = np.empty((m, n), dtype=np.int32)
    oracle().oracle_unpack(w.ctypes.data, out.ctypes.data, m, n)
    return out


def linear_ref(x: np.ndarray, w: np.ndarray, threads: int = 1) -> np.ndarray:
    """x: (m, k) ints, w: (n, k) ints (unpacked) -> (m, n) int32."""
    x = _i32(x)
    w = _i32(w)
    m, k = x.shape
    n, k2 = w.shape
    assert k == k2
    y = np.empty((m, n), dtype=np.int32)
    if threads <= 1:
        oracle().oracle_linear_ref(x.ctypes.data, w.ctypes.data, y.ctypes.data, m, n, k)
    else:
        oracle().oracle_linear_ref_mt(x.ctypes.data, w.ctypes.data, y.ctypes.data, m, n, k, threads)
    return y


OUT_KINDS = {"s32": 0, "f32": 1, "f16": 2, "bf16": 3}


def epilogue(y: np.ndarray, bias=None, row_scale=None, col_scale=None, f32: bool = False, out: str | None = None) -> np.ndarray:
    """Applies the linear layer's epilogue to an int32 product; returns int32, float32 (f32 set
    or out == "f32"), or the uint16 bit patterns of the half / bfloat16 output (out == "f16",
    "bf16")."""
    kind = OUT_KINDS[out] if out is not None else (1 if f32 else 0)
    buf = np.ascontiguousarray(_i32(y)).copy()
    m, n = buf.shape
    keep = []

    def ptr(a, dtype, count):
        if a is None:
            return None
        a = np.ascontiguousarray(a, dtype=dtype)
        assert a.size == count
        keep.append(a)
        return a.ctypes.data

    fn = oracle().oracle_epilogue
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                   ctypes.c_int]
    fn(buf.ctypes.data, m, n, ptr(bias, np.int32, n), ptr(row_scale, np.float32, m), ptr(col_scale, np.float32, n),
       kind)
    if kind >= 2:
        return buf.astype(np.uint16)
    return buf.view(np.float32) if kind == 1 else buf


def convert_f32(values: np.ndarray, out: str) -> np.ndarray:
    """float32 values to the uint16 bit patterns of half ("f16") or bfloat16 ("bf16"), as the
    epilogue rounds them."""
    src = np.ascontiguousarray(values, dtype=np.float32).ravel()
    dst = np.empty(src.size, dtype=np.uint16)
    fn = oracle().oracle_convert_f32
    fn.restype = None
    fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    fn(src.ctypes.data, dst.ctypes.data, src.size, OUT_KINDS[out])
    return dst.reshape(np.shape(values))


def is_same(a: np.ndarray, b: np.ndarray) -> bool:
    a = _i32(a).ravel()
    b = _i32(b).ravel()
    assert a.size == b.size
    return bool(oracle().oracle_is_same(a.ctypes.data, b.ctypes.data, a.size))
