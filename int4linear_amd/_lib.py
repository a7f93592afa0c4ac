"""ctypes binding of libint4linear.so -- the C ABI declared in include/int4linear.h.

There is no CPU fallback: if the shared library has not been built, importing the
symbols raises, and every compute call needs a gfx950 device.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int, c_size_t, c_void_p
from pathlib import Path

# INT4LINEAR_LIBRARY overrides the in-tree location (e.g. to try a differently built copy).
LIB_PATH = Path(os.environ.get("INT4LINEAR_LIBRARY") or
                Path(__file__).resolve().parent / "lib" / "libint4linear.so")

# (name, restype, argtypes) for every extern "C" symbol of include/int4linear.h.
C_ABI = [
    ("int4linear_init", c_int, []),
    ("int4linear_gemm_s4s4s32", c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    ("int4linear_gemm_s4s4s32_static", c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    ("int4linear_gemm_s4s4s32_ex", c_int,
     [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    ("int4linear_pack_s32_to_s4", c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    ("int4linear_unpack_s4_to_s32", c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    ("int4linear_linear_s32", c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    ("int4linear_linear_f32", c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                      c_int, c_void_p]),
    ("int4linear_linear_f16", c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                      c_int, c_void_p]),
    ("int4linear_linear_bf16", c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                       c_int, c_void_p]),
    ("int4linear_fp6_operand_bytes", c_size_t, [c_int, c_int]),
    ("int4linear_fp6_convert", c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    ("int4linear_gemm_fp6_converted", c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    ("int4linear_linear_fp6_converted", c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                c_int, c_int, c_int, c_void_p]),
    ("int4linear_workspace_bytes", c_size_t, [c_int, c_int, c_int]),
    ("int4linear_set_workspace_limit", None, [c_size_t]),
    ("int4linear_release_workspace", c_int, []),
    ("int4linear_kernel_for_shape", c_char_p, [c_int, c_int, c_int]),
    ("int4linear_status_string", c_char_p, [c_int]),
    ("int4linear_last_hip_error", c_int, []),
    ("int4linear_device_cu_count", c_int, []),
]

# The reference's C++-linkage entry points (Itanium-mangled) exported next to the C ABI.
_LAUNCH_ARGS = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]
CXX_ABI = [
    ("_Z16linear_v0_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z16linear_v1_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z16linear_v2_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z17linear_v10_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z17linear_v11_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z17linear_v20_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z17linear_v21_launchPvS_S_iii", None, _LAUNCH_ARGS),
    ("_Z4packPKiPiii", None, [c_void_p, c_void_p, c_int, c_int]),
    ("_Z6unpackPKiPiii", None, [c_void_p, c_void_p, c_int, c_int]),
]

_lib = None


class Int4LinearError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, status: int, message: str, hip_error: int = 0):
        super().__init__(f"int4linear status {status}: {message}"
                         + (f" (hip error {hip_error})" if hip_error else ""))
        self.status = status
        self.hip_error = hip_error


def load() -> ctypes.CDLL:
    """Load the shared library once and attach prototypes to every exported symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m int4linear_amd.build` "
            "(there is no CPU fallback for the GPU path)")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, restype, argtypes in C_ABI + CXX_ABI:
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != 0:
        lib = load()
        raise Int4LinearError(status, lib.int4linear_status_string(status).decode(),
                              lib.int4linear_last_hip_error())
