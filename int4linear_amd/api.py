"""Host-side mirror of the reference's interface, on top of the C ABI.

Names and argument meaning follow the reference:
  linear_vN_launch(x_packed_d, w_packed_d, y_d, m, n, k)   kernels/linear_v21.h:760 (and v0..v20)
  pack(src, dst, m, n) / unpack(src, dst, m, n)            utils/packer.h:5-6
Device operands are torch tensors on a ROCm device (torch is only the owner of the
device memory and the stream) or raw integer device addresses.
"""
from __future__ import annotations

import ctypes

import numpy as np

from . import _lib

KERNELS = {"auto": 0, "simple": 1, "mfma": 2, "skinny": 3, "fp6": 4, "mfma128": 5, "mfma256": 6}


def _ptr(obj) -> int:
    """Device (or host) address of a torch tensor / numpy array / raw int."""
    if obj is None:
        return 0
    if isinstance(obj, int):
        return obj
    if isinstance(obj, np.ndarray):
        return obj.ctypes.data
    return obj.data_ptr()  # torch.Tensor


def _current_stream() -> int:
    import torch

    return torch.cuda.current_stream().cuda_stream


def init() -> None:
    """One-time device set-up (idempotent)."""
    lib = _lib.load()
    _lib.check(lib.int4linear_init())


def gemm_s4s4s32(a_packed_d, b_packed_d, c_d, m: int, n: int, k: int, *, kernel: str = "auto",
                 stream: int | None = None) -> None:
    """Asynchronous C = A * B^T on `stream` (default: torch's current stream)."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    st = lib.int4linear_gemm_s4s4s32_ex(_ptr(a_packed_d), _ptr(b_packed_d), _ptr(c_d), m, n, k,
                                        KERNELS[kernel], ctypes.c_void_p(stream))
    _lib.check(st)


STATIC_SCRATCH_BYTES = 128 << 20  # INT4LINEAR_STATIC_SCRATCH_BYTES


def gemm_s4s4s32_static(a_packed_d, b_packed_d, c_d, m: int, n: int, k: int, *, stream: int | None = None) -> None:
    """gemm_s4s4s32 with automatic dispatch on the library's fixed scratch array: allocates
    nothing; shapes that need more scratch than the array holds raise (status 7)."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_gemm_s4s4s32_static(_ptr(a_packed_d), _ptr(b_packed_d), _ptr(c_d), m, n, k,
                                                  ctypes.c_void_p(stream)))


def linear_s32(x_packed_d, w_packed_d, bias_d, y_d, m: int, n: int, k: int, *, kernel: str = "auto",
               stream: int | None = None) -> None:
    """Y = X * W^T + bias (int32); bias_d may be None."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_linear_s32(_ptr(x_packed_d), _ptr(w_packed_d), _ptr(bias_d), _ptr(y_d), m, n, k,
                                         KERNELS[kernel], ctypes.c_void_p(stream)))


def linear_f32(x_packed_d, w_packed_d, bias_d, row_scale_d, col_scale_d, y_d, m: int, n: int, k: int, *,
               kernel: str = "auto", stream: int | None = None) -> None:
    """Y (float32) = ((float)(X * W^T + bias) * row_scale[i]) * col_scale[j]; each of bias_d,
    row_scale_d, col_scale_d may be None."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_linear_f32(_ptr(x_packed_d), _ptr(w_packed_d), _ptr(bias_d), _ptr(row_scale_d),
                                         _ptr(col_scale_d), _ptr(y_d), m, n, k, KERNELS[kernel],
                                         ctypes.c_void_p(stream)))


def linear_f16(x_packed_d, w_packed_d, bias_d, row_scale_d, col_scale_d, y_d, m: int, n: int, k: int, *,
               kernel: str = "auto", stream: int | None = None) -> None:
    """Y (float16) = the value of linear_f32 rounded to nearest even once more."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_linear_f16(_ptr(x_packed_d), _ptr(w_packed_d), _ptr(bias_d), _ptr(row_scale_d),
                                         _ptr(col_scale_d), _ptr(y_d), m, n, k, KERNELS[kernel],
                                         ctypes.c_void_p(stream)))


def linear_bf16(x_packed_d, w_packed_d, bias_d, row_scale_d, col_scale_d, y_d, m: int, n: int, k: int, *,
                kernel: str = "auto", stream: int | None = None) -> None:
    """Y (bfloat16) = the value of linear_f32 rounded to nearest even once more."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_linear_bf16(_ptr(x_packed_d), _ptr(w_packed_d), _ptr(bias_d), _ptr(row_scale_d),
                                          _ptr(col_scale_d), _ptr(y_d), m, n, k, KERNELS[kernel],
                                          ctypes.c_void_p(stream)))


def fp6_operand_bytes(rows: int, k: int) -> int:
    """Bytes of the converted (FP6) form of a rows x k operand; 0 if k is unsupported."""
    return int(_lib.load().int4linear_fp6_operand_bytes(rows, k))


def fp6_convert(packed_d, converted_d, rows: int, k: int, *, stream: int | None = None) -> None:
    """Packed s4 operand -> the FP6 kernel's own operand form (convert static weights once)."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_fp6_convert(_ptr(packed_d), _ptr(converted_d), rows, k, ctypes.c_void_p(stream)))


def gemm_fp6_converted(a_conv_d, b_conv_d, c_d, m: int, n: int, k: int, *, stream: int | None = None) -> None:
    """C = A * B^T from two operands already converted with fp6_convert."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_gemm_fp6_converted(_ptr(a_conv_d), _ptr(b_conv_d), _ptr(c_d), m, n, k,
                                                 ctypes.c_void_p(stream)))


OUT_TYPES = {"s32": 0, "f32": 1, "f16": 2, "bf16": 3}  # INT4LINEAR_OUT_*


def linear_fp6_converted(x_conv_d, w_conv_d, bias_d, row_scale_d, col_scale_d, y_d, out_type: str, m: int, n: int,
                         k: int, *, stream: int | None = None) -> None:
    """gemm_fp6_converted with the epilogue of linear_s32 / linear_f32 / linear_f16 / linear_bf16
    (out_type "s32", "f32", "f16" or "bf16"); bias_d and the scales may each be None."""
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_linear_fp6_converted(_ptr(x_conv_d), _ptr(w_conv_d), _ptr(bias_d), _ptr(row_scale_d),
                                                   _ptr(col_scale_d), _ptr(y_d), OUT_TYPES[out_type], m, n, k,
                                                   ctypes.c_void_p(stream)))


def workspace_bytes(m: int, n: int, k: int) -> int:
    """Internal workspace the automatic dispatch would use for this shape."""
    return int(_lib.load().int4linear_workspace_bytes(m, n, k))


def set_workspace_limit(nbytes: int) -> None:
    _lib.load().int4linear_set_workspace_limit(nbytes)


def release_workspace() -> None:
    _lib.check(_lib.load().int4linear_release_workspace())


def kernel_for_shape(m: int, n: int, k: int) -> str:
    return _lib.load().int4linear_kernel_for_shape(m, n, k).decode()


def pack_device(src_d, dst_d, m: int, n: int, *, stream: int | None = None) -> None:
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_pack_s32_to_s4(_ptr(src_d), _ptr(dst_d), m, n, ctypes.c_void_p(stream)))


def unpack_device(src_d, dst_d, m: int, n: int, *, stream: int | None = None) -> None:
    lib = _lib.load()
    if stream is None:
        stream = _current_stream()
    _lib.check(lib.int4linear_unpack_s4_to_s32(_ptr(src_d), _ptr(dst_d), m, n, ctypes.c_void_p(stream)))


def _launch(symbol: str, x_packed_d, w_packed_d, y_d, m: int, n: int, k: int) -> None:
    lib = _lib.load()
    getattr(lib, symbol)(_ptr(x_packed_d), _ptr(w_packed_d), _ptr(y_d), m, n, k)


# Blocking entry points with the reference's names: default stream, device-synchronised
# on return, no status (a failure prints one line to stderr).
def linear_v0_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z16linear_v0_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def linear_v1_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z16linear_v1_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def linear_v2_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z16linear_v2_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def linear_v10_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z17linear_v10_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def linear_v11_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z17linear_v11_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def linear_v20_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z17linear_v20_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def linear_v21_launch(x_packed_d, w_packed_d, y_d, m, n, k):
    _launch("_Z17linear_v21_launchPvS_S_iii", x_packed_d, w_packed_d, y_d, m, n, k)


def pack(src: np.ndarray, dst: np.ndarray, m: int, n: int) -> None:
    """Host packer: src is m*n int32 values, dst receives m*ceil(n/8) int32 words."""
    lib = _lib.load()
    assert src.dtype == np.int32 and dst.dtype == np.int32
    assert src.flags.c_contiguous and dst.flags.c_contiguous
    assert src.size >= m * n and dst.size >= m * ((n + 7) // 8)
    lib._Z4packPKiPiii(_ptr(src), _ptr(dst), m, n)


def unpack(src: np.ndarray, dst: np.ndarray, m: int, n: int) -> None:
    """Host unpacker: inverse of pack."""
    lib = _lib.load()
    assert src.dtype == np.int32 and dst.dtype == np.int32
    assert src.flags.c_contiguous and dst.flags.c_contiguous
    assert src.size >= m * ((n + 7) // 8) and dst.size >= m * n
    lib._Z6unpackPKiPiii(_ptr(src), _ptr(dst), m, n)


def pack_rows(values: np.ndarray) -> np.ndarray:
    """Convenience: pack a 2-D integer array (any int dtype, values in [-8, 7]) into the
    m x ceil(n/8) int32 word layout."""
    m, n = values.shape
    src = np.ascontiguousarray(values, dtype=np.int32)
    dst = np.empty((m, (n + 7) // 8), dtype=np.int32)
    pack(src, dst, m, n)
    return dst
