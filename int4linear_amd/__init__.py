"""MI355X (gfx950) signed-int4 linear-layer GEMM behind the Int4Linear host API.

The compute lives in ``lib/libint4linear.so`` (HIP kernels + C ABI, declared in
``include/int4linear.h``); this package is the thin host-side mirror of the reference's
``linear_vN_launch`` / ``pack`` / ``unpack`` interface.
"""
from .api import (  # noqa: F401
    fp6_convert,
    fp6_operand_bytes,
    gemm_fp6_converted,
    gemm_s4s4s32,
    gemm_s4s4s32_static,
    init,
    kernel_for_shape,
    linear_bf16,
    linear_f16,
    linear_f32,
    linear_fp6_converted,
    linear_s32,
    linear_v0_launch,
    linear_v1_launch,
    linear_v2_launch,
    linear_v10_launch,
    linear_v11_launch,
    linear_v20_launch,
    linear_v21_launch,
    pack,
    pack_device,
    pack_rows,
    release_workspace,
    set_workspace_limit,
    unpack,
    unpack_device,
    workspace_bytes,
)
from ._lib import Int4LinearError  # noqa: F401
