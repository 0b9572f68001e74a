"""Python loader of the MI355X block-scaled FP8 GEMM library (libfp8gemm.so).

The directory name contains a hyphen, so the package is loaded by path: the repository's
__graft_entry__.load_package() registers it as module ``fp8_quant_matmul_amd``.
Everything numerical happens in the HIP library behind the C ABI declared in
include/fp8_block_gemm.h; this module only declares the ctypes prototypes and offers
pointer-level helpers for torch tensors.  There is no CPU fallback: a missing library or
a failing call raises.
"""
from .capi import (  # noqa: F401
    Fp8GemmError, Options,
    KERNEL_AUTO, KERNEL_SCALAR, KERNEL_LARGE, KERNEL_SPLITK, KERNEL_SKINNY,
    DTYPE_BF16, DTYPE_F32, DTYPE_BF16_F32MATH, FLAG_WORKSPACE_ZEROED, WORKSPACE_HEADER_BYTES,
    quantize_a_1x128, quantize_b_128x128,
    abi_symbols, build, convert_f32_to_e4m3fn, custom_kernel, error_string, force_config, gemm, gemm_ex, gemm_grouped, gemm_grouped_ex, gemm_noalloc, gemm_scalar, NOALLOC_MAX_BYTES,
    grouped_workspace_bytes, workspace_bytes_ex,
    last_kernel, lib, lib_path, plan, release, select, set_fused_reduction, set_persistent, set_workspace, workspace_bytes,
)
