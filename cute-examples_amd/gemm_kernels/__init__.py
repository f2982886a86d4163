"""gemm_kernels — dense GEMM for AMD Instinct MI355X (gfx950).

Same package name and entry point as the reference (kernels/gemm_kernels/__init__.py:1):

    from gemm_kernels import gemm_tn_test
    gemm_tn_test(A, B, C)        # C[M,N] = A[M,K] @ B[N,K].T, returns C

plus the variant-selecting and fp8 entry points of the native module.  The native module is
required: importing this package without a built gemm_kernels/_C*.so raises ImportError.
"""
from ._C import (gemm_tn, gemm_tn_fp8, gemm_tn_mxfp8, gemm_tn_test, quantize_e4m3, quantize_mxfp8,
                 select_variant, shuffle_mx_scales, version)

__all__ = ["gemm_tn_test", "gemm_tn", "gemm_tn_fp8", "gemm_tn_mxfp8", "quantize_e4m3", "quantize_mxfp8",
           "shuffle_mx_scales", "select_variant", "version"]
