"""CPU oracle for the GEMM path — TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module, and
only as the checker.  The shipped package (cute-examples_amd/) never imports it.

Two independent restatements of what the reference computes are offered:

* ``gemm_tn_fp32`` — the reference's own ground truth, ``torch.matmul(A.float(), B.float().T)``
  in fp32 on the CPU (kernels/tests/gemm_test.py:36).
* ``c_gemm_tn`` / ``c_gemm_tn_f32`` — the plain-C restatement in oracle/gemm_oracle.c
  (double accumulation, RNE down-conversion as in gemm.cuh:368-377), loaded with ctypes.

plus the reference test's acceptance checks (gemm_test.py:4-11, :28) and the relative Frobenius
error the build's tolerance is stated in.
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "liboracle.so")

BF16, F16, E4M3 = 0, 1, 2
_TORCH_TO_CODE = {torch.bfloat16: BF16, torch.float16: F16, torch.float8_e4m3fn: E4M3}
_CODE_TO_TORCH = {v: k for k, v in _TORCH_TO_CODE.items()}

_lib = None


def build():
    """Compile oracle/gemm_oracle.c with gcc (used by __graft_entry__.build())."""
    subprocess.run(["make", "-C", HERE, "-B"], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        i64, vp, f32, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
        L.oracle_gemm_tn_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, f32]
        L.oracle_gemm_tn_f32.restype = ci
        L.oracle_gemm_tn.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, f32]
        L.oracle_gemm_tn.restype = ci
        L.oracle_decode_array.argtypes = [vp, vp, i64, ci]
        L.oracle_decode_array.restype = None
        L.oracle_round_array.argtypes = [vp, vp, i64, ci]
        L.oracle_round_array.restype = None
        _lib = L
    return _lib


def _cpu2d(t):
    assert t.dim() == 2 and t.device.type == "cpu" and t.is_contiguous()
    return t


def c_gemm_tn_f32(A, B, scale=1.0):
    """fp32 tensor (M,N) = scale * A @ B.T via the C oracle (double accumulation)."""
    A, B = _cpu2d(A), _cpu2d(B)
    M, K = A.shape
    N = B.shape[0]
    assert B.shape[1] == K and A.dtype == B.dtype
    C = torch.empty((M, N), dtype=torch.float32)
    rc = lib().oracle_gemm_tn_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, K, N,
                                  _TORCH_TO_CODE[A.dtype], float(scale))
    assert rc == 0
    return C


def c_gemm_tn(A, B, out_dtype=None, scale=1.0):
    """(M,N) tensor of out_dtype = rne(scale * A @ B.T) via the C oracle."""
    A, B = _cpu2d(A), _cpu2d(B)
    M, K = A.shape
    N = B.shape[0]
    out_dtype = out_dtype or A.dtype
    C = torch.empty((M, N), dtype=out_dtype)
    rc = lib().oracle_gemm_tn(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, K, K, N,
                              _TORCH_TO_CODE[A.dtype], _TORCH_TO_CODE[out_dtype], float(scale))
    assert rc == 0
    return C


def c_decode(bits, dtype_code):
    """uint16/uint8 numpy bit patterns -> float32 numpy via the C decoders."""
    bits = np.ascontiguousarray(bits)
    out = np.empty(bits.shape, dtype=np.float32)
    lib().oracle_decode_array(bits.ctypes.data, out.ctypes.data, bits.size, dtype_code)
    return out


def c_round(values, dtype_code):
    """float32 numpy -> uint16/uint8 bit patterns via the C rounders (RNE; e4m3 saturating)."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, dtype=np.uint8 if dtype_code == E4M3 else np.uint16)
    lib().oracle_round_array(values.ctypes.data, out.ctypes.data, values.size, dtype_code)
    return out


def gemm_tn_fp32(A, B, scale=1.0):
    """The reference test's ground truth (gemm_test.py:36): fp32 matmul on the CPU."""
    C = torch.matmul(A.cpu().float(), B.cpu().float().T)
    return C * scale if scale != 1.0 else C


def rel_frobenius(pred, label):
    """||pred - label||_F / ||label||_F in float64."""
    p, l = pred.detach().cpu().double(), label.detach().cpu().double()
    return float((p - l).norm() / l.norm().clamp_min(1e-300))


def reference_accepts(pred, label):
    """The reference's acceptance test (gemm_test.py:10): allclose(atol=1e-2, rtol=1e-2)."""
    return bool(torch.allclose(pred.detach().cpu().float(), label.detach().cpu().float(),
                               atol=1e-2, rtol=1e-2))


def no_nan_left(C):
    """The output was NaN-prefilled (gemm_test.py:28); any NaN left marks an unwritten element."""
    return not bool(torch.isnan(C.detach().cpu().float()).any())


def quantize_e4m3(x):
    """Per-tensor e4m3 quantisation restated with the C rounder: scale = amax/448 (fp32),
    x_q = e4m3_rne_sat(x / scale).  Returns (x_q as float8_e4m3fn tensor, scale as float)."""
    x = x.detach().cpu().float().contiguous()
    amax = float(x.abs().max())
    scale = np.float32(amax) / np.float32(448.0) if amax > 0 else np.float32(1.0)
    q = c_round((x.numpy() / scale).astype(np.float32), E4M3)
    return torch.from_numpy(q).view(torch.float8_e4m3fn).reshape(x.shape), float(scale)


# --- OCP MX block scaling (MXFP8) -----------------------------------------------------------------
# The reference has no fp8 path; these restate the published format (OCP Microscaling Formats (MX)
# specification v1.0: section 5.1 block = 32 elements sharing an E8M0 scale 2^(byte-127); section
# 6.3 conversion: shared exponent floor(log2(amax)) - emax_elem, emax_elem = 8 for e4m3, elements
# x / scale rounded to nearest even and saturated).  Pinned in tests/test_oracle.py by closed-form
# blocks, torch's float8_e8m0fnu / float8_e4m3fn decoders and an exact rational brute force.

MX_BLOCK = 32
E4M3_EMAX = 8


def quantize_mxfp8(x):
    """x (rows, K) float tensor, K % 32 == 0 -> (x_q float8_e4m3fn (rows, K), scales uint8 (rows, K/32))."""
    x = x.detach().cpu().float().contiguous()
    rows, K = x.shape
    assert K % MX_BLOCK == 0
    blocks = x.numpy().reshape(rows, K // MX_BLOCK, MX_BLOCK).astype(np.float64)
    amax = np.abs(blocks).max(axis=-1)
    with np.errstate(divide="ignore"):
        shared = np.floor(np.log2(amax)) - E4M3_EMAX          # -inf for a block of zeros
    byte = np.where(amax > 0, np.clip(shared + 127, 0, 254), 127).astype(np.int64)
    scaled = blocks * np.exp2(127.0 - byte)[..., None]          # exact: a power of two
    q = c_round(scaled.astype(np.float32).reshape(rows, K), E4M3)
    return (torch.from_numpy(q).view(torch.float8_e4m3fn).reshape(rows, K),
            torch.from_numpy(byte.astype(np.uint8)))


def dequantize_mxfp8(x_q, scales):
    """(float8_e4m3fn (rows, K), uint8 (rows, K/32)) -> float32 (rows, K), exact."""
    rows, K = x_q.shape
    vals = c_decode(x_q.detach().cpu().contiguous().view(torch.uint8).numpy(), E4M3).astype(np.float64)
    s = np.exp2(scales.detach().cpu().view(torch.uint8).numpy().astype(np.float64) - 127.0)
    out = vals.reshape(rows, K // MX_BLOCK, MX_BLOCK) * s[..., None]
    return torch.from_numpy(out.reshape(rows, K).astype(np.float32))


def gemm_tn_mxfp8_fp32(A_q, scale_a, B_q, scale_b):
    """Ground truth of the block-scaled GEMM: fp32 matmul of the dequantised operands
    (the reference test's ground truth, gemm_test.py:36, applied to what the operands mean)."""
    return torch.matmul(dequantize_mxfp8(A_q, scale_a), dequantize_mxfp8(B_q, scale_b).T)
