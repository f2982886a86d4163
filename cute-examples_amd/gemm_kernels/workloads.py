"""Seeded synthetic operands for the five benchmark configurations of this library.

Every generator returns K-contiguous operands in the layout gemm_tn_test takes: A (M,K) and
B (N,K).  Shapes and distributions:

  fp16_512      fp16, M=N=K=512, entries Normal(0,1)/sqrt(K)
  bf16_4096     bf16, M=N=K=4096, entries Uniform(-1,1)
  bf16_8192     bf16, M=N=K=8192, entries Normal(0,1)
  skinny        bf16, activations X (M,K) Normal(0,1), weights W (N,K) Normal(0,0.02),
                M in {16,64,256}, (N,K) in {(14336,4096),(4096,14336),(6144,4096)}
  fp8_8192      e4m3, M=N=K=8192, quantised from Normal(0,1) with per-tensor scales amax/448
  mxfp8_8192    e4m3 + E8M0 block scales (OCP MX), M=N=K=8192, quantised from Normal(0,1)

The reference's own test draws unseeded torch.randn bf16 squares of side 4096/2048/1024
(kernels/tests/gemm_test.py:15,23-24); `reference_test_shapes` keeps that list.
"""
import torch

from .quant import quantize_e4m3, quantize_mxfp8

reference_test_shapes = [(4096, 4096), (2048, 2048), (1024, 1024)]

SKINNY_M = (16, 64, 256)
SKINNY_NK = ((14336, 4096), (4096, 14336), (6144, 4096))


def _gen(seed, device):
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


def normal(shape, seed, device="cpu", std=1.0, dtype=torch.bfloat16):
    x = torch.randn(shape, generator=_gen(seed, device), device=device, dtype=torch.float32)
    if std != 1.0:
        x.mul_(std)
    return x.to(dtype)


def uniform_pm1(shape, seed, device="cpu", dtype=torch.bfloat16):
    x = torch.rand(shape, generator=_gen(seed, device), device=device, dtype=torch.float32)
    return x.mul_(2.0).sub_(1.0).to(dtype)


def fp16_512(seed=0, device="cpu", size=512):
    s = size ** -0.5
    return (normal((size, size), seed, device, s, torch.float16),
            normal((size, size), seed + 1, device, s, torch.float16))


def bf16_4096(seed=0, device="cpu", size=4096):
    return uniform_pm1((size, size), seed, device), uniform_pm1((size, size), seed + 1, device)


def bf16_8192(seed=0, device="cpu", size=8192):
    return normal((size, size), seed, device), normal((size, size), seed + 1, device)


def skinny(M, N, K, seed=0, device="cpu"):
    """(X, W): activations (M,K) ~ Normal(0,1), weights (N,K) ~ Normal(0,0.02)."""
    return normal((M, K), seed, device), normal((N, K), seed + 1, device, 0.02)


def fp8_8192(seed=0, device="cpu", size=8192):
    """(A_q, B_q, scale_a, scale_b) with A_q, B_q float8_e4m3fn and 0-dim fp32 scales."""
    a = normal((size, size), seed, device, dtype=torch.float32)
    a_q, sa = quantize_e4m3(a)
    del a
    b = normal((size, size), seed + 1, device, dtype=torch.float32)
    b_q, sb = quantize_e4m3(b)
    return a_q, b_q, sa, sb


def mxfp8_8192(seed=0, device="cpu", size=8192):
    """(A_q, scale_a, B_q, scale_b): float8_e4m3fn operands with uint8 E8M0 block scales (rows, K/32)."""
    a = normal((size, size), seed, device, dtype=torch.float32)
    a_q, sa = quantize_mxfp8(a)
    del a
    b = normal((size, size), seed + 1, device, dtype=torch.float32)
    b_q, sb = quantize_mxfp8(b)
    return a_q, sa, b_q, sb
