"""Per-tensor fp8 quantisation: the host-side step in front of gemm_tn_fp8.

scale = amax(|x|) / 448 in fp32, x_q = (x / scale) cast to float8_e4m3fn (OCP e4m3, max 448),
so that x ~= scale * x_q.  Pure torch ops; runs on whatever device x lives on.  The reference
has no fp8 path; the contract is the one the build's fp8 configuration states (operands
quantised from Normal(0,1) with per-tensor fp32 scales amax/448).
"""
import torch

E4M3_MAX = 448.0


def quantize_e4m3(x):
    """Returns (x_q, scale): x_q float8_e4m3fn with x's shape, scale a 0-dim fp32 tensor."""
    xf = x.detach().float()
    amax = xf.abs().amax()
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    # Clamp before the cast: torch's e4m3fn cast maps values that round above 448 to NaN.
    x_q = (xf / scale).clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return x_q, scale
