"""Per-tensor fp8 quantisation: the step in front of gemm_tn_fp8.

scale = amax(|x|) / 448 in fp32, x_q = (x / scale) cast to float8_e4m3fn (OCP e4m3, max 448),
so that x ~= scale * x_q.  Tensors on a HIP device go through the library's own kernels
(gemm_kernels.quantize_e4m3, no host synchronisation); tensors on the CPU (test inputs, workload
generators) are quantised with the equivalent torch ops.  The reference has no fp8 path; the
contract is the one the build's fp8 configuration states (operands quantised from Normal(0,1)
with per-tensor fp32 scales amax/448).
"""
import torch

E4M3_MAX = 448.0


def quantize_e4m3(x):
    """Returns (x_q, scale): x_q float8_e4m3fn with x's shape, scale a 0-dim fp32 tensor."""
    if x.is_cuda and x.dtype in (torch.float32, torch.bfloat16, torch.float16):
        from ._C import quantize_e4m3 as _native
        return _native(x.detach().contiguous())
    return quantize_e4m3_torch(x)


def quantize_e4m3_torch(x):
    """The same contract in torch ops, on whatever device x lives on."""
    xf = x.detach().float()
    amax = xf.abs().amax()
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax))
    # Clamp before the cast: torch's e4m3fn cast maps values that round above 448 to NaN.
    x_q = (xf / scale).clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return x_q, scale
