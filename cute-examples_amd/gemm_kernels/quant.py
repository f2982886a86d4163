"""fp8 quantisation: the step in front of gemm_tn_fp8 (per-tensor scales) and gemm_tn_mxfp8
(OCP MX block scales).

Per tensor:

scale = amax(|x|) / 448 in fp32, x_q = (x / scale) cast to float8_e4m3fn (OCP e4m3, max 448),
so that x ~= scale * x_q.  Tensors on a HIP device go through the library's own kernels
(gemm_kernels.quantize_e4m3, no host synchronisation); tensors on the CPU (test inputs, workload
generators) are quantised with the equivalent torch ops.  The reference has no fp8 path; the
contract is the one the build's fp8 configuration states (operands quantised from Normal(0,1)
with per-tensor fp32 scales amax/448).

MX (OCP Microscaling Formats v1.0): every 32 consecutive elements of a row share one E8M0 scale
byte, scale = 2^(byte-127) = 2^(floor(log2(amax_block)) - 8) (1 for a block of zeros), elements
x / scale rounded to nearest even into float8_e4m3fn and saturated at +-448.
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
    # A tensor divisor: with a Python scalar torch multiplies by the reciprocal on a device, one ulp off.
    scale = torch.where(amax > 0, amax / torch.full_like(amax, E4M3_MAX), torch.ones_like(amax))
    # Clamp before the cast: torch's e4m3fn cast maps values that round above 448 to NaN.
    x_q = (xf / scale).clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return x_q, scale


def quantize_mxfp8(x, shuffled=False):
    """Returns (x_q, scales): x (rows, K) -> float8_e4m3fn (rows, K), uint8 scale bytes (rows, K/32);
    with shuffled=True (HIP tensors only) the scales come back in the layout the GEMM reads."""
    if x.is_cuda and x.dtype in (torch.float32, torch.bfloat16, torch.float16):
        from ._C import quantize_mxfp8 as _native
        return _native(x.detach().contiguous(), shuffled)
    if shuffled:
        raise ValueError("shuffled scales are produced on a HIP device only")
    return quantize_mxfp8_torch(x)


def quantize_mxfp8_torch(x):
    """The same contract in torch ops, on whatever device x lives on."""
    rows, K = x.shape
    xf = x.detach().float().reshape(rows, K // 32, 32)
    amax = xf.abs().amax(-1)
    _, ex = torch.frexp(amax)                       # amax = m * 2^ex, m in [0.5, 1): floor(log2) = ex - 1
    byte = torch.where(amax > 0, (ex - 1 - 8 + 127).clamp(0, 254), torch.full_like(ex, 127))
    # 1/scale = 2^(127-byte), built from its bits (exponent field 254-byte; 2^-127 is subnormal) so that
    # the product is exact on every device: torch.ldexp goes through pow, which is not on a GPU.
    field = (254 - byte).to(torch.int32)
    inv_scale = torch.where(field > 0, field << 23, torch.full_like(field, 0x00400000)).view(torch.float32)
    scaled = xf * inv_scale[..., None]
    x_q = scaled.clamp_(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn).reshape(rows, K)
    return x_q, byte.to(torch.uint8)
