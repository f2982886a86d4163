"""Pins every function of oracle/ against a source that is independent of it: exhaustive
bit-pattern sweeps against torch's dtype casts, torch.matmul in fp32 (the reference's own ground
truth, kernels/tests/gemm_test.py:36), a numpy float64 product, and the closed-form fixtures in
tests/golden/.  CPU only."""
import numpy as np
import pytest
import torch

from oracle import oracle


def test_decode_bf16_exhaustive():
    b = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).float().numpy()
    got = oracle.c_decode(b, oracle.BF16)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_decode_f16_exhaustive():
    b = np.arange(65536, dtype=np.uint16)
    want = torch.from_numpy(b.view(np.int16)).view(torch.float16).float().numpy()
    got = oracle.c_decode(b, oracle.F16)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_decode_e4m3_exhaustive():
    b = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(b).view(torch.float8_e4m3fn).float().numpy()
    got = oracle.c_decode(b, oracle.E4M3)
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert got[0x7e] == 448.0 and got[0x01] == 2.0 ** -9


def _sweep_f32():
    """Values around every rounding boundary of the 16-bit formats plus random bit patterns."""
    rng = np.random.default_rng(7)
    rand = rng.integers(0, 2 ** 32, size=400000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    # every bf16 value +- {0, half ulp, half ulp +- 1 fp32 ulp}: exercises ties both ways
    hi = (np.arange(65536, dtype=np.uint32) << 16)
    ties = np.concatenate([hi, hi | 0x8000, hi | 0x7fff, hi | 0x8001]).view(np.float32)
    # fp16 ties: fp32 values with 13 dropped bits = 0x1000 (half), incl. subnormal range
    h = np.arange(0, 0x47800000, 0x1000, dtype=np.uint32)
    small = np.linspace(0, 2.0 ** -13, 20001, dtype=np.float32)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 65504, 65519.99, 65520, 1e-8, 2.0 ** -24,
                        2.0 ** -25, 2.0 ** -25 * 1.0001, 3.0e38, -3.0e38], dtype=np.float32)
    return np.concatenate([rand, ties, h.view(np.float32), -h.view(np.float32), small, special])


@pytest.mark.parametrize("code,dtype", [(oracle.BF16, torch.bfloat16), (oracle.F16, torch.float16)])
def test_round_16bit_matches_torch(code, dtype):
    x = _sweep_f32()
    want = torch.from_numpy(x).to(dtype).view(torch.int16).numpy().view(np.uint16)
    got = oracle.c_round(x, code)
    nan = np.isnan(x)
    # NaN payloads are not specified; both must stay NaN.
    back = torch.from_numpy(got.view(np.int16)).view(dtype).float().numpy()
    assert np.all(np.isnan(back[nan]))
    assert np.array_equal(got[~nan], want[~nan])


def test_round_e4m3_matches_torch_in_range_and_saturates():
    rng = np.random.default_rng(11)
    x = np.concatenate([rng.uniform(-448, 448, 200000), rng.normal(0, 1, 200000),
                        rng.normal(0, 0.01, 100000), np.linspace(-0.02, 0.02, 40001),
                        # every midpoint between neighbouring e4m3 values (ties)
                        _e4m3_midpoints()]).astype(np.float32)
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = oracle.c_round(x, oracle.E4M3)
    assert np.array_equal(got, want)
    sat = oracle.c_round(np.array([448.0, 449.0, 1e9, -1e9, np.inf, -np.inf], dtype=np.float32), oracle.E4M3)
    assert list(sat) == [0x7e, 0x7e, 0x7e, 0xfe, 0x7e, 0xfe]
    assert oracle.c_round(np.array([np.nan], dtype=np.float32), oracle.E4M3)[0] & 0x7f == 0x7f


def _e4m3_midpoints():
    v = torch.arange(0, 0x7f, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    mid = (v[:-1] + v[1:]) / 2
    return np.concatenate([mid, -mid])


def test_quantizer_matches_torch_e4m3_cast():
    """The per-tensor quantiser against torch's own ops, restated here: scale = amax / 448 in fp32
    (a tensor divisor, as a division and not a multiplication by the reciprocal), clamp to +-448,
    torch's float8_e4m3fn cast (round to nearest even)."""
    for seed, std in [(0, 1.0), (1, 0.02), (2, 37.0)]:
        x = torch.randn(257, 129, generator=torch.Generator().manual_seed(seed)) * std
        q_o, s_o = oracle.quantize_e4m3(x)
        scale = x.abs().amax() / torch.tensor(448.0)
        q_t = (x / scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
        assert s_o == float(scale)
        assert torch.equal(q_o.view(torch.uint8), q_t.view(torch.uint8))
        assert float(q_o.float().abs().max()) == 448.0
    q, s = oracle.quantize_e4m3(torch.zeros(4, 4))
    assert s == 1.0 and not q.float().any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
def test_c_gemm_against_numpy_float64_and_torch_fp32(dtype):
    g = torch.Generator().manual_seed(3)
    M, N, K = 70, 45, 200
    A = torch.randn(M, K, generator=g).to(dtype)
    B = torch.randn(N, K, generator=g).to(dtype)
    scale = 0.37 if dtype == torch.float8_e4m3fn else 1.0
    exact = (A.double().numpy() @ B.double().numpy().T) * np.float32(scale).astype(np.float64)
    got = oracle.c_gemm_tn_f32(A, B, scale).numpy()
    # double accumulation of exact products: only the final fp32 rounding separates them
    assert np.array_equal(got, exact.astype(np.float32))
    ref = oracle.gemm_tn_fp32(A, B, scale)
    assert oracle.rel_frobenius(torch.from_numpy(got), ref) < 1e-6
    # a transposed operand, a dropped k term or a wrong stride cannot pass this:
    assert oracle.rel_frobenius(oracle.c_gemm_tn_f32(A, B.flip(0), scale), ref) > 0.5
    out_dtype = torch.bfloat16 if dtype == torch.float8_e4m3fn else dtype
    rounded = oracle.c_gemm_tn(A, B, out_dtype, scale)
    assert torch.equal(rounded.view(torch.int16), torch.from_numpy(exact.astype(np.float32)).to(out_dtype).view(torch.int16))


def test_c_gemm_bruteforce_tiny():
    """Pure-Python triple loop at 5x4x7."""
    g = torch.Generator().manual_seed(5)
    A = torch.randn(5, 7, generator=g).bfloat16()
    B = torch.randn(4, 7, generator=g).bfloat16()
    want = [[sum(float(A[m, k]) * float(B[n, k]) for k in range(7)) for n in range(4)] for m in range(5)]
    got = oracle.c_gemm_tn_f32(A, B)
    assert torch.equal(got, torch.tensor(want, dtype=torch.float64).float())


CASES = ["identity", "ones", "onehot", "integers"]
DTYPES = {"bf16": torch.bfloat16, "f16": torch.float16, "e4m3": torch.float8_e4m3fn}


def _load(golden, case, name):
    dt = DTYPES[name]
    A = torch.from_numpy(golden[f"{case}/{name}/A"]).view(dt)
    B = torch.from_numpy(golden[f"{case}/{name}/B"]).view(dt)
    out_dt = torch.bfloat16 if name == "e4m3" else dt
    C = torch.from_numpy(golden[f"{case}/{name}/C"]).view(out_dt)
    return A, B, C, float(golden[f"{case}/{name}/scale"])


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("name", list(DTYPES))
def test_oracle_reproduces_closed_forms(golden, case, name):
    A, B, C, scale = _load(golden, case, name)
    got = oracle.c_gemm_tn(A, B, C.dtype, scale)
    assert torch.equal(got.view(torch.int16), C.view(torch.int16))
    assert torch.equal(oracle.gemm_tn_fp32(A, B, scale).to(C.dtype).view(torch.int16), C.view(torch.int16))


def test_metrics():
    label = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    assert oracle.rel_frobenius(label, label) == 0.0
    assert abs(oracle.rel_frobenius(label * 1.01, label) - 0.01) < 1e-6
    assert oracle.reference_accepts(label + 0.009, label)
    assert not oracle.reference_accepts(label + 0.2, label)
    assert oracle.no_nan_left(label) and not oracle.no_nan_left(label / torch.tensor(0.0) * 0)


# --- MX block scaling ------------------------------------------------------------------------------

def test_mx_quantizer_closed_forms():
    """Blocks whose quantisation the format fixes by hand (OCP MX v1.0, 6.3)."""
    x = torch.zeros(4, 64)
    x[0, :32] = torch.tensor([2.0 ** k for k in range(-10, 22)])       # amax 2^21 -> shared exp 13
    x[0, 32:] = 0.0                                                     # zeros -> scale 1
    x[1, :32] = 448.0                                                   # amax 448 -> 2^0, elements 448
    x[1, 32:] = torch.linspace(-500.0, 500.0, 32)                       # amax 500 -> 2^0, |x|>448 saturates
    x[2, :32] = 1.0
    x[2, 32] = 3.0e-5                                                   # floor(log2)=-16 -> shared -24
    x[3, 0] = -255.9999                                                 # amax in [128,256) -> 2^-1
    q, s = oracle.quantize_mxfp8(x)
    qf = q.float()
    assert s[0, 0] == 127 + 13 and s[0, 1] == 127
    # elements 2^k / 2^13 for k = -10..21: below 2^-9 they vanish or hit the subnormal grid
    want = torch.tensor([2.0 ** (k - 13) for k in range(-10, 22)])
    want[want < 2.0 ** -10] = 0.0
    want[(want >= 2.0 ** -10) & (want < 2.0 ** -9)] = 0.0              # 2^-10 is a tie between 0 and 2^-9 -> even (0)
    assert torch.equal(qf[0, :32], want)
    assert s[1, 0] == 127 and torch.all(qf[1, :32] == 448.0)
    assert s[1, 1] == 127 and qf[1, 32] == -448.0 and qf[1, 63] == 448.0
    assert s[2, 0] == 127 - 8 and torch.all(qf[2, :32] == 256.0)
    assert s[2, 1] == 127 - 24 and qf[2, 32] == 448.0                  # 3e-5 * 2^24 = 503.3 saturates
    assert s[3, 0] == 127 - 1 and qf[3, 0] == -448.0                   # 511.9998 saturates


def test_mx_scale_and_element_decoders_match_torch():
    """The byte -> value maps against torch's own float8_e8m0fnu and float8_e4m3fn decoders."""
    b = torch.arange(0, 255, dtype=torch.uint8)                         # 255 is NaN in E8M0
    want = b.view(torch.float8_e8m0fnu).float().double()
    q = torch.full((255, 32), 1.0).to(torch.float8_e4m3fn)
    got = oracle.dequantize_mxfp8(q, b.reshape(255, 1)).double()[:, 0]
    ok = want >= 2.0 ** -126                                            # fp32 output: the smallest scales are subnormal
    assert torch.equal(got[ok], want[ok])
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 256, size=(8, 64), dtype=np.uint8)
    bits[(bits & 0x7f) == 0x7f] = 0
    qq = torch.from_numpy(bits).view(torch.float8_e4m3fn)
    sc = torch.from_numpy(rng.integers(110, 140, size=(8, 2), dtype=np.uint8))
    want = qq.float().reshape(8, 2, 32) * sc.view(torch.float8_e8m0fnu).float()[..., None]
    assert torch.equal(oracle.dequantize_mxfp8(qq, sc), want.reshape(8, 64))


def test_mx_quantizer_invariants():
    """Properties the conversion must have whatever the data: the largest element of every block
    lands in the top binade [256, 448], scaling a block by 2^k moves only the scale byte, and the
    round trip stays within half an e4m3 ulp of the block's top binade (2^-4 of 2^(e+8)... ) except
    where saturation (amax in (448, 512) * 2^e) applies."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(64, 256, generator=g) * torch.exp2(torch.randint(-20, 20, (64, 1), generator=g).float())
    q, s = oracle.quantize_mxfp8(x)
    top = q.float().abs().reshape(64, 8, 32).amax(-1)
    assert torch.all((top >= 256.0) & (top <= 448.0))
    q2, s2 = oracle.quantize_mxfp8(x * 8.0)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s + 3)
    back = oracle.dequantize_mxfp8(q, s)
    unit = torch.exp2(s.float() - 127.0).repeat_interleave(32, dim=1)    # value of one unit of x/scale
    err = (back - x).abs() / unit
    scaled = (x / unit).abs()
    assert torch.all(err[scaled <= 448.0] <= 16.0 + 1e-3)                # half an ulp of [256, 512): 32/2
    assert torch.all(err[scaled > 448.0] <= 64.0)                        # saturated from below 512
    # e4m3 keeps 4 significant bits: relative error of normal values <= 2^-4
    normal = scaled >= 2.0 ** -6
    assert torch.all(((back - x).abs() / x.abs())[normal & (scaled <= 448.0)] <= 2.0 ** -4 + 1e-6)


def test_mx_gemm_bruteforce_exact():
    """The block-scaled product against exact rational arithmetic on a tiny case."""
    from fractions import Fraction
    rng = np.random.default_rng(11)
    M, N, K = 3, 4, 64
    def operand(rows):
        bits = rng.integers(0, 256, size=(rows, K), dtype=np.uint8)
        bits[(bits & 0x7f) == 0x7f] = 0x30
        bits[(bits & 0x78) > 0x50] &= 0x3f                                # keep products exact in fp32 sums
        return torch.from_numpy(bits).view(torch.float8_e4m3fn), \
            torch.from_numpy(rng.integers(120, 134, size=(rows, K // 32), dtype=np.uint8))
    A, sa = operand(M)
    B, sb = operand(N)
    got = oracle.gemm_tn_mxfp8_fp32(A, sa, B, sb).double()
    Af, Bf = A.float().numpy(), B.float().numpy()
    for m in range(M):
        for n in range(N):
            acc = Fraction(0)
            for k in range(K):
                acc += Fraction(float(Af[m, k])) * Fraction(float(Bf[n, k])) * \
                    Fraction(2) ** (int(sa[m, k // 32]) - 127) * Fraction(2) ** (int(sb[n, k // 32]) - 127)
            assert abs(float(acc) - float(got[m, n])) <= 1e-5 * max(1.0, abs(float(acc))), (m, n)
