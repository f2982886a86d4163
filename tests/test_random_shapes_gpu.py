"""Seeded random problems through the C ABI: shapes, row strides, variants, scales, output types and
workspaces drawn at random inside what each entry point accepts, every result compared with the
fp32 product of the (dequantised) operands computed by torch on the same device.

The hand-picked shapes of the other GPU tests cover the known edges; this one looks for the edges
nobody thought of.  Tolerances as everywhere: relative Frobenius error <= 1e-2 for bf16/fp16
inputs, <= 3e-2 for fp8 and block-scaled fp8; C is prefilled with NaN (gemm_test.py:28) and
everything outside its M x N window, padding columns and rows behind it, must still be NaN."""
import random

import pytest
import torch

from tests import abi_ctypes as ac

pytestmark = pytest.mark.gpu

INPUTS = [(torch.bfloat16, ac.BF16, 2, 1e-2), (torch.float16, ac.F16, 2, 1e-2), (torch.float8_e4m3fn, ac.E4M3, 1, 3e-2)]


def window(M, N, ldc, dtype):
    full = torch.full((M + 4, ldc), float("nan"), dtype=dtype, device="cuda")
    return full, full[:M, :N]


def judge(full, C, ref, M, N, tol, what):
    out = C.float()
    assert not torch.isnan(out).any(), what
    assert torch.isnan(full[M:].float()).all() and torch.isnan(full[:M, N:].float()).all(), "wrote outside C: " + what
    err = float((out - ref).norm() / (ref.norm() + 1e-30))
    assert err <= tol, (err, what)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_problems_against_fp32_matmul(abi, seed):
    rng = random.Random(seed)
    stream = torch.cuda.current_stream().cuda_stream
    for it in range(250):
        tdt, code, es, tol = rng.choice(INPUTS)
        per16 = 16 // es
        M = rng.choice([rng.randint(1, 40), rng.randint(1, 300), rng.randint(1, 3000)])
        N = 4 * rng.choice([rng.randint(1, 40), rng.randint(1, 400), rng.randint(1, 1500)])
        K = per16 * rng.choice([rng.randint(1, 16), rng.randint(1, 200), rng.randint(1, 1100)])
        lda, ldb, ldc = K + per16 * rng.choice([0, 0, 1, 5]), K + per16 * rng.choice([0, 0, 2, 7]), N + 4 * rng.choice([0, 0, 1, 9])
        v = rng.choice([ac.AUTO, ac.BASIC, ac.PINGPONG] + ([ac.ALTERNATE] if es == 2 else []) + ([ac.SKINNY] if M <= 256 else []))
        if v == ac.AUTO and rng.random() < 0.4:   # AUTO takes anything: the generic kernel, or repacking
            N, K = max(1, N - rng.randint(0, 3)), max(1, K - rng.randint(0, per16 - 1))
            lda, ldb, ldc = K + rng.choice([0, 0, 1, 5]), K + rng.choice([0, 0, 3]), N + rng.choice([0, 0, 1, 3])
        scale = rng.choice([1.0, 0.5, 0.37])
        odt = rng.choice([torch.bfloat16, torch.float16])
        g = torch.Generator(device="cuda").manual_seed(1000 * seed + it)
        A = torch.randn(M, lda, device="cuda", generator=g).clamp_(-200, 200).to(tdt)[:, :K]
        B = torch.randn(N, ldb, device="cuda", generator=g).clamp_(-200, 200).to(tdt)[:, :K]
        full, C = window(M, N, ldc, odt)
        need = abi.mi355_gemm_workspace_bytes(M, N, K, code, v)
        streams = v == ac.SKINNY or (v == ac.AUTO and abi.mi355_gemm_select_variant(M, N, K, code) == ac.SKINNY)
        give = bool(need) and (streams or rng.random() < 0.8)      # only the streaming kernel insists on it
        ws = torch.empty(need + 256, dtype=torch.uint8, device="cuda") if give else None
        wp = (ws.data_ptr() + 255) // 256 * 256 if give else None
        what = f"seed {seed} case {it}: {tdt} M={M} N={N} K={K} lda={lda} ldb={ldb} ldc={ldc} variant={v} scale={scale} out={odt} workspace={give}"
        rc = abi.mi355_gemm_tn(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, lda, ldb, ldc, code, ac.torch_code(odt),
                               scale, v, wp, need if give else 0, stream)
        assert rc == 0, (rc, what)
        torch.cuda.synchronize()
        judge(full, C, (A.float() @ B.float().t()) * scale, M, N, tol, what)


@pytest.mark.parametrize("seed", [21, 22])
def test_random_block_scaled_problems_against_fp32_matmul(abi, seed):
    rng = random.Random(seed)
    for it in range(150):
        M = rng.choice([rng.randint(1, 40), rng.randint(1, 300), rng.randint(1, 2500)])
        N = 4 * rng.choice([rng.randint(1, 40), rng.randint(1, 400), rng.randint(1, 1200)])
        K = 128 * rng.choice([rng.randint(1, 4), rng.randint(1, 40), rng.randint(1, 70)])
        lda, ldb, ldc = K + 16 * rng.choice([0, 0, 3]), K + 16 * rng.choice([0, 0, 8]), N + 4 * rng.choice([0, 0, 5])
        shuffled = rng.random() < 0.5
        odt = rng.choice([torch.bfloat16, torch.float16])
        g = torch.Generator(device="cuda").manual_seed(1000 * seed + it)
        Aq = torch.randn(M, lda, device="cuda", generator=g).clamp_(-100, 100).to(torch.float8_e4m3fn)[:, :K]
        Bq = torch.randn(N, ldb, device="cuda", generator=g).clamp_(-100, 100).to(torch.float8_e4m3fn)[:, :K]
        sa = torch.randint(120, 131, (M, K // 32), device="cuda", generator=g, dtype=torch.uint8)   # 2^-7 .. 2^3
        sb = torch.randint(120, 131, (N, K // 32), device="cuda", generator=g, dtype=torch.uint8)
        full, C = window(M, N, ldc, odt)
        what = f"seed {seed} case {it}: M={M} N={N} K={K} lda={lda} ldb={ldb} ldc={ldc} shuffled={shuffled} out={odt}"
        rc = ac.gemm_tn_mxfp8(abi, Aq, Bq, sa, sb, C, shuffled)
        assert rc == 0, (rc, what)
        torch.cuda.synchronize()
        da = Aq.float() * torch.exp2(sa.float() - 127).repeat_interleave(32, dim=1)
        db = Bq.float() * torch.exp2(sb.float() - 127).repeat_interleave(32, dim=1)
        judge(full, C, da @ db.t(), M, N, 3e-2, what)
