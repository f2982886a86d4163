"""gemm_kernels' Python surface without a GPU: names, keywords and the argument contract of the
reference's launcher (kernels/gemm_kernels/__init__.cpp:7-8, sm90a/gemm_test.cu:15-41).  All of
these checks fire before the first HIP call."""
import pytest
import torch

import gemm_kernels


def _abc(M=256, N=256, K=64, dtype=torch.bfloat16):
    return (torch.zeros(M, K, dtype=dtype), torch.zeros(N, K, dtype=dtype),
            torch.zeros(M, N, dtype=dtype))


def test_surface():
    import gemm_kernels._C as _C
    assert gemm_kernels.gemm_tn_test is _C.gemm_tn_test
    doc = _C.gemm_tn_test.__doc__
    assert "A:" in doc and "B:" in doc and "C:" in doc
    assert gemm_kernels.version() >= 1


def test_keywords_accepted_and_cpu_tensors_rejected_last():
    A, B, C = _abc()
    with pytest.raises(RuntimeError, match="HIP device"):
        gemm_kernels.gemm_tn_test(A=A, B=B, C=C)


@pytest.mark.parametrize("mutate,msg", [
    (lambda A, B, C: (A.t().contiguous().t(), B, C), "contiguous"),
    (lambda A, B, C: (A[None], B, C), "2D"),
    (lambda A, B, C: (A, B[:, :32].contiguous(), C), "Inner dimensions"),
    (lambda A, B, C: (A.float(), B.float(), C), "bfloat16 or float16"),
    (lambda A, B, C: (A, B.half(), C), "same dtype"),
    (lambda A, B, C: (A, B, C.half()), "dtype of A and B"),
    (lambda A, B, C: (A, B, C[:128]), "shape"),
    (lambda A, B, C: (A, B, torch.zeros(256, 512, dtype=C.dtype)[:, ::2]), "last dimension"),
])
def test_contract_violations(mutate, msg):
    A, B, C = mutate(*_abc())
    with pytest.raises(RuntimeError, match=msg):
        gemm_kernels.gemm_tn_test(A, B, C)


def test_variant_argument():
    A, B, C = _abc()
    with pytest.raises(RuntimeError, match="unknown variant"):
        gemm_kernels.gemm_tn(A, B, C, "fastest")
    A, B, C = _abc(K=68)
    with pytest.raises(RuntimeError, match="constraint"):
        gemm_kernels.gemm_tn(A, B, C, variant="basic")
    with pytest.raises(RuntimeError, match="HIP device"):  # auto falls back to the simple kernel
        gemm_kernels.gemm_tn(A, B, C)
    A, B, C = _abc(M=512)
    with pytest.raises(RuntimeError, match="constraint"):
        gemm_kernels.gemm_tn(A, B, C, variant="skinny")


def test_fp8_contract():
    A = torch.zeros(256, 128, dtype=torch.float8_e4m3fn)
    C = torch.zeros(256, 256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="HIP device"):
        gemm_kernels.gemm_tn_fp8(A, A, 1.0, torch.tensor(2.0), C)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        gemm_kernels.gemm_tn_fp8(A.view(torch.uint8).bfloat16(), A.view(torch.uint8).bfloat16(), 1.0, 1.0, C)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        gemm_kernels.gemm_tn_fp8(A, A, 1.0, 1.0, C.float())
    with pytest.raises(RuntimeError, match="one element"):
        gemm_kernels.gemm_tn_fp8(A, A, torch.ones(2), 1.0, C)


def test_mxfp8_contract():
    A = torch.zeros(256, 256, dtype=torch.float8_e4m3fn)
    s = torch.full((256, 8), 127, dtype=torch.uint8)
    C = torch.zeros(256, 256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="HIP device"):
        gemm_kernels.gemm_tn_mxfp8(A_q=A, B_q=A, scale_a=s, scale_b=s.view(torch.float8_e8m0fnu), C=C)
    with pytest.raises(RuntimeError, match="float8_e4m3fn"):
        gemm_kernels.gemm_tn_mxfp8(A.view(torch.uint8), A.view(torch.uint8), s, s, C)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        gemm_kernels.gemm_tn_mxfp8(A, A, s, s, C.float())
    with pytest.raises(RuntimeError, match="constraint"):                 # K % 128
        gemm_kernels.gemm_tn_mxfp8(A[:, :160].contiguous(), A[:, :160].contiguous(), s[:, :5], s[:, :5], C)
    with pytest.raises(RuntimeError, match="multiple of the MX block"):
        gemm_kernels.gemm_tn_mxfp8(A[:, :48].contiguous(), A[:, :48].contiguous(), s, s, C)
    with pytest.raises(RuntimeError, match="HIP device"):
        gemm_kernels.quantize_mxfp8(torch.zeros(4, 64))
    with pytest.raises(RuntimeError, match="multiple of the MX block"):
        gemm_kernels.quantize_mxfp8(torch.zeros(4, 48))
    with pytest.raises(RuntimeError, match="HIP device"):
        gemm_kernels.shuffle_mx_scales(s)


def test_mx_quantizer_in_torch_ops_matches_the_oracle():
    """The package's torch-op MX quantiser (used for CPU tensors) against the oracle's restatement."""
    from gemm_kernels import quant
    from oracle import oracle
    g = torch.Generator().manual_seed(1)
    x = torch.randn(40, 256, generator=g) * torch.exp2(torch.randint(-15, 15, (40, 1), generator=g).float())
    x[3, 32:64] = 0
    q, s = quant.quantize_mxfp8(x)
    wq, ws = oracle.quantize_mxfp8(x)
    assert torch.equal(s, ws) and torch.equal(q.view(torch.uint8), wq.view(torch.uint8))


def test_select_variant():
    assert gemm_kernels.select_variant(8192, 8192, 8192, torch.bfloat16) in ("basic", "pingpong")
    assert gemm_kernels.select_variant(100, 30, 77, torch.float16) == "simple"
    assert gemm_kernels.select_variant(64, 14336, 4096, torch.bfloat16) == "skinny"
    with pytest.raises(RuntimeError):
        gemm_kernels.select_variant(1, 1, 1, torch.float32)


def test_product_never_imports_the_oracle():
    import os
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cute-examples_amd")
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, os.path.join(dirpath, f)
