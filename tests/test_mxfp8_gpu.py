"""MX block-scaled fp8 GEMM and its quantiser on the GPU, through the C ABI and the Python module,
against the oracle's restatement of the OCP MX format.

Tolerance: relative Frobenius error <= 3e-2 against the fp32 product of the dequantised operands
(in practice ~2e-3: the products and block scales are exact, only the fp32 accumulation order and
the bf16/fp16 output rounding differ); the quantiser, the power-of-two cases and the permutation
case are bit-exact."""
import numpy as np
import ctypes

import pytest
import torch

from oracle import oracle
from tests import abi_ctypes as ac

pytestmark = pytest.mark.gpu

TOL = 3e-2


def random_mx(rows, K, seed, scale_lo=112, scale_hi=142):
    """Random e4m3 bytes (no NaN codes) and random scale bytes: every byte pattern, a wide range of scales."""
    rng = np.random.default_rng(seed)
    bits = rng.integers(0, 256, size=(rows, K), dtype=np.uint8)
    bits[(bits & 0x7f) == 0x7f] ^= 0x08
    sc = rng.integers(scale_lo, scale_hi, size=(rows, K // 32), dtype=np.uint8)
    return torch.from_numpy(bits).view(torch.float8_e4m3fn), torch.from_numpy(sc)


def run_mx(abi, A, sa, B, sb, out_dtype=torch.bfloat16, shuffled=False, ldc=None):
    M, N = A.shape[0], B.shape[0]
    guard = 8
    Cfull = torch.full((M + guard, ldc or N), float("nan"), dtype=out_dtype, device="cuda")
    C = Cfull[:M, :N]
    rc = ac.gemm_tn_mxfp8(abi, A.cuda(), B.cuda(), sa.cuda(), sb.cuda(), C, shuffled)
    assert rc == 0, abi.mi355_gemm_strerror(rc)
    torch.cuda.synchronize()
    assert torch.isnan(Cfull[M:].float()).all(), "wrote behind the M rows of C"
    if ldc:
        assert torch.isnan(Cfull[:M, N:].float()).all(), "wrote outside the N columns of C"
    return C.cpu()


def check(C, A, sa, B, sb):
    ref = oracle.gemm_tn_mxfp8_fp32(A, sa, B, sb)
    assert oracle.no_nan_left(C)
    err = oracle.rel_frobenius(C, ref)
    assert err <= TOL, err
    return err, ref


@pytest.mark.parametrize("shuffled", [False, True])
@pytest.mark.parametrize("shape", [(256, 256, 128), (256, 256, 1024), (512, 768, 640), (1024, 1024, 2048)])
def test_random_bytes_and_scales(abi, shape, shuffled):
    M, N, K = shape
    A, sa = random_mx(M, K, 1)
    B, sb = random_mx(N, K, 2)
    C = run_mx(abi, A, sa, B, sb, shuffled=shuffled)
    err, _ = check(C, A, sa, B, sb)
    assert err < 5e-3


@pytest.mark.parametrize("shape", [(100, 260, 256), (257, 255 * 4, 384), (1, 4, 128), (300, 516, 128), (640, 128, 1152),
                                   (129, 132, 512)])
def test_ragged_tiles(abi, shape):
    """M and N that do not fill the 256-row tiles or the 128-row scale groups; padded C rows."""
    M, N, K = shape
    A, sa = random_mx(M, K, 3)
    B, sb = random_mx(N, K, 4)
    C = run_mx(abi, A, sa, B, sb, ldc=N + 12)
    check(C, A, sa, B, sb)


@pytest.mark.parametrize("shuffled", [False, True])
@pytest.mark.parametrize("shape", [(768, 768, 8192), (256, 4096, 14336), (6144, 4096, 4096), (300, 1000, 8192)])
def test_k_split_and_tail_split(abi, shape, shuffled):
    """Few tiles: K split 4 ways on 128x128 tiles, 7 ways on 256x128 tiles; 384 tiles of 256x256: the
    last round cut in two.  Same result as without the workspace for the partial results (unsplit),
    up to the summation order."""
    M, N, K = shape
    assert abi.mi355_gemm_mx_workspace_bytes(M, N, K, 1) > 0
    A, sa = random_mx(M, K, 11, 120, 132)
    B, sb = random_mx(N, K, 12, 120, 132)
    C = run_mx(abi, A, sa, B, sb, shuffled=shuffled)
    err, ref = check(C, A, sa, B, sb)
    assert err < 5e-3
    C2 = run_mx(abi, A, sa, B, sb, shuffled=shuffled)
    assert torch.equal(C.view(torch.int16), C2.view(torch.int16))       # deterministic
    if shuffled:
        return
    # natural-layout scales with a workspace that only holds the shuffled scales: runs unsplit
    Ad, Bd, sad, sbd = A.cuda(), B.cuda(), sa.cuda(), sb.cuda()
    only_scales = abi.mi355_mx_shuffled_bytes(M, K) + abi.mi355_mx_shuffled_bytes(N, K)
    ws = torch.empty(only_scales, dtype=torch.uint8, device="cuda")
    C3 = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = abi.mi355_gemm_tn_mxfp8(Ad.data_ptr(), Bd.data_ptr(), C3.data_ptr(), M, N, K, K, K, N, sad.data_ptr(), K // 32,
                                 sbd.data_ptr(), K // 32, 0, ac.BF16, ws.data_ptr(), only_scales,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert oracle.rel_frobenius(C3.cpu(), ref) < 5e-3


@pytest.mark.parametrize("shape,tile", [((2048, 2048, 2048), (128, 128)), ((512, 6144, 4096), (128, 128)),
                                        ((1024, 6144, 4096), (256, 128)), ((1000, 6100, 4224), (256, 128)),
                                        ((2048, 6144, 4096), (256, 256)), ((100, 260, 256), (128, 128))])
def test_every_tile_shape(abi, shape, tile):
    """The block-scaled kernel runs on the tile the planner picks for plain e4m3; a wave with 64 rows
    of an operand reads half a 128-row scale unit."""
    M, N, K = shape
    assert ac.plan(abi, M, N, K, ac.E4M3, ac.BASIC)[1:3] == tile
    A, sa = random_mx(M, K, 21)
    B, sb = random_mx(N, K, 22)
    C = run_mx(abi, A, sa, B, sb, ldc=N + 4)
    err, _ = check(C, A, sa, B, sb)
    assert err < 5e-3


@pytest.mark.parametrize("M,N", [(128, 128), (256, 128), (256, 256)])
def test_each_scale_byte_reaches_its_block_only_on_every_tile(abi, M, N):
    """One doubled scale byte changes exactly its row (or column) by exactly +32, for rows in every
    16-row block of every wave, whichever tile shape the planner gives the problem."""
    K = 256
    big_m, big_n = {(128, 128): (2048, 2048), (256, 128): (1024, 6144), (256, 256): (2048, 6144)}[(M, N)]
    K = {(128, 128): 2048, (256, 128): 4096, (256, 256): 4096}[(M, N)]
    assert ac.plan(abi, big_m, big_n, K, ac.E4M3)[1:3] == (M, N)
    ones_a = torch.ones(big_m, K).to(torch.float8_e4m3fn)
    ones_b = torch.ones(big_n, K).to(torch.float8_e4m3fn)
    base_a = torch.full((big_m, K // 32), 127, dtype=torch.uint8)
    base_b = torch.full((big_n, K // 32), 127, dtype=torch.uint8)
    rows = [0, 17, 63, 64, 127, 128, 191, 255, 256 + 70, big_m - 1]
    sa = base_a.clone()
    for i, r in enumerate(rows):
        sa[r, (5 * i + 3) % (K // 32)] = 128
    C = run_mx(abi, ones_a, sa, ones_b, base_b).float()
    want = torch.full((big_m, big_n), float(K))
    want[rows, :] += 32.0
    assert torch.equal(C, want)
    cols = [0, 15, 16, 63, 64, 100, 127, 128, 255, 300, big_n - 1]
    sb = base_b.clone()
    for i, c in enumerate(cols):
        sb[c, (7 * i + 1) % (K // 32)] = 128
    C = run_mx(abi, ones_a, base_a, ones_b, sb).float()
    want = torch.full((big_m, big_n), float(K))
    want[:, cols] += 32.0
    assert torch.equal(C, want)


def test_each_scale_byte_reaches_its_block_only(abi):
    """All elements 1, all scales 1 except ONE (row, block) of A doubled: exactly row m changes, by
    exactly +32 per column, for every position of the block in the k-step, the scale group and the
    k-step.  Pins the shuffle and which lane's byte the matrix core applies to which 32 elements."""
    M = N = 256
    K = 384
    ones = torch.ones(M, K).to(torch.float8_e4m3fn)
    base = torch.full((M, K // 32), 127, dtype=torch.uint8)
    for m, blk in [(0, 0), (5, 1), (17, 2), (130, 3), (255, 11), (64, 6), (127, 9), (200, 4)]:
        sa = base.clone()
        sa[m, blk] = 128
        C = run_mx(abi, ones, sa, ones, base).float()
        want = torch.full((M, N), float(K))
        want[m, :] += 32.0
        assert torch.equal(C, want), (m, blk)
        C = run_mx(abi, ones, base, ones, sa).float()      # and on the B side: column m
        assert torch.equal(C, want.t()), (m, blk)


def test_block_order_inside_a_k_step(abi):
    """Elements of ONE 32-element block are 1, the rest 0, and that block's scale is 2^3: the result
    is 32*8 only if the kernel pairs the block's elements with the block's own scale."""
    M = N = 256
    K = 256
    base = torch.full((M, K // 32), 127, dtype=torch.uint8)
    ones = torch.ones(N, K).to(torch.float8_e4m3fn)
    for blk in range(K // 32):
        A = torch.zeros(M, K)
        A[:, 32 * blk:32 * blk + 32] = 1.0
        sa = base.clone()
        sa[:, blk] = 130
        C = run_mx(abi, A.to(torch.float8_e4m3fn), sa, ones, base).float()
        assert torch.all(C == 256.0), blk


def test_permutation_is_exact(abi):
    """B = permutation with power-of-two block scales: C[m][n] = A[m][perm[n]] * scales, exactly."""
    M = N = K = 512
    A, sa = random_mx(M, K, 5, 125, 130)
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(6))
    P = torch.zeros(N, K)
    P[torch.arange(N), perm] = 1.0
    sb = torch.from_numpy(np.random.default_rng(7).integers(125, 130, size=(N, K // 32), dtype=np.uint8))
    C = run_mx(abi, A, sa, P.to(torch.float8_e4m3fn), sb)
    want = oracle.gemm_tn_mxfp8_fp32(A, sa, P.to(torch.float8_e4m3fn), sb)
    assert torch.equal(C.view(torch.int16), (want + 0.0).to(torch.bfloat16).view(torch.int16))


def test_scale_shift_is_exact(abi):
    """Adding 1 to every scale byte of A doubles C exactly (bf16 scaling by 2 is exact)."""
    M, N, K = 512, 512, 1024
    A, sa = random_mx(M, K, 8, 120, 130)
    B, sb = random_mx(N, K, 9, 120, 130)
    C1 = run_mx(abi, A, sa, B, sb).float()
    C2 = run_mx(abi, A, sa + 1, B, sb).float()
    assert torch.equal(C2, 2 * C1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_quantizer_is_bit_exact(abi, dtype):
    g = torch.Generator().manual_seed(12)
    x = torch.randn(300, 1024, generator=g) * torch.exp2(torch.randint(-12, 12, (300, 1), generator=g).float())
    x[7, 64:96] = 0.0                       # a block of zeros
    x[8, :32] = 448.0
    x[9, 32:64] = torch.linspace(-500, 500, 32)
    x = x.to(dtype)
    q = torch.empty(x.shape, dtype=torch.uint8, device="cuda")
    sc = torch.empty(x.shape[0], x.shape[1] // 32, dtype=torch.uint8, device="cuda")
    xd = x.cuda()
    code = {torch.bfloat16: ac.BF16, torch.float16: ac.F16, torch.float32: ac.F32}[dtype]
    rc = abi.mi355_quantize_mxfp8(xd.data_ptr(), code, x.shape[0], x.shape[1], xd.stride(0), q.data_ptr(), sc.data_ptr(),
                                  0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    want_q, want_s = oracle.quantize_mxfp8(x)
    assert torch.equal(sc.cpu(), want_s)
    assert torch.equal(q.cpu(), want_q.view(torch.uint8))


def test_quantizer_conversion_on_a_dense_sweep_of_fp32_patterns(abi):
    """The kernels convert fp32 to e4m3 with the hardware instruction; the oracle does it in integer arithmetic.
    Blocks whose first element is 256 have the scale 1, so their other 31 elements come out as the conversion of the
    raw fp32 pattern: 4.2 million patterns spread evenly over [0, 448] (and a few beyond, which must saturate), both
    signs, every binade down to the fp32 subnormals, must give the oracle's code."""
    import numpy as np
    rows, K = 4096, 1024
    i = np.arange(rows * K, dtype=np.uint64)
    bits = ((i * 1021 * 268) % 0x43f00000).astype(np.uint32)          # magnitudes up to 480
    bits |= ((i >> 3) & 1).astype(np.uint32) << 31                     # both signs
    x = torch.from_numpy(bits.view(np.float32).copy()).reshape(rows, K)
    x[:, ::32] = 256.0
    assert float(x.abs().max()) < 512.0 and bool(torch.isfinite(x).all())
    q = torch.empty(x.shape, dtype=torch.uint8, device="cuda")
    sc = torch.empty(rows, K // 32, dtype=torch.uint8, device="cuda")
    xd = x.cuda()
    rc = abi.mi355_quantize_mxfp8(xd.data_ptr(), ac.F32, rows, K, xd.stride(0), q.data_ptr(), sc.data_ptr(), 0,
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((sc.cpu() == 127).all())                               # every block: scale 2^0
    want_q, want_s = oracle.quantize_mxfp8(x)
    assert torch.equal(sc.cpu(), want_s) and torch.equal(q.cpu(), want_q.view(torch.uint8))
    codes = q.cpu()
    assert len(torch.unique(codes)) >= 250                             # the sweep reaches (nearly) every code


@pytest.mark.parametrize("rows", [300, 256, 1])
def test_quantizer_writes_shuffled_scales_directly(abi, rows):
    """The quantiser's shuffled output is byte for byte what mi355_mx_shuffle_scales makes of its
    natural output (padding rows included), and feeds the GEMM without a shuffle launch."""
    import gemm_kernels
    g = torch.Generator().manual_seed(rows)
    x = (torch.randn(rows, 1024, generator=g) * torch.exp2(torch.randint(-8, 8, (rows, 1), generator=g).float())).bfloat16().cuda()
    q1, s_nat = gemm_kernels.quantize_mxfp8(x)
    q2, s_shuf = gemm_kernels.quantize_mxfp8(x, shuffled=True)
    torch.cuda.synchronize()
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(s_shuf, gemm_kernels.shuffle_mx_scales(s_nat))
    w = torch.randn(512, 1024, generator=g).bfloat16().cuda()
    wq, sw = gemm_kernels.quantize_mxfp8(w, shuffled=True)
    C1 = torch.empty(rows, 512, dtype=torch.bfloat16, device="cuda")
    C2 = torch.empty_like(C1)
    gemm_kernels.gemm_tn_mxfp8(q2, wq, s_shuf, sw, C1, scales_shuffled=True)
    wq_n, sw_n = gemm_kernels.quantize_mxfp8(w)
    gemm_kernels.gemm_tn_mxfp8(q1, wq_n, s_nat, sw_n, C2)
    torch.cuda.synchronize()
    assert torch.equal(C1.view(torch.int16), C2.view(torch.int16))


def test_end_to_end_from_bf16(abi):
    """quantise -> block-scaled GEMM against the fp32 product of the ORIGINAL operands: the error is
    the quantisation's (e4m3 keeps 4 significant bits: ~2.7e-2 per element, averaging down over K)."""
    import gemm_kernels
    g = torch.Generator().manual_seed(20)
    # per-row magnitudes spread over 2^+-6: what block scaling is for
    A = (torch.randn(512, 2048, generator=g) * torch.exp2(torch.randint(-6, 6, (512, 1), generator=g).float())).bfloat16()
    B = (torch.randn(768, 2048, generator=g) * torch.exp2(torch.randint(-6, 6, (768, 1), generator=g).float())).bfloat16()
    Aq, sa = gemm_kernels.quantize_mxfp8(A.cuda())
    Bq, sb = gemm_kernels.quantize_mxfp8(B.cuda())
    C = torch.full((512, 768), float("nan"), dtype=torch.bfloat16, device="cuda")
    out = gemm_kernels.gemm_tn_mxfp8(Aq, Bq, sa, sb, C)
    assert out.data_ptr() == C.data_ptr()
    torch.cuda.synchronize()
    check(C.cpu(), Aq.cpu(), sa.cpu(), Bq.cpu(), sb.cpu())
    err = oracle.rel_frobenius(C.cpu(), oracle.gemm_tn_fp32(A, B))
    assert err <= 5e-2, err


def test_python_module_with_preshuffled_scales(abi):
    import gemm_kernels
    A, sa = random_mx(384, 512, 30, 116, 124)     # small scales: the fp16 output must not overflow
    B, sb = random_mx(520, 512, 31, 116, 124)
    Ad, Bd, sad, sbd = A.cuda(), B.cuda(), sa.cuda(), sb.cuda()
    C1 = torch.full((384, 520), float("nan"), dtype=torch.float16, device="cuda")
    C2 = torch.full((384, 520), float("nan"), dtype=torch.float16, device="cuda")
    gemm_kernels.gemm_tn_mxfp8(Ad, Bd, sad.view(torch.float8_e8m0fnu), sbd, C1)
    pa, pb = gemm_kernels.shuffle_mx_scales(sad), gemm_kernels.shuffle_mx_scales(sbd)
    gemm_kernels.gemm_tn_mxfp8(Ad, Bd, pa, pb, C2, scales_shuffled=True)
    torch.cuda.synchronize()
    assert torch.equal(C1.view(torch.int16), C2.view(torch.int16))
    ref = oracle.gemm_tn_mxfp8_fp32(A, sa, B, sb)
    assert torch.isfinite(C1.cpu().float()).all()
    assert oracle.rel_frobenius(C1.cpu(), ref) <= TOL
    with pytest.raises(RuntimeError, match="shuffle_mx_scales"):
        gemm_kernels.gemm_tn_mxfp8(Ad, Bd, sad, sbd, C2, scales_shuffled=True)


def test_full_size_properties(abi):
    """8192^3: the sampled rows against the oracle, and linearity in the scales."""
    from gemm_kernels import workloads
    A, sa, B, sb = workloads.mxfp8_8192(seed=0, device="cuda")
    C = torch.full((8192, 8192), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn_mxfp8(abi, A, B, sa, sb, C) == 0
    torch.cuda.synchronize()
    assert not torch.isnan(C.float()).any()
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 4095, 4096, 8191])
    ref = oracle.gemm_tn_mxfp8_fp32(A[rows].cpu(), sa[rows].cpu(), B.cpu(), sb.cpu())
    assert oracle.rel_frobenius(C[rows].cpu(), ref) <= TOL
    C2 = torch.empty_like(C)
    assert ac.gemm_tn_mxfp8(abi, A, B, sa + 2, sb - 1, C2) == 0
    torch.cuda.synchronize()
    assert torch.equal(C2.float(), 2 * C.float())


def test_rejects_bad_arguments(abi):
    assert abi.mi355_gemm_mx_check(256, 256, 64, 64, 64, 256, ac.BF16) == ac.ERR_SHAPE      # K % 128
    A, sa = random_mx(256, 128, 1)
    C = torch.empty(256, 256, dtype=torch.bfloat16, device="cuda")
    Ad, sad = A.cuda(), sa.cuda()
    s = torch.cuda.current_stream().cuda_stream
    rc = abi.mi355_gemm_tn_mxfp8(Ad.data_ptr(), Ad.data_ptr(), C.data_ptr(), 256, 256, 128, 128, 128, 256, sad.data_ptr(), 4,
                                 sad.data_ptr(), 4, 0, ac.BF16, None, 0, s)
    assert rc == ac.ERR_WORKSPACE
    rc = abi.mi355_gemm_tn_mxfp8(Ad.data_ptr(), Ad.data_ptr(), C.data_ptr(), 256, 256, 128, 128, 128, 256, None, 4,
                                 sad.data_ptr(), 4, 0, ac.BF16, None, 0, s)
    assert rc == ac.ERR_NULL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("std", [1.0, 1e-4, 30.0])
def test_torch_op_quantisers_agree_with_the_kernels_on_the_device(dtype, std):
    """gemm_kernels.quant's torch-op versions state the same contract "on whatever device"; on the GPU
    that needs exact arithmetic (torch.ldexp and division by a Python scalar are not exact there)."""
    import gemm_kernels
    from gemm_kernels.quant import quantize_e4m3_torch, quantize_mxfp8_torch
    x = (torch.randn(257, 512, device="cuda", generator=torch.Generator(device="cuda").manual_seed(5)) * std).to(dtype)

    def same_codes(a, b):   # the sign of a zero aside
        a, b = a.view(torch.uint8), b.view(torch.uint8)
        nz = (b & 0x7f) != 0
        return torch.equal(a[nz], b[nz]) and not (a[~nz] & 0x7f).any()

    q, s = gemm_kernels.quantize_mxfp8(x)
    qt, st = quantize_mxfp8_torch(x)
    assert torch.equal(s, st) and same_codes(q, qt)
    q, s = gemm_kernels.quantize_e4m3(x)
    qt, st = quantize_e4m3_torch(x)
    assert float(s) == float(st) and same_codes(q, qt)


# ---------------------------------------------------------------- a few rows of activations: the streaming kernel

@pytest.mark.parametrize("shuffled", [False, True])
@pytest.mark.parametrize("shape", [(1, 256, 128), (16, 14336, 4096), (17, 2052, 1024), (33, 6144, 4096), (64, 4096, 5760),
                                   (48, 14340, 2048), (64, 28672, 1024), (7, 260, 14336)])
def test_few_rows_stream_the_weights(abi, shape, shuffled):
    """M <= 64 goes to the weight-streaming kernel: every tile height, with and without a K split (and
    splits that do not divide the k-steps), ragged N, both scale layouts; deterministic."""
    M, N, K = shape
    A, sa = random_mx(M, K, 31, 120, 132)
    B, sb = random_mx(N, K, 32, 120, 132)
    C = run_mx(abi, A, sa, B, sb, shuffled=shuffled, ldc=N + 4)
    err, _ = check(C, A, sa, B, sb)
    assert err < 5e-3
    assert torch.equal(run_mx(abi, A, sa, B, sb, shuffled=shuffled, ldc=N + 4).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("M", [1, 16, 40, 64])
def test_each_scale_byte_reaches_its_block_only_with_few_rows(abi, M):
    """One doubled scale byte changes exactly its row (or column) by exactly +32, for rows in every
    16-row block of the tile and columns in every block of every wave, across several k-steps and
    K splits of the streaming kernel."""
    N, K = 4096, 2048
    ones_a = torch.ones(M, K).to(torch.float8_e4m3fn)
    ones_b = torch.ones(N, K).to(torch.float8_e4m3fn)
    base_a = torch.full((M, K // 32), 127, dtype=torch.uint8)
    base_b = torch.full((N, K // 32), 127, dtype=torch.uint8)
    rows = sorted({0, M // 3, M // 2, M - 1, min(M - 1, 15), min(M - 1, 16), min(M - 1, 47)})
    sa = base_a.clone()
    for i, r in enumerate(rows):
        sa[r, (5 * i + 3) % (K // 32)] = 128
    C = run_mx(abi, ones_a, sa, ones_b, base_b).float()
    want = torch.full((M, N), float(K))
    want[rows, :] += 32.0
    assert torch.equal(C, want)
    cols = [0, 15, 16, 31, 32, 47, 48, 63, 64, 100, 127, 128, 191, 255, 300, N - 65, N - 1]
    sb = base_b.clone()
    for i, c in enumerate(cols):
        sb[c, (7 * i + 1) % (K // 32)] = 128
    for shuffled in (False, True):
        C = run_mx(abi, ones_a, base_a, ones_b, sb, shuffled=shuffled).float()
        want = torch.full((M, N), float(K))
        want[:, cols] += 32.0
        assert torch.equal(C, want), shuffled


def test_few_rows_without_room_for_the_k_split_fall_back_to_the_tile_kernel(abi):
    """The streaming kernel needs the workspace of its K split; a call that brings only the room for
    the shuffled scales still succeeds (on the tile kernel, whose split is optional)."""
    M, N, K = 16, 4096, 14336
    A, sa = random_mx(M, K, 41, 120, 132)
    B, sb = random_mx(N, K, 42, 120, 132)
    full = abi.mi355_gemm_mx_workspace_bytes(M, N, K, 0)
    only_scales = abi.mi355_mx_shuffled_bytes(M, K) + abi.mi355_mx_shuffled_bytes(N, K)
    assert full > only_scales
    Ad, Bd, sad, sbd = A.cuda(), B.cuda(), sa.cuda(), sb.cuda()
    ws = torch.empty(only_scales, dtype=torch.uint8, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = abi.mi355_gemm_tn_mxfp8(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, K, N, sad.data_ptr(), K // 32,
                                 sbd.data_ptr(), K // 32, 0, ac.BF16, ws.data_ptr(), only_scales,
                                 torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    err, _ = check(C.cpu(), A, sa, B, sb)
    assert err < 5e-3


@pytest.mark.parametrize("shuffled", [False, True])
@pytest.mark.parametrize("shape", [(256, 256, 1024), (512, 768, 640), (257, 1020, 384), (768, 768, 8192), (4096, 6144, 4096),
                                   (2048, 2048, 2048), (512, 6144, 4096), (33, 6144, 4096)])
def test_fallback_build_of_the_block_scaled_kernel_gives_the_same_bits(abi, shape, shuffled):
    """libmi355gemm_syncscales.so is the library with the block-scaled tile kernel built in its fallback form (scale
    loads that wait for themselves, what the build switches to when the compiler copies the registers of the
    asynchronous ones).  Same arithmetic in the same order: its results must pass the oracle check and equal the default
    build's bit for bit, on every tile shape, with K and tail splits, ragged edges and few rows."""
    fallback = ac.load(ac.LIB_SYNC_SCALES)
    M, N, K = shape
    A, sa = random_mx(M, K, 61)
    B, sb = random_mx(N, K, 62)
    want = run_mx(abi, A, sa, B, sb, shuffled=shuffled)
    got = run_mx(fallback, A, sa, B, sb, shuffled=shuffled)
    if M * N * K <= 768 * 768 * 8192:
        check(got, A, sa, B, sb)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("shuffled", [False, True])
@pytest.mark.parametrize("shape,along_m", [((4096, 6144, 4096), False), ((5120, 4096, 5120), True), ((2048, 10100, 2048), False)])
def test_two_launches_where_the_last_round_would_be_partly_filled(abi, shape, along_m, shuffled):
    """Block-scaled problems are cut like plain ones (mi355_gemm_pieces for e4m3 operands says where): the result must
    pass the oracle on sampled rows and be, bit for bit, what the caller gets by running the two pieces as problems of
    their own, each with its own rows of the operands and of the scales."""
    M, N, K = shape
    rows, cols = ctypes.c_int64(), ctypes.c_int64()
    assert abi.mi355_gemm_pieces(M, N, K, ac.E4M3, ac.AUTO, ctypes.byref(rows), ctypes.byref(cols)) == 2
    first = rows.value if along_m else cols.value
    assert (rows.value != M) == along_m and (cols.value != N) == (not along_m) and first % 256 == 0
    A, sa = random_mx(M, K, 71)
    B, sb = random_mx(N, K, 72)
    C = run_mx(abi, A, sa, B, sb, shuffled=shuffled, ldc=N + 16)
    idx = torch.arange(0, M, max(1, M // 24))
    ref = oracle.gemm_tn_mxfp8_fp32(A[idx], sa[idx], B, sb)
    assert oracle.no_nan_left(C) and oracle.rel_frobenius(C[idx], ref) <= TOL
    if along_m:
        top = run_mx(abi, A[:first], sa[:first], B, sb, shuffled=shuffled)
        bottom = run_mx(abi, A[first:], sa[first:], B, sb, shuffled=shuffled)
        pieces = torch.cat([top, bottom], dim=0)
    else:
        left = run_mx(abi, A, sa, B[:first], sb[:first], shuffled=shuffled)
        right = run_mx(abi, A, sa, B[first:], sb[first:], shuffled=shuffled)
        pieces = torch.cat([left, right], dim=1)
    assert torch.equal(pieces.view(torch.int16), C.contiguous().view(torch.int16))
