"""Parity of the HIP path with the oracle, called through the C ABI (ctypes) and through the
gemm_kernels Python module.  Mirrors the reference's own test (kernels/tests/gemm_test.py:13-41:
NaN-prefilled C, fp32 ground truth, allclose(1e-2, 1e-2)) with seeds added, and extends it to
the dtypes, ragged shapes and full sizes of the benchmark configurations.

Tolerances: relative Frobenius error <= 1e-2 for bf16/fp16 and <= 3e-2 for fp8 (against the fp32
product of the dequantised operands); closed-form and permutation cases are bit-exact."""
import ctypes

import pytest
import torch

from oracle import oracle
from tests import abi_ctypes as ac

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 1e-2, torch.float16: 1e-2, torch.float8_e4m3fn: 3e-2}
TILED = [ac.BASIC, ac.PINGPONG]
DTYPES = {"bf16": torch.bfloat16, "f16": torch.float16, "e4m3": torch.float8_e4m3fn}


def out_dtype_of(dt):
    return torch.bfloat16 if dt == torch.float8_e4m3fn else dt


def run_abi(abi, A, B, variant=ac.AUTO, scale=1.0, out_dtype=None, ldc=None):
    """NaN-prefilled C (gemm_test.py:28), one call through the C ABI, result on the CPU."""
    M, N = A.shape[0], B.shape[0]
    out_dtype = out_dtype or out_dtype_of(A.dtype)
    guard = 8  # rows after the last one: the kernels clip rows in hardware, so watch what lies behind them
    Cfull = torch.full((M + guard, ldc or N), float("nan"), dtype=out_dtype, device="cuda")
    C = Cfull[:M, :N]
    rc = ac.gemm_tn(abi, A.cuda(), B.cuda(), C, scale, variant)
    assert rc == 0, abi.mi355_gemm_strerror(rc)
    torch.cuda.synchronize()
    assert torch.isnan(Cfull[M:].float()).all(), "wrote behind the M rows of C"
    if ldc:
        assert torch.isnan(Cfull[:M, N:].float()).all(), "wrote outside the N columns of C"
    return C.cpu()


def rand(shape, seed, dtype, std=1.0):
    x = torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * std
    return x.to(dtype)


def check(C, A, B, scale=1.0):
    ref = oracle.gemm_tn_fp32(A, B, scale)
    assert oracle.no_nan_left(C)
    err = oracle.rel_frobenius(C, ref)
    assert err <= TOL[A.dtype], err
    return err, ref


# ---------------------------------------------------------------- closed forms, bit-exact

@pytest.mark.parametrize("variant", [ac.AUTO, ac.BASIC, ac.PINGPONG, ac.SIMPLE])
@pytest.mark.parametrize("name", list(DTYPES))
@pytest.mark.parametrize("case", ["identity", "ones", "onehot", "integers"])
def test_golden_closed_forms(abi, golden, case, name, variant):
    dt = DTYPES[name]
    A = torch.from_numpy(golden[f"{case}/{name}/A"]).view(dt)
    B = torch.from_numpy(golden[f"{case}/{name}/B"]).view(dt)
    want = torch.from_numpy(golden[f"{case}/{name}/C"]).view(out_dtype_of(dt))
    got = run_abi(abi, A, B, variant, float(golden[f"{case}/{name}/scale"]))
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("variant", TILED)
@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_permutation_matrix_moves_columns_exactly(abi, dt, variant):
    """B = permutation matrix => C[m][n] = A[m][perm[n]] bit for bit.  Pins every (row, k) ->
    LDS address -> MFMA lane mapping: a swizzle or chunk mix-up moves or zeroes columns."""
    M, N, K = 512, 512, 512
    A = rand((M, K), 1, torch.float32).clamp_(-200, 200).to(dt)
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(2))
    P = torch.zeros(N, K)
    P[torch.arange(N), perm] = 1.0
    got = run_abi(abi, A, P.to(dt), variant)
    # + 0.0: the kernel adds each product to a +0 accumulator, which turns -0 into +0
    want = (A.float()[:, perm] + 0.0).to(out_dtype_of(dt))
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    got_t = run_abi(abi, P.to(dt), A, variant)   # and with the permutation on the A side
    assert torch.equal(got_t.view(torch.int16), want.t().contiguous().view(torch.int16))


@pytest.mark.parametrize("variant", [ac.BASIC, ac.PINGPONG, ac.SKINNY, ac.SIMPLE])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_epilogue_rounds_ties_to_even(abi, dt, variant):
    """Every output is x + h or x + h + tiny with h exactly half an ulp of x in the output type: the
    fp32 accumulator holds the sum exactly, so the result pins the down-conversion (the
    reference's NumericArrayConverter, gemm.cuh:375-377) to round-to-nearest-even, ties included,
    for both signs, odd and even last bits and across exponent boundaries."""
    mant = 7 if dt == torch.bfloat16 else 10
    M = 256
    g = torch.Generator().manual_seed(31)
    # x: random values of the type with exponents -4..8; h = half an ulp of x (a power of two)
    x = (torch.rand(M, generator=g) + 1.0) * torch.exp2(torch.randint(-4, 9, (M,), generator=g).float())
    x = (x * torch.where(torch.rand(M, generator=g) < 0.5, -1.0, 1.0)).to(dt)
    x[0], x[1], x[2], x[3] = 1.0, -1.0, 2.0 - 2.0 ** -mant, -(4.0 - 2.0 ** (1 - mant))     # even, even, all-ones mantissas
    exp = torch.floor(torch.log2(x.float().abs()))
    h = torch.exp2(exp - mant - 1) * torch.sign(x.float())
    K = 16
    A = torch.zeros(M, K)
    A[:, 0], A[:, 1], A[:, 2] = x.float(), h, h * 2.0 ** -8            # the third term breaks the tie upwards
    B = torch.zeros(8, K)
    B[0:4, 0] = 1.0
    B[0:4, 1] = 1.0                                                    # columns 0-3: exact ties
    B[4:8, 0] = 1.0
    B[4:8, 1] = 1.0
    B[4:8, 2] = 1.0                                                    # columns 4-7: just above the tie
    A, B = A.to(dt), B.to(dt)
    assert torch.equal(A.float()[:, 1], h) and torch.equal(A.float()[:, 2], h * 2.0 ** -8)
    exact = A.double() @ B.double().t()                                # three-term sums, exact in fp32 too
    assert torch.equal(exact.float().double(), exact)
    want = exact.float().to(dt)                                        # torch rounds to nearest even
    got = run_abi(abi, A, B, variant)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # the ties went to the even neighbour, the others up (away from x)
    assert torch.equal(want[:, 0].float() == x.float(), (x.view(torch.int16) & 1) == 0)
    assert torch.all(want[:, 4].float().abs() > x.float().abs())


# ---------------------------------------------------------------- oracle parity, seeded random

@pytest.mark.parametrize("variant", [ac.AUTO] + TILED)
def test_config1_fp16_512(abi, variant):
    from gemm_kernels import workloads
    A, B = workloads.fp16_512(seed=10)
    C = run_abi(abi, A, B, variant)
    err, ref = check(C, A, B)
    assert oracle.reference_accepts(C, ref)
    # and against the C restatement, bit for bit except where fp32 summation order flips a tie
    c_ref = oracle.c_gemm_tn(A, B)
    mism = (C.view(torch.int16) != c_ref.view(torch.int16)).float().mean()
    assert mism < 0.02, mism
    assert (C.float() - c_ref.float()).abs().max() <= 2 ** -10 * ref.abs().max()


@pytest.mark.parametrize("variant", [ac.AUTO] + TILED)
@pytest.mark.parametrize("size", [1024, 2048, 4096])
def test_reference_test_shapes_bf16_randn(abi, size, variant):
    """The reference's three shapes and its acceptance check (gemm_test.py:15, :10)."""
    A, B = rand((size, size), size, torch.bfloat16), rand((size, size), size + 1, torch.bfloat16)
    C = run_abi(abi, A, B, variant)
    err, ref = check(C, A, B)
    assert err < 4e-3  # bf16 output rounding alone is ~1.7e-3
    # gemm_test.py:10, :36 as written: allclose(atol=1e-2, rtol=1e-2) against the fp32 product
    assert oracle.reference_accepts(C, ref)


@pytest.mark.parametrize("variant", TILED)
def test_config2_bf16_uniform_4096(abi, variant):
    from gemm_kernels import workloads
    A, B = workloads.bf16_4096(seed=20)
    check(run_abi(abi, A, B, variant), A, B)


@pytest.mark.parametrize("variant", [ac.AUTO] + TILED)
@pytest.mark.parametrize("size", [512, 2048])
def test_fp8_per_tensor_scaled(abi, size, variant):
    from gemm_kernels.quant import quantize_e4m3
    a, b = rand((size, size), 30, torch.float32), rand((size, size), 31, torch.float32)
    (A, sa), (B, sb) = quantize_e4m3(a), quantize_e4m3(b)
    scale = float(sa) * float(sb)
    C = run_abi(abi, A, B, variant, scale)
    err, ref = check(C, A, B, scale)
    assert err < 4e-3
    # for information: error against the unquantised product is dominated by e4m3 rounding
    full = oracle.rel_frobenius(C, a @ b.T)
    assert 1e-2 < full < 8e-2, full


@pytest.mark.parametrize("variant", [ac.AUTO] + TILED + [ac.SIMPLE])
@pytest.mark.parametrize("M,N,K", [(300, 260, 256), (16, 512, 128), (1, 4, 64), (257, 1028, 192), (5000, 4100, 512),
                                   (512, 512, 8), (300, 516, 72), (768, 260, 1000), (520, 256, 328),
                                   (256, 256, 64), (511, 252, 640)])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_ragged_shapes(abi, dt, M, N, K, variant):
    A, B = rand((M, K), M, dt), rand((N, K), N, dt)
    C = run_abi(abi, A, B, variant)
    check(C, A, B)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B)) <= TOL[dt]


def _random_shapes(count, seed):
    """Seeded shapes that the tiled kernels accept: any M, N a multiple of 4, K*elem_bytes a multiple of 16."""
    import random
    rng = random.Random(seed)
    shapes = []
    for _ in range(count):
        M = rng.choice([rng.randint(1, 64), rng.randint(65, 700), rng.randint(701, 2200)])
        N = 4 * rng.choice([rng.randint(1, 16), rng.randint(17, 200), rng.randint(201, 600)])
        K = 16 * rng.choice([rng.randint(1, 8), rng.randint(9, 64), rng.randint(65, 300)])
        shapes.append((M, N, K))
    return shapes


@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_random_shape_sweep(abi, dt):
    """40 seeded random shapes per input type through AUTO and both tiled variants, each against
    the oracle's fp32 product and with NaN guards around C (edge tiles in M and N, ragged and tiny K,
    128- and 256-wide tiles, K splits, the streaming kernel)."""
    for (M, N, K) in _random_shapes(40, 2024):
        if dt == torch.float8_e4m3fn:
            a, b = rand((M, K), M + K, torch.float32), rand((N, K), N + K, torch.float32)
            (A, sa), (B, sb) = oracle.quantize_e4m3(a), oracle.quantize_e4m3(b)
            scale = float(sa) * float(sb)
        else:
            A, B, scale = rand((M, K), M + K, dt), rand((N, K), N + K, dt), 1.0
        ref = oracle.gemm_tn_fp32(A, B, scale)
        for variant in [ac.AUTO] + TILED:
            C = run_abi(abi, A, B, variant, scale=scale, ldc=N + 8 if (M + N) % 3 == 0 else None)
            assert oracle.no_nan_left(C), (M, N, K, variant)
            err = oracle.rel_frobenius(C, ref)
            assert err <= TOL[dt], (M, N, K, variant, err)


def _random_mid_shapes(count, seed):
    """Seeded shapes from a few hundred to a few thousand rows: between them they make the planner
    use every tile shape, with and without a K split, and the tail split."""
    import random
    rng = random.Random(seed)
    shapes = []
    for _ in range(count):
        M = rng.choice([rng.randint(200, 700), rng.randint(701, 2300), rng.randint(2301, 4700)])
        N = 4 * rng.choice([rng.randint(100, 400), rng.randint(401, 1600), rng.randint(1601, 3700)])
        K = 16 * rng.choice([rng.randint(64, 160), rng.randint(161, 400), rng.randint(401, 900)])
        shapes.append((M, N, K))
    return shapes


@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_random_mid_shape_sweep(abi, dt):
    """16 seeded mid-sized shapes per input type through AUTO: every element against the
    one-thread-per-output kernel, 64 sampled rows against the oracle, NaN guards around C."""
    plans = set()
    for (M, N, K) in _random_mid_shapes(16, 4):
        plan = ac.plan(abi, M, N, K, ac.torch_code(dt))
        plans.add((plan[1], plan[2], plan[3] > 1, plan[4] > 0))
        if dt == torch.float8_e4m3fn:
            g = torch.Generator().manual_seed(M + K)
            A = torch.randint(0, 120, (M, K), dtype=torch.uint8, generator=g).view(dt)
            B = torch.randint(0, 120, (N, K), dtype=torch.uint8, generator=g).view(dt)
            scale = 2.0 ** -6
        else:
            A, B, scale = rand((M, K), M + K, dt), rand((N, K), N + K, dt), 1.0
        C = run_abi(abi, A, B, ac.AUTO, scale=scale, ldc=N + 8 if (M + N) % 3 == 0 else None)
        S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
        assert ac.gemm_tn(abi, A.cuda(), B.cuda(), S, scale, ac.SIMPLE) == 0
        torch.cuda.synchronize()
        Sf = S.cpu().float()
        d = (C.float() - Sf).abs()
        bad = d > 2e-2 * Sf.abs() + 2e-2 * (K ** 0.5) * scale * (40.0 if dt == torch.float8_e4m3fn else 1.0)
        assert oracle.no_nan_left(C) and int(bad.sum()) == 0, (M, N, K, plan, int(bad.sum()), float(d.max()))
        rows = torch.randperm(M, generator=torch.Generator().manual_seed(M))[:64]
        assert oracle.rel_frobenius(C[rows], oracle.gemm_tn_fp32(A[rows], B, scale)) <= TOL[dt], (M, N, K, plan)
    if dt != torch.float8_e4m3fn:
        assert len(plans) >= 6, plans   # 256x256 / 256x128 / 128x128, split and unsplit, a tail split


@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (33, 17, 50), (100, 30, 77), (64, 64, 4)])
@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_shapes_only_the_simple_kernel_takes(abi, dt, M, N, K):
    A, B = rand((M, K), 3, torch.float32).clamp_(-100, 100).to(dt), rand((N, K), 4, torch.float32).clamp_(-100, 100).to(dt)
    assert abi.mi355_gemm_select_variant(M, N, K, ac.torch_code(dt)) == ac.SIMPLE
    C = run_abi(abi, A, B, ac.AUTO, 0.25)
    ref = oracle.c_gemm_tn_f32(A, B, 0.25)
    assert oracle.rel_frobenius(C, ref) <= TOL[dt]
    rc = ac.gemm_tn(abi, A.cuda(), B.cuda(), torch.empty(M, N, dtype=out_dtype_of(dt), device="cuda"), 1.0, ac.BASIC)
    assert rc == ac.ERR_SHAPE


@pytest.mark.parametrize("variant", TILED)
@pytest.mark.parametrize("K", [16, 48, 144, 400])
def test_fp8_ragged_last_k_step(abi, K, variant):
    """K*1 byte not a multiple of 128: the missing chunks of the last k-step must read as zeros."""
    A = rand((300, K), 1, torch.float32).clamp_(-100, 100).to(torch.float8_e4m3fn)
    B = rand((264, K), 2, torch.float32).clamp_(-100, 100).to(torch.float8_e4m3fn)
    C = run_abi(abi, A, B, variant, 0.5)
    check(C, A, B, 0.5)


@pytest.mark.parametrize("M,N,K", [(512, 512, 8192), (256, 512, 4096), (300, 260, 4096), (384, 640, 2128), (128, 128, 2048)])
@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_basic_kernel_with_128_tiles_and_k_splits(abi, dt, M, N, K):
    """Shapes with too few 256x256 tiles: the single-group kernel switches to 128x128 tiles and,
    when even those leave most CUs idle, splits K through the fp32 workspace."""
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    C = run_abi(abi, A, B, ac.BASIC, 0.125)
    check(C, A, B, 0.125)
    C2 = run_abi(abi, A, B, ac.BASIC, 0.125)
    assert torch.equal(C.view(torch.int16), C2.view(torch.int16))   # fixed summation order


@pytest.mark.parametrize("dt,M,N,K", [(torch.bfloat16, 3491, 1364, 288), (torch.float16, 2062, 3316, 488), (torch.float8_e4m3fn, 2589, 3220, 976),
                                      (torch.bfloat16, 1024, 3072, 4096), (torch.float16, 1030, 3076, 4104), (torch.float8_e4m3fn, 296, 8768, 5136)])
def test_small_tiles_two_per_cu_and_single_round(abi, dt, M, N, K):
    """128x128 tiles: more of them than CUs (the five-slot ring, two workgroups per CU) and a single round (the nine-slot
    ring without the staggered start), ragged edges and last k-steps; element by element against the generic kernel."""
    plan = ac.plan(abi, M, N, K, ac.torch_code(dt), ac.BASIC)
    assert plan[1:3] == (128, 128), plan
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    scale = 2.0 ** -4
    C = run_abi(abi, A, B, ac.BASIC, scale)
    check(C, A, B, scale)
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, A.cuda(), B.cuda(), S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    d = (C.float() - S.cpu().float()).abs()
    bad = d > 2e-2 * S.cpu().float().abs() + 2e-2 * (K ** 0.5) * scale
    assert int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    assert torch.equal(run_abi(abi, A, B, ac.AUTO, scale).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("dt,M,N,K", [
    (torch.bfloat16, 4096, 6144, 4096),        # 384 tiles of 256: one full round + 128 tiles cut in two
    (torch.bfloat16, 6144, 6144, 6144),        # two full rounds + 64 tiles cut in four
    (torch.bfloat16, 4352, 4352, 4096),        # 289 tiles: one full round + 33 tiles cut in four
    (torch.float8_e4m3fn, 4096, 6144, 8192),
    (torch.float16, 4000, 6100, 4200),         # ragged M, N and last k-step: 384 tiles of 256, 66 k-steps cut in two
    (torch.bfloat16, 5746, 5832, 5648),        # 529 tiles: 17 cut in five, 89 k-steps (the last ragged): items of 17 and 18
    (torch.bfloat16, 4352, 4608, 3008),        # 306 tiles: 50 cut in two, 47 k-steps: 23 + 24
    (torch.float8_e4m3fn, 4352, 4352, 6784),   # 33 tiles cut in three, 53 k-steps: 17 + 18 + 18
])
def test_tail_split(abi, dt, M, N, K):
    """More tiles than workgroup slots with a last round at most half full: the tiles of that round
    are cut along K.  Checked against the oracle, element by element against the one-thread-per-
    output kernel, for determinism, and without a workspace (the split is then skipped)."""
    assert abi.mi355_gemm_workspace_bytes(M, N, K, ac.torch_code(dt), ac.BASIC) > 0
    plan = ac.plan(abi, M, N, K, ac.torch_code(dt), ac.BASIC)
    assert plan[1:4] == (256, 256, 1) and plan[4] > 0 and plan[5] > 1, plan
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    scale = 2.0 ** -4
    C = run_abi(abi, A, B, ac.BASIC, scale)
    check(C, A, B, scale)
    Ad, Bd = A.cuda(), B.cuda()
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    d = (C.float() - S.cpu().float()).abs()
    bad = d > 2e-2 * S.cpu().float().abs() + 2e-2 * (K ** 0.5) * scale
    assert int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    C2 = run_abi(abi, A, B, ac.AUTO, scale)
    if abi.mi355_gemm_pieces(M, N, K, ac.torch_code(dt), ac.AUTO, None, None) == 1:
        assert torch.equal(C.view(torch.int16), C2.view(torch.int16))
    else:       # two launches instead of a tail split: other summation order inside the tiles that were cut
        check(C2, A, B, scale)
    # no workspace: same tiles, no split; differs from C only by the summation order inside the tail tiles
    C3 = torch.full((M, N), float("nan"), dtype=out_dtype_of(dt), device="cuda")
    rc = abi.mi355_gemm_tn(Ad.data_ptr(), Bd.data_ptr(), C3.data_ptr(), M, N, K, K, K, N, ac.torch_code(dt),
                           ac.torch_code(C3.dtype), scale, ac.BASIC, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    check(C3.cpu(), A, B, scale)
    same = (C3.cpu().view(torch.int16) == C.view(torch.int16)).float().mean()
    assert 0.5 < same < 1.0 or dt == torch.float8_e4m3fn, same


@pytest.mark.parametrize("dt,M,N,K,tile,splits", [
    (torch.bfloat16, 512, 6144, 5696, (256, 256), 5),        # 48 tiles, 89 k-steps: 17 + 18 + 18 + 18 + 18
    (torch.bfloat16, 500, 6100, 5648, (256, 256), 5),        # the same with ragged rows, columns and last k-step
    (torch.float8_e4m3fn, 256, 4096, 8320, (128, 128), 4),   # 64 small tiles, 65 k-steps cut in four
    (torch.float16, 200, 2048, 4160, (128, 128), 4),         # 32 small tiles, 65 k-steps: 16 + 16 + 16 + 17
])
def test_k_split_that_does_not_divide_the_k_steps(abi, dt, M, N, K, tile, splits):
    """A K split cuts a tile's k-steps into ranges whose lengths differ by one when they do not divide:
    every k-step must be used exactly once.  Oracle, element-by-element comparison with the
    one-thread-per-output kernel, determinism."""
    plan = ac.plan(abi, M, N, K, ac.torch_code(dt), ac.BASIC)
    assert plan[1:4] == tile + (splits,), plan
    assert (-(-K * (1 if dt == torch.float8_e4m3fn else 2) // 128)) % splits != 0
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    scale = 2.0 ** -4
    C = run_abi(abi, A, B, ac.BASIC, scale)
    check(C, A, B, scale)
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, A.cuda(), B.cuda(), S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    d = (C.float() - S.cpu().float()).abs()
    bad = d > 2e-2 * S.cpu().float().abs() + 2e-2 * (K ** 0.5) * scale
    assert int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    assert torch.equal(run_abi(abi, A, B, ac.BASIC, scale).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("dt,M,N,K", [
    (torch.bfloat16, 512, 14336, 4096),        # 2 x 112 tiles
    (torch.bfloat16, 500, 14000, 1960),        # ragged rows, columns and last k-step
    (torch.bfloat16, 250, 6100, 4104),         # ragged, 48 tiles, 65 k-steps cut in four: 16 + 16 + 16 + 17
    (torch.float16, 256, 4096, 14336),         # 32 tiles, K split 8 ways
    (torch.float8_e4m3fn, 1024, 6144, 4096),
    (torch.float8_e4m3fn, 1000, 6100, 4112),   # ragged; 4112 fp8 bytes = 32 k-steps + 16 bytes
    (torch.float8_e4m3fn, 256, 6144, 14336),   # 48 tiles, 112 k-steps cut in five: 22 + 22 + 23 + 22 + 23
    (torch.bfloat16, 500, 3000, 16400),        # 2 x 24 tiles, 257 k-steps (the last ragged) cut in five
])
def test_rectangular_tile(abi, dt, M, N, K):
    """Problems the planner gives the 256x128 tile: against the oracle and, element by element,
    against the one-thread-per-output kernel; twice for determinism."""
    v, rows, cols, splits, _, _ = ac.plan(abi, M, N, K, ac.torch_code(dt), ac.BASIC)
    assert (v, rows, cols) == (ac.BASIC, 256, 128), (rows, cols, splits)
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    scale = 2.0 ** -4
    C = run_abi(abi, A, B, ac.BASIC, scale, ldc=N + 8)
    check(C, A, B, scale)
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, A.cuda(), B.cuda(), S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    d = (C.float() - S.cpu().float()).abs()
    bad = d > 2e-2 * S.cpu().float().abs() + 2e-2 * (K ** 0.5) * scale
    assert int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    C2 = run_abi(abi, A, B, ac.AUTO, scale)
    assert torch.equal(C.view(torch.int16), C2.view(torch.int16))


def test_rectangular_tile_permutation_is_exact(abi):
    """B = permutation matrix on a problem that runs on 256x128 tiles: pins the narrower B slot's
    copy and fragment addressing bit for bit."""
    M, N, K = 512, 14336, 1024
    assert ac.plan(abi, M, N, K, ac.BF16, ac.BASIC)[1:3] == (256, 128)
    A = rand((M, K), 1, torch.float32).clamp_(-200, 200).to(torch.bfloat16)
    idx = torch.randint(0, K, (N,), generator=torch.Generator().manual_seed(2))
    P = torch.zeros(N, K)
    P[torch.arange(N), idx] = 1.0
    got = run_abi(abi, A, P.to(torch.bfloat16), ac.BASIC)
    want = (A.float()[:, idx] + 0.0).to(torch.bfloat16)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_tiled_kernel_runs_unsplit_without_a_workspace(abi):
    """The K split of the tiled variant is optional: with no workspace (or one that is too small)
    the call succeeds and gives the unsplit result."""
    M, N, K = 256, 6144, 4096
    v, rows, cols, splits, _, _ = ac.plan(abi, M, N, K, ac.BF16, ac.BASIC)
    assert splits > 1
    A, B = rand((M, K), 5, torch.bfloat16), rand((N, K), 6, torch.bfloat16)
    Ad, Bd = A.cuda(), B.cuda()
    s = torch.cuda.current_stream().cuda_stream
    small = torch.empty(1024, dtype=torch.uint8, device="cuda")
    for ws, nbytes in ((None, 0), (small.data_ptr(), 1024)):
        C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = abi.mi355_gemm_tn(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, K, N, ac.BF16, ac.BF16, 1.0,
                               ac.BASIC, ws, nbytes, s)
        assert rc == 0
        torch.cuda.synchronize()
        check(C.cpu(), A, B)


@pytest.mark.parametrize("variant", [ac.AUTO, ac.BASIC, ac.PINGPONG, ac.SKINNY, ac.SIMPLE])
@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_operands_with_padded_rows(abi, dt, variant):
    """lda > K and ldb > K (rows of a wider matrix), which the reference's contiguity check
    (gemm_test.cu:18) excludes: the padding holds NaN and must never be read into a result."""
    M, N, K = (48, 520, 1024) if variant == ac.SKINNY else (300, 520, 1024)
    pad_a, pad_b = 64, 160
    es = 1 if dt == torch.float8_e4m3fn else 2
    g = torch.Generator().manual_seed(9)
    def padded(rows, pad):
        if dt == torch.float8_e4m3fn:
            full = torch.full((rows, K + pad), 0x7f, dtype=torch.uint8)          # e4m3 NaN
            full[:, :K] = torch.randint(0, 120, (rows, K), dtype=torch.uint8, generator=g)
            return full.view(dt).cuda()
        full = torch.full((rows, K + pad), float("nan"), dtype=dt)
        full[:, :K] = torch.randn(rows, K, generator=g).to(dt)
        return full.cuda()
    Af, Bf = padded(M, pad_a), padded(N, pad_b)
    A, B = Af[:, :K], Bf[:, :K]                       # views with row strides K + pad
    assert A.stride(0) == K + pad_a and (A.stride(0) * es) % 16 == 0
    scale = 2.0 ** -6 if dt == torch.float8_e4m3fn else 1.0
    C = torch.full((M, N), float("nan"), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, A, B, C, scale, variant) == 0
    torch.cuda.synchronize()
    check(C.cpu(), A.cpu().contiguous(), B.cpu().contiguous(), scale)


@pytest.mark.parametrize("dt,M,N,K", [
    (torch.bfloat16, 1000, 50257, 768),        # an odd vocabulary size: N % 4 != 0
    (torch.bfloat16, 1001, 1003, 1001),        # everything odd: K*2 % 16 != 0 too
    (torch.float16, 515, 2050, 4100),          # N % 4 == 2, K*2 % 16 == 8
    (torch.float8_e4m3fn, 777, 1001, 1003),    # fp8 rows of 1003 bytes
    (torch.bfloat16, 48, 50257, 768),          # few rows: the repacked problem streams the weights
])
def test_auto_repacks_misaligned_problems(abi, dt, M, N, K):
    """Problems the tiled kernels cannot address run on them all the same when the caller lends a
    workspace: operands copied to aligned zero-padded rows, C computed padded and copied out.  The
    result must be the one the generic kernel gives (same products, fp32 sums), nothing may be
    written outside C, and without the workspace the call still succeeds (generic kernel)."""
    code = ac.torch_code(dt)
    assert abi.mi355_gemm_select_variant(M, N, K, code) == ac.SIMPLE
    need = abi.mi355_gemm_workspace_bytes(M, N, K, code, ac.AUTO)
    assert need > 0
    if dt == torch.float8_e4m3fn:
        g = torch.Generator().manual_seed(M + K)
        A = torch.randint(0, 120, (M, K), dtype=torch.uint8, generator=g).view(dt)
        B = torch.randint(0, 120, (N, K), dtype=torch.uint8, generator=g).view(dt)
        scale = 2.0 ** -6
    else:
        A, B, scale = rand((M, K), M + K, dt), rand((N, K), N + K, dt), 1.0
    C = run_abi(abi, A, B, ac.AUTO, scale, ldc=N + 3)          # odd row stride of C as well, NaN guards around it
    Ad, Bd = A.cuda(), B.cuda()
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    Sf = S.cpu().float()
    d = (C.float() - Sf).abs()
    bad = d > 2e-2 * Sf.abs() + 2e-2 * (K ** 0.5) * scale * (40.0 if dt == torch.float8_e4m3fn else 1.0)
    assert oracle.no_nan_left(C) and int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(1))[:32]
    assert oracle.rel_frobenius(C[rows], oracle.gemm_tn_fp32(A[rows], B, scale)) <= TOL[dt]
    # no workspace: the generic kernel, same contract
    C2 = torch.full((M, N), float("nan"), dtype=out_dtype_of(dt), device="cuda")
    rc = abi.mi355_gemm_tn(Ad.data_ptr(), Bd.data_ptr(), C2.data_ptr(), M, N, K, K, K, N, code, ac.torch_code(C2.dtype),
                           scale, ac.AUTO, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(C2.cpu().view(torch.int16), S.cpu().view(torch.int16))


def test_auto_repacks_misaligned_pointers_and_strides(abi):
    """Aligned shape, but A starts 2 bytes into an allocation and B has a row stride that is not a
    multiple of 16 bytes: repacked when the workspace allows, generic kernel otherwise."""
    M, N, K = 1024, 2048, 1024
    g = torch.Generator().manual_seed(2)
    a_store = torch.randn(M * K + 8, generator=g).bfloat16().cuda()
    A = a_store[1:1 + M * K].view(M, K)                        # 2-byte aligned only
    b_store = torch.randn(N, K + 4, generator=g).bfloat16().cuda()
    B = b_store[:, :K]                                         # row stride 2056 bytes
    assert A.data_ptr() % 16 != 0 and (B.stride(0) * 2) % 16 != 0
    ref = oracle.gemm_tn_fp32(A.cpu().contiguous(), B.cpu().contiguous())
    s = torch.cuda.current_stream().cuda_stream
    big = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    for ws, nbytes in ((big.data_ptr(), big.numel()), (None, 0)):
        C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        rc = abi.mi355_gemm_tn(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0), N, ac.BF16,
                               ac.BF16, 1.0, ac.AUTO, ws, nbytes, s)
        assert rc == 0
        torch.cuda.synchronize()
        assert oracle.no_nan_left(C) and oracle.rel_frobenius(C.cpu(), ref) <= 1e-2
    # an explicit tiled variant still refuses
    rc = abi.mi355_gemm_tn(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0), N, ac.BF16,
                           ac.BF16, 1.0, ac.BASIC, big.data_ptr(), big.numel(), s)
    assert rc in (ac.ERR_SHAPE, ac.ERR_ALIGN)


def test_k_zero_and_empty(abi):
    A, B = torch.zeros(8, 0, dtype=torch.bfloat16), torch.zeros(4, 0, dtype=torch.bfloat16)
    C = run_abi(abi, A, B)
    assert torch.equal(C, torch.zeros(8, 4, dtype=torch.bfloat16))
    E = torch.empty(0, 64, dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, E, torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda"),
                      torch.empty(0, 4, dtype=torch.bfloat16, device="cuda")) == 0


@pytest.mark.parametrize("variant", TILED + [ac.SIMPLE])
def test_strided_c_and_fp16_output_from_bf16(abi, variant):
    A, B = rand((384, 256), 5, torch.bfloat16), rand((320, 256), 6, torch.bfloat16)
    C = run_abi(abi, A, B, variant, ldc=352)
    check(C, A, B)
    C16 = run_abi(abi, A, B, variant, out_dtype=torch.float16)
    assert oracle.rel_frobenius(C16, oracle.gemm_tn_fp32(A, B)) < 1e-3


# ---------------------------------------------------------------- full benchmark sizes

def _sampled_rows_check(C, A, B, scale, tol, rows=48):
    idx = torch.randperm(A.shape[0], generator=torch.Generator().manual_seed(9))[:rows]
    ref = oracle.gemm_tn_fp32(A[idx].contiguous(), B, scale)
    err = oracle.rel_frobenius(C[idx], ref)
    assert err <= tol, err


@pytest.mark.parametrize("variant", TILED)
def test_config3_bf16_8192_full_size(abi, variant):
    """8192^3: every element against the independent one-thread-per-output kernel on the GPU,
    sampled rows against the CPU oracle, and linearity C(A, 2B) == 2 C(A, B) exactly."""
    from gemm_kernels import workloads
    A, B = workloads.bf16_8192(seed=40)
    Ad, Bd = A.cuda(), B.cuda()
    C = torch.full((8192, 8192), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, C, 1.0, variant) == 0
    S = torch.empty_like(C)
    assert ac.gemm_tn(abi, Ad, Bd, S, 1.0, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    assert not torch.isnan(C).any()
    d = (C.float() - S.float())
    assert float(d.norm() / S.float().norm()) < 3e-3
    C2 = torch.empty_like(C)
    assert ac.gemm_tn(abi, Ad, Bd * 2, C2, 1.0, variant) == 0
    assert torch.equal(C2, C * 2)   # scaling by 2 is exact in every step
    _sampled_rows_check(C.cpu(), A, B, 1.0, 1e-2)


@pytest.mark.parametrize("variant", TILED)
def test_config5_fp8_8192_full_size(abi, variant):
    from gemm_kernels import workloads
    A, B, sa, sb = workloads.fp8_8192(seed=50, device="cuda")
    scale = float(sa) * float(sb)
    C = torch.full((8192, 8192), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, A, B, C, scale, variant) == 0
    S = torch.empty_like(C)
    assert ac.gemm_tn(abi, A, B, S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    assert not torch.isnan(C).any()
    assert float((C.float() - S.float()).norm() / S.float().norm()) < 3e-3
    _sampled_rows_check(C.cpu(), A.cpu(), B.cpu(), scale, 3e-2)


@pytest.mark.parametrize("variant", TILED)
@pytest.mark.parametrize("dt,M,N,K", [(torch.bfloat16, 4352, 4352, 1024), (torch.float16, 4352, 4096, 1032),
                                      (torch.float8_e4m3fn, 4352, 4352, 1024), (torch.bfloat16, 4352, 4100, 520)])
def test_uneven_work_per_workgroup_every_element(abi, variant, dt, M, N, K):
    """17 tile rows over 256 workgroups: some store a tile while others are still in their main loop,
    the load pattern under which a store once picked up the registers of the one after it.  Every
    element is compared with the one-thread-per-output kernel, three launches in a row."""
    if dt == torch.float8_e4m3fn:
        A = torch.randint(0, 120, (M, K), dtype=torch.uint8, generator=torch.Generator().manual_seed(70)).view(dt)
        B = torch.randint(0, 120, (N, K), dtype=torch.uint8, generator=torch.Generator().manual_seed(71)).view(dt)
        scale = 2.0 ** -6
    else:
        A, B, scale = rand((M, K), 70, dt), rand((N, K), 71, dt), 1.0
    Ad, Bd = A.cuda(), B.cuda()
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, S, scale, ac.SIMPLE) == 0
    for _ in range(3):
        C = torch.full((M, N), float("nan"), dtype=out_dtype_of(dt), device="cuda")
        assert ac.gemm_tn(abi, Ad, Bd, C, scale, variant) == 0
        torch.cuda.synchronize()
        d = (C.float() - S.float()).abs()
        bad = d > 2e-2 * S.float().abs() + 2e-2 * (K ** 0.5) * scale
        assert not torch.isnan(C).any() and int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))


@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336), (6144, 4096)])
@pytest.mark.parametrize("M", [16, 64, 256])
def test_config4_skinny_projections(abi, M, N, K):
    from gemm_kernels import workloads
    X, W = workloads.skinny(M, N, K, seed=60)
    assert abi.mi355_gemm_select_variant(M, N, K, ac.BF16) == (ac.SKINNY if M <= 64 else ac.BASIC)
    C = run_abi(abi, X, W, ac.AUTO)
    err, ref = check(C, X, W)
    assert err < 4e-3
    # the other kernel families must agree on the same inputs
    for v in (ac.BASIC, ac.SKINNY, ac.PINGPONG):
        assert oracle.rel_frobenius(run_abi(abi, X, W, v), ref) < 4e-3, v


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(256, 14336, 4096), (200, 11012, 2056), (130, 12288, 1032), (256, 10880, 1024)])
def test_one_or_two_tile_rows_on_the_nine_slot_ring(abi, dt, M, N, K):
    """Problems of one or two rows of 128 x 128 tiles that nearly fill the CUs run on the deep ring
    (four k-steps of copies in flight, k-steps walked from a per-workgroup starting point): ragged
    M, N and K, both 16-bit input types, every element against the oracle."""
    code = ac.torch_code(dt)
    v, rows, cols, splits, tail_tiles, tail_splits = ac.plan(abi, M, N, K, code)
    assert (v, rows, cols, splits, tail_tiles) == (ac.BASIC, 128, 128, 1, 0)
    assert 170 <= -(-M // 128) * -(-N // 128) <= 256
    A, B = rand((M, K), M + 3, dt), rand((N, K), N + 4, dt)
    C = run_abi(abi, A, B, ac.AUTO, 0.5)
    err, ref = check(C, A, B, 0.5)
    assert err < 4e-3
    # and bit for bit what the unrotated, five-slot form of the same kernel gives on a problem with
    # the same k range per tile but fewer tiles: only the order of the k-steps differs between the
    # two, so the results agree to fp32 summation order
    small = run_abi(abi, A, B[:2048].contiguous(), ac.BASIC, 0.5)
    assert oracle.rel_frobenius(C[:, :2048], small) < 2e-3


@pytest.mark.parametrize("dt,M,N,K", [(dt, M, N, K) for dt in (torch.bfloat16, torch.float16) for M, N, K in
                                      [(128, 8192, 4096), (100, 4100, 8200), (72, 2052, 8200), (65, 28672, 520), (90, 6144, 4096)]] +
                         [(torch.float8_e4m3fn, 128, 8192, 4096), (torch.float8_e4m3fn, 100, 4100, 8208),
                          (torch.float8_e4m3fn, 72, 2052, 16400), (torch.float8_e4m3fn, 65, 28672, 528)])
def test_one_tile_row_with_k_splits_on_the_nine_slot_ring(abi, dt, M, N, K):
    """65...128 rows: AUTO takes the tile kernel's 128x128 tiles on the nine-slot ring, K split evenly or not
    (129 k-steps in 7 and in 8 parts, the last k-step ragged), ragged M and N, and unsplit."""
    v, rows, cols, splits, _, _ = ac.plan(abi, M, N, K, ac.torch_code(dt))
    assert (v, rows, cols) == (ac.BASIC, 128, 128) and (splits > 1) == (N < 28672), (v, rows, cols, splits)
    if dt == torch.float8_e4m3fn:
        A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
        B = rand((N, K), N + 1, torch.float32, 0.05).to(dt)
    else:
        A, B = rand((M, K), M, dt), rand((N, K), N + 1, dt, 0.05)
    C = run_abi(abi, A, B, ac.AUTO, 0.5)
    check(C, A, B, 0.5)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B, 0.5)) <= TOL[dt]
    assert torch.equal(run_abi(abi, A, B, ac.AUTO, 0.5).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("dt,M,N,K,steps", [(torch.bfloat16, 100, 16384, 64, 1), (torch.bfloat16, 100, 16388, 72, 2),
                                            (torch.float16, 128, 20000, 200, 4), (torch.float8_e4m3fn, 90, 12288, 512, 4),
                                            (torch.bfloat16, 128, 12288, 320, 5), (torch.float8_e4m3fn, 70, 32768, 1008, 8)])
def test_one_tile_row_with_fewer_k_steps_than_the_nine_slot_ring_keeps_in_flight(abi, dt, M, N, K, steps):
    """One row of 128x128 tiles, unsplit, with 1...8 k-steps: fewer than the nine-slot ring's five
    opening operand-steps (or than its nine slots), so its copies are clamped to the last k-step and
    the rotated starting points wrap inside a handful of steps; ragged K, M and N among them."""
    es = 1 if dt == torch.float8_e4m3fn else 2
    assert -(-K * es // 128) == steps
    v, rows, cols, splits, _, _ = ac.plan(abi, M, N, K, ac.torch_code(dt))
    assert (v, rows, cols, splits) == (ac.BASIC, 128, 128, 1), (v, rows, cols, splits)
    if dt == torch.float8_e4m3fn:
        A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
        B = rand((N, K), N + 1, torch.float32, 0.05).to(dt)
    else:
        A, B = rand((M, K), M, dt), rand((N, K), N + 1, dt, 0.05)
    C = run_abi(abi, A, B, ac.AUTO, 0.5)
    check(C, A, B, 0.5)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B, 0.5)) <= TOL[dt]
    assert torch.equal(run_abi(abi, A, B, ac.AUTO, 0.5).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("dt,M,N,K", [(torch.bfloat16, 8200, 128, 4096), (torch.float16, 12289, 100, 2056), (torch.float8_e4m3fn, 8192, 96, 8208),
                                      (torch.bfloat16, 32768, 64, 1024)])
def test_one_tile_column_on_the_nine_slot_ring(abi, dt, M, N, K):
    """Many rows against at most 128 columns: one column of 128x128 tiles on the nine-slot ring, with and without a K split."""
    v, rows, cols, splits, _, _ = ac.plan(abi, M, N, K, ac.torch_code(dt))
    assert (v, rows, cols) == (ac.BASIC, 128, 128), (v, rows, cols, splits)
    if dt == torch.float8_e4m3fn:
        A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
        B = rand((N, K), N + 1, torch.float32, 0.05).to(dt)
    else:
        A, B = rand((M, K), M, dt), rand((N, K), N + 1, dt, 0.05)
    C = run_abi(abi, A, B, ac.AUTO, 0.5)
    check(C, A, B, 0.5)
    assert torch.equal(run_abi(abi, A, B, ac.AUTO, 0.5).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (16, 512, 128), (16, 128, 8), (48, 260, 1096), (256, 64, 4104), (10, 260, 256), (17, 64, 1024), (33, 512, 4096),
                                   (64, 1024, 2048), (100, 640, 1024), (129, 72, 512), (256, 768, 2048)])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float8_e4m3fn])
def test_skinny_kernel_every_tile_height_and_split(abi, dt, M, N, K):
    """Each TM configuration (16/32/64/128/256), with and without K splits, ragged M and N."""
    if dt == torch.float8_e4m3fn:
        K = max(16, K // 16 * 16)   # fp8 rows are moved in 16-byte chunks
        A = rand((M, K), M + 1, torch.float32).clamp_(-100, 100).to(dt)
        B = rand((N, K), N + 2, torch.float32).clamp_(-100, 100).to(dt)
    else:
        A, B = rand((M, K), M + 1, dt), rand((N, K), N + 2, dt)
    C = run_abi(abi, A, B, ac.SKINNY, 0.25)
    check(C, A, B, 0.25)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B, 0.25)) <= TOL[dt]


@pytest.mark.parametrize("dt,M,N,K", [(torch.bfloat16, 64, 8192, 4096), (torch.float16, 33, 8200, 4104), (torch.bfloat16, 50, 4100, 8200),
                                      (torch.float16, 64, 20484, 520), (torch.float8_e4m3fn, 48, 8192, 8192),
                                      (torch.float8_e4m3fn, 64, 4100, 16400), (torch.bfloat16, 40, 32768, 256),
                                      (torch.float16, 9, 20484, 264), (torch.float8_e4m3fn, 32, 24576, 1040),
                                      (torch.bfloat16, 40, 16640, 8448), (torch.bfloat16, 64, 3072, 8192),
                                      (torch.float16, 20, 17412, 1032)])
def test_skinny_kernel_on_128_wide_tiles(abi, dt, M, N, K):
    """33...64 rows against enough columns and k-steps, fewer rows against 16512...26496 columns: 64 x 128
    tiles, split and unsplit, ragged M, N and K; k-steps started evenly spread (few rows, or many tile columns
    with few k-steps) and clustered by XCD (more than 32 rows: 33 tile columns split along K, 130 unsplit)."""
    plan = ac.plan(abi, M, N, K, ac.torch_code(dt), ac.SKINNY)
    assert plan[:3] == (ac.SKINNY, 64, 128), plan
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    C = run_abi(abi, A, B, ac.SKINNY, 0.25)
    check(C, A, B, 0.25)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B, 0.25)) <= TOL[dt]
    assert torch.equal(run_abi(abi, A, B, ac.SKINNY, 0.25).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("dt,M,N,K", [(torch.bfloat16, 16, 4096, 5696), (torch.bfloat16, 48, 4100, 11016),
                                      (torch.float8_e4m3fn, 64, 2048, 13584), (torch.float16, 200, 1024, 5768)])
def test_skinny_k_split_that_does_not_divide_the_k_steps(abi, dt, M, N, K):
    """89, 173 (the last ragged), 107 and 91 k-steps with split counts that do not divide them."""
    es = 1 if dt == torch.float8_e4m3fn else 2
    splits = ac.plan(abi, M, N, K, ac.torch_code(dt), ac.SKINNY)[3]
    assert splits > 1 and (-(-K * es // 128)) % splits != 0, splits
    A = rand((M, K), M, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N, torch.float32).clamp_(-50, 50).to(dt)
    C = run_abi(abi, A, B, ac.SKINNY, 0.25)
    check(C, A, B, 0.25)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B, 0.25)) <= TOL[dt]
    assert torch.equal(run_abi(abi, A, B, ac.SKINNY, 0.25).view(torch.int16), C.view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(16, 4096, 14336), (90, 2048, 4096)])
def test_auto_without_a_workspace_takes_the_tile_kernel_for_few_rows(abi, M, N, K):
    """The streaming kernel's K split needs a workspace; MI355_VARIANT_AUTO called without one still
    succeeds (on the tile kernel, unsplit), an explicit MI355_VARIANT_SKINNY does not."""
    A, B = rand((M, K), 7, torch.bfloat16), rand((N, K), 8, torch.bfloat16)
    assert abi.mi355_gemm_select_variant(M, N, K, ac.BF16) == ac.SKINNY
    assert abi.mi355_gemm_workspace_bytes(M, N, K, ac.BF16, ac.AUTO) > 0
    Ad, Bd = A.cuda(), B.cuda()
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    call = lambda v: abi.mi355_gemm_tn(Ad.data_ptr(), Bd.data_ptr(), C.data_ptr(), M, N, K, K, K, N, ac.BF16, ac.BF16, 1.0, v,
                                       None, 0, s)
    assert call(ac.SKINNY) == ac.ERR_WORKSPACE
    assert call(ac.AUTO) == 0
    torch.cuda.synchronize()
    check(C.cpu(), A, B)


def test_skinny_split_k_is_deterministic_and_needs_its_workspace(abi):
    M, N, K = 16, 256, 4096
    A, B = rand((M, K), 1, torch.bfloat16).cuda(), rand((N, K), 2, torch.bfloat16).cuda()
    need = abi.mi355_gemm_workspace_bytes(M, N, K, ac.BF16, ac.SKINNY)
    assert need > 0 and need % (M * N * 4) == 0
    C1 = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    C2 = torch.empty_like(C1)
    assert ac.gemm_tn(abi, A, B, C1, 1.0, ac.SKINNY) == 0
    assert ac.gemm_tn(abi, A, B, C2, 1.0, ac.SKINNY) == 0
    torch.cuda.synchronize()
    assert torch.equal(C1, C2)
    s = torch.cuda.current_stream().cuda_stream
    rc = abi.mi355_gemm_tn(A.data_ptr(), B.data_ptr(), C1.data_ptr(), M, N, K, K, K, N, ac.BF16, ac.BF16, 1.0,
                           ac.SKINNY, None, 0, s)
    assert rc == ac.ERR_WORKSPACE
    small = torch.empty(need - 16, dtype=torch.uint8, device="cuda")
    rc = abi.mi355_gemm_tn(A.data_ptr(), B.data_ptr(), C1.data_ptr(), M, N, K, K, K, N, ac.BF16, ac.BF16, 1.0,
                           ac.SKINNY, small.data_ptr(), need - 16, s)
    assert rc == ac.ERR_WORKSPACE
    big = torch.empty(300, 64, dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, big, torch.empty(64, 64, dtype=torch.bfloat16, device="cuda"),
                      torch.empty(300, 64, dtype=torch.bfloat16, device="cuda"), 1.0, ac.SKINNY) == ac.ERR_SHAPE


@pytest.mark.parametrize("variant", [ac.AUTO, ac.PINGPONG, ac.SIMPLE])
def test_c_larger_than_4_gib(abi, variant):
    """65836 x 32772 bf16 outputs (4.3 GB): row offsets into C pass 2^31 elements and 2^32 bytes.
    Sampled rows against the oracle; the reference narrows sizes and strides to int
    (gemm_test.cu:29-31, :44-46) and could not run this."""
    M, N, K = 65536 + 300, 32768 + 4, 64
    g = torch.Generator(device="cuda").manual_seed(3)
    A = torch.randn(M, K, generator=g, device="cuda").bfloat16()
    B = torch.randn(N, K, generator=g, device="cuda").bfloat16()
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert C.numel() * 2 > 2 ** 32
    assert ac.gemm_tn(abi, A, B, C, 1.0, variant) == 0
    torch.cuda.synchronize()
    rows = torch.tensor([0, 1, 255, 256, 32767, 32768, 65535, 65536, 65537, 65791, 65792, M - 2, M - 1])
    got = C[rows.cuda()].cpu()
    assert oracle.no_nan_left(got)
    assert oracle.rel_frobenius(got, oracle.gemm_tn_fp32(A[rows.cuda()].cpu(), B.cpu())) <= 1e-2
    # every element was written: no NaN left anywhere (checked on the device, in slabs)
    for r0 in range(0, M, 8192):
        assert not torch.isnan(C[r0:r0 + 8192]).any(), r0


@pytest.mark.parametrize("variant", [ac.AUTO, ac.PINGPONG])
def test_a_larger_than_4_gib(abi, variant):
    """A is 70000 x 32768 bf16 (4.6 GB): the byte offset of the last row panels passes 2^32."""
    M, N, K = 70000, 256, 32768
    g = torch.Generator(device="cuda").manual_seed(4)
    A = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, M, 10000):
        A[r0:r0 + 10000] = torch.randn(min(10000, M - r0), K, generator=g, device="cuda").bfloat16()
    B = torch.randn(N, K, generator=g, device="cuda").bfloat16()
    assert A.numel() * 2 > 2 ** 32
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, A, B, C, 1.0, variant) == 0
    torch.cuda.synchronize()
    assert not torch.isnan(C).any()
    rows = torch.tensor([0, 255, 256, 65535, 65536, 65537, 69887, 69888, M - 1])
    ref = oracle.gemm_tn_fp32(A[rows.cuda()].cpu(), B.cpu())
    assert oracle.rel_frobenius(C[rows.cuda()].cpu(), ref) <= 1e-2
    # and with the big matrix on the B side (columns of C)
    Ct = torch.full((N, M), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, B, A, Ct, 1.0, variant) == 0
    torch.cuda.synchronize()
    assert not torch.isnan(Ct).any()
    assert oracle.rel_frobenius(Ct[:, rows.cuda()].cpu(), ref.t()) <= 1e-2
    if variant == ac.AUTO:   # 16 rows against the 4.6 GB of weights: the streaming kernel
        assert abi.mi355_gemm_select_variant(16, M, K, ac.BF16) == ac.SKINNY
        Cs = torch.full((16, M), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert ac.gemm_tn(abi, B[:16].contiguous(), A, Cs, 1.0, ac.AUTO) == 0
        torch.cuda.synchronize()
        assert not torch.isnan(Cs).any()
        assert oracle.rel_frobenius(Cs[:, rows.cuda()].cpu(), ref[:, :16].t()) <= 1e-2


# ---------------------------------------------------------------- Python module

def test_python_module_is_the_reference_call(abi):
    """gemm_test.py:23-36 verbatim in spirit: randn bf16 on 'cuda', NaN prefill, call, compare."""
    from gemm_kernels import gemm_tn_test
    torch.manual_seed(0)
    A = torch.randn((1024, 1024), device="cuda", dtype=torch.bfloat16)
    B = torch.randn((1024, 1024), device="cuda", dtype=torch.bfloat16)
    C = torch.empty((1024, 1024), device="cuda", dtype=torch.bfloat16)
    C.fill_(float("nan"))
    out = gemm_tn_test(A, B, C)
    assert out.data_ptr() == C.data_ptr()
    err, ref = check(C, A, B)
    assert oracle.reference_accepts(C, ref)   # gemm_test.py:10 against the fp32 product of :36


def test_python_module_repacks_odd_shapes():
    """gemm_tn_test on an odd vocabulary-sized problem: the binding lends the workspace, so the tiled
    kernels run (the result matches the oracle; the generic kernel would take ~70 ms here)."""
    import time
    import gemm_kernels
    M, N, K = 1000, 50257, 768
    A, B = rand((M, K), 1, torch.bfloat16).cuda(), rand((N, K), 2, torch.bfloat16).cuda()
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    gemm_kernels.gemm_tn_test(A, B, C)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        gemm_kernels.gemm_tn_test(A, B, C)
    torch.cuda.synchronize()
    per_call = (time.perf_counter() - t0) / 5
    assert per_call < 10e-3, per_call            # ~0.25 ms repacked; ~68 ms on the generic kernel
    rows = torch.arange(0, M, 37)
    assert oracle.no_nan_left(C)
    assert oracle.rel_frobenius(C[rows.cuda()].cpu(), oracle.gemm_tn_fp32(A[rows.cuda()].cpu(), B.cpu())) <= 1e-2


def test_python_module_variants_streams_and_fp8():
    import gemm_kernels
    from gemm_kernels.quant import quantize_e4m3
    A, B = rand((192, 1024), 70, torch.bfloat16).cuda(), rand((768, 1024), 71, torch.bfloat16).cuda()
    want = oracle.gemm_tn_fp32(A, B)
    side = torch.cuda.Stream()
    for v in ["auto", "basic", "pingpong", "skinny", "simple"]:
        C = torch.full((192, 768), float("nan"), dtype=torch.bfloat16, device="cuda")
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            gemm_kernels.gemm_tn(A, B, C, variant=v)
        side.synchronize()
        assert oracle.rel_frobenius(C, want) < 1e-2, v
    a, b = rand((256, 512), 72, torch.float32).cuda(), rand((256, 512), 73, torch.float32).cuda()
    (Aq, sa), (Bq, sb) = quantize_e4m3(a), quantize_e4m3(b)
    C = torch.empty(256, 256, dtype=torch.bfloat16, device="cuda")
    gemm_kernels.gemm_tn_fp8(Aq, Bq, sa, sb, C)
    assert oracle.rel_frobenius(C, oracle.gemm_tn_fp32(Aq, Bq, float(sa) * float(sb))) < 3e-2


# ---------------------------------------------------------------- device quantiser

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,std", [((257, 129), 1.0), ((8192, 64), 0.02), ((3, 5), 37.0), ((1, 1), 1.0), ((1000, 1000), 1.0)])
def test_device_quantiser_matches_oracle_bit_for_bit(dtype, shape, std):
    import gemm_kernels
    x = (torch.randn(shape, generator=torch.Generator().manual_seed(shape[0])) * std).to(dtype)
    q, s = gemm_kernels.quantize_e4m3(x.cuda())
    q_o, s_o = oracle.quantize_e4m3(x.float())
    assert q.dtype == torch.float8_e4m3fn and q.shape == x.shape and s.dim() == 0
    assert float(s) == s_o
    assert torch.equal(q.cpu().view(torch.uint8), q_o.view(torch.uint8))


def test_device_quantiser_every_code_and_every_tie():
    """amax = 448 makes scale exactly 1, so the kernel's rounding is compared value by value with
    torch's e4m3fn cast: every representable value, every midpoint between neighbours (ties to
    even), subnormals and zeros."""
    import gemm_kernels
    v = torch.arange(0, 0x7f, dtype=torch.uint8).view(torch.float8_e4m3fn).float().double()
    mid = (v[:-1] + v[1:]) / 2
    pts = torch.cat([v, mid, mid * (1 + 2 ** -20), mid * (1 - 2 ** -20), torch.tensor([448.0, 0.0, 2.0 ** -10, 2.0 ** -11])])
    x = torch.cat([pts, -pts]).float()
    q, s = gemm_kernels.quantize_e4m3(x.cuda())
    assert float(s) == 1.0
    want = x.to(torch.float8_e4m3fn)
    assert torch.equal(q.cpu().view(torch.uint8) & 0x7f, want.view(torch.uint8) & 0x7f)   # -0 vs +0 sign aside
    nz = want.float() != 0
    assert torch.equal(q.cpu().view(torch.uint8)[nz], want.view(torch.uint8)[nz])
    z, sz = gemm_kernels.quantize_e4m3(torch.zeros(40, device="cuda"))
    assert float(sz) == 1.0 and not z.float().any()


def test_fp8_gemm_with_device_resident_scales(abi):
    """quantise -> GEMM without a host round trip: the scales stay on the device."""
    import gemm_kernels
    a = rand((512, 1024), 80, torch.float32).cuda()
    b = rand((768, 1024), 81, torch.float32).cuda()
    (Aq, sa), (Bq, sb) = gemm_kernels.quantize_e4m3(a), gemm_kernels.quantize_e4m3(b)
    assert sa.is_cuda and sb.is_cuda
    C = torch.full((512, 768), float("nan"), dtype=torch.bfloat16, device="cuda")
    gemm_kernels.gemm_tn_fp8(Aq, Bq, sa, sb, C)
    ref = oracle.gemm_tn_fp32(Aq, Bq, float(sa) * float(sb))
    assert oracle.no_nan_left(C) and oracle.rel_frobenius(C, ref) < 4e-3
    C2 = torch.empty_like(C)
    gemm_kernels.gemm_tn_fp8(Aq, Bq, float(sa), sb.cpu(), C2)      # host-side scales give the same bits
    assert torch.equal(C, C2)
    # the same through the C ABI, for every kernel family that takes fp8
    for variant in (ac.BASIC, ac.PINGPONG, ac.SIMPLE):
        C3 = torch.empty_like(C)
        ws_bytes = abi.mi355_gemm_workspace_bytes(512, 768, 1024, ac.E4M3, variant)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
        rc = abi.mi355_gemm_tn_scaled(Aq.data_ptr(), Bq.data_ptr(), C3.data_ptr(), 512, 768, 1024, 1024, 1024, 768,
                                      ac.E4M3, ac.BF16, 1.0, sa.data_ptr(), sb.data_ptr(), variant,
                                      ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert oracle.rel_frobenius(C3, ref) < 4e-3, variant


@pytest.mark.parametrize("dt,M,N,K,along_m", [
    (torch.bfloat16, 4096, 14336, 4096, False),       # 3.5 rounds of 256 x 256 tiles: 12288 + 2048 columns
    (torch.bfloat16, 14336, 4096, 4096, True),        # the same cut along M
    (torch.float8_e4m3fn, 4096, 6144, 4096, False),   # 1.5 rounds: 4096 + 2048 columns instead of a tail split
    (torch.float16, 4000, 14300, 2056, False),        # ragged rows, columns and last k-step
    (torch.bfloat16, 14300, 4000, 2056, True),
    (torch.float8_e4m3fn, 2048, 10240, 2048, False),
])
def test_two_launches_where_the_last_round_would_be_partly_filled(abi, dt, M, N, K, along_m):
    """MI355_VARIANT_AUTO cuts such a problem into a first piece of whole rounds and a rest (mi355_gemm_pieces says
    where): the result must pass the oracle on sampled rows, agree element by element with the one-thread-per-output
    kernel, leave everything outside C alone (padded rows of C, guard rows), come out the same twice, and be what the
    two pieces give when the caller runs them as problems of their own."""
    code = ac.torch_code(dt)
    rows, cols = ctypes.c_int64(), ctypes.c_int64()
    assert abi.mi355_gemm_pieces(M, N, K, code, ac.AUTO, ctypes.byref(rows), ctypes.byref(cols)) == 2
    assert (rows.value != M) == along_m and (cols.value != N) == (not along_m)
    first = rows.value if along_m else cols.value
    assert first % 256 == 0 and 0 < first < (M if along_m else N)
    A = rand((M, K), M + 1, torch.float32).clamp_(-50, 50).to(dt)
    B = rand((N, K), N + 2, torch.float32).clamp_(-50, 50).to(dt)
    scale = 2.0 ** -3
    C = run_abi(abi, A, B, ac.AUTO, scale, ldc=N + 24)
    _sampled_rows_check(C, A, B, scale, TOL[dt])
    Ad, Bd = A.cuda(), B.cuda()
    S = torch.empty((M, N), dtype=out_dtype_of(dt), device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, S, scale, ac.SIMPLE) == 0
    torch.cuda.synchronize()
    d = (C.float() - S.cpu().float()).abs()
    bad = d > 2e-2 * S.cpu().float().abs() + 2e-2 * (K ** 0.5) * scale * 50
    assert int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    assert torch.equal(run_abi(abi, A, B, ac.AUTO, scale).view(torch.int16), C.contiguous().view(torch.int16))
    # the caller's own two calls on the pieces (explicit variants never cut)
    P = torch.full((M, N), float("nan"), dtype=out_dtype_of(dt), device="cuda")
    if along_m:
        assert ac.gemm_tn(abi, Ad[:first], Bd, P[:first], scale, ac.BASIC) == 0
        assert ac.gemm_tn(abi, Ad[first:], Bd, P[first:], scale, ac.BASIC) == 0
    else:
        assert ac.gemm_tn(abi, Ad, Bd[:first], P[:, :first], scale, ac.BASIC) == 0
        assert ac.gemm_tn(abi, Ad, Bd[first:], P[:, first:], scale, ac.BASIC) == 0
    torch.cuda.synchronize()
    assert torch.equal(P.cpu().view(torch.int16), C.contiguous().view(torch.int16))
