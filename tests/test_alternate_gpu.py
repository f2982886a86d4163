"""The `alternate` variant (two workgroups per CU, each on its own stream of 256x128 tiles, one
storing while the other computes; counterpart of the reference's ping-pong kernel,
kernels/gemm_kernels/sm90a/gemm_pingpong.cuh:121-349) against the oracle, through the C ABI.
16-bit inputs only.  Tolerances as for the other variants: closed forms and permutations bit for
bit, seeded random cases within a relative Frobenius error of 1e-2, the reference's own
acceptance check (gemm_test.py:10) on its own three shapes."""
import pytest
import torch

from oracle import oracle
from tests import abi_ctypes as ac
from tests.test_gemm_gpu import check, rand, run_abi

pytestmark = pytest.mark.gpu

DTYPES = {"bf16": torch.bfloat16, "f16": torch.float16}


@pytest.mark.parametrize("name", list(DTYPES))
@pytest.mark.parametrize("case", ["identity", "ones", "onehot", "integers"])
def test_golden_closed_forms(abi, golden, case, name):
    dt = DTYPES[name]
    A = torch.from_numpy(golden[f"{case}/{name}/A"]).view(dt)
    B = torch.from_numpy(golden[f"{case}/{name}/B"]).view(dt)
    want = torch.from_numpy(golden[f"{case}/{name}/C"]).view(dt)
    got = run_abi(abi, A, B, ac.ALTERNATE, float(golden[f"{case}/{name}/scale"]))
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("dt", list(DTYPES.values()))
def test_permutation_matrix_moves_columns_exactly(abi, dt):
    """B = permutation matrix => C[m][n] = A[m][perm[n]] bit for bit: pins every (row, k) -> LDS
    address -> MFMA lane mapping of this kernel's own slots, and the same with the roles exchanged."""
    M, N, K = 512, 512, 512
    A = rand((M, K), 1, torch.float32).clamp_(-200, 200).to(dt)
    perm = torch.randperm(K, generator=torch.Generator().manual_seed(2))
    P = torch.zeros(N, K)
    P[torch.arange(N), perm] = 1.0
    got = run_abi(abi, A, P.to(dt), ac.ALTERNATE)
    want = (A.float()[:, perm] + 0.0).to(dt)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    got_t = run_abi(abi, P.to(dt), A, ac.ALTERNATE)
    assert torch.equal(got_t.view(torch.int16), want.t().contiguous().view(torch.int16))


@pytest.mark.parametrize("size", [1024, 2048, 4096])
def test_reference_test_shapes_bf16_randn(abi, size):
    """The reference's three shapes and its acceptance check (gemm_test.py:15, :10, :36)."""
    A, B = rand((size, size), size, torch.bfloat16), rand((size, size), size + 1, torch.bfloat16)
    C = run_abi(abi, A, B, ac.ALTERNATE)
    err, ref = check(C, A, B)
    assert err < 4e-3
    assert oracle.reference_accepts(C, ref)


@pytest.mark.parametrize("dt", list(DTYPES.values()))
@pytest.mark.parametrize("M,N,K", [(256, 128, 64), (256, 128, 128), (256, 128, 192), (1, 4, 8), (300, 260, 256), (257, 1028, 72),
                                   (5000, 4100, 512), (512, 512, 8), (768, 260, 1000), (520, 132, 328), (17 * 256, 33 * 128, 640)])
def test_ragged_shapes_against_the_oracle(abi, dt, M, N, K):
    """One to many k-steps (odd and even counts: the two slots of A alternate), ragged last k-step,
    rows and columns that do not fill a tile, more tiles than resident workgroups and fewer."""
    A, B = rand((M, K), M + 1, dt), rand((N, K), N + 2, dt)
    C = run_abi(abi, A, B, ac.ALTERNATE, 0.5)
    check(C, A, B, 0.5)
    assert oracle.rel_frobenius(C, oracle.c_gemm_tn_f32(A, B, 0.5)) <= 1e-2
    assert torch.equal(run_abi(abi, A, B, ac.ALTERNATE, 0.5).view(torch.int16), C.view(torch.int16))


def test_row_strides_and_output_type(abi):
    """lda, ldb, ldc beyond the row lengths, fp16 output from bf16 inputs; nothing outside C is written."""
    M, N, K = 700, 392, 456
    A = rand((M, K + 24), 5, torch.bfloat16)[:, :K]
    B = rand((N, K + 8), 6, torch.bfloat16)[:, :K]
    C = run_abi(abi, A, B, ac.ALTERNATE, 1.0, out_dtype=torch.float16, ldc=N + 12)
    check(C, A.contiguous(), B.contiguous())


def test_auto_takes_it_for_tiles_that_are_all_epilogue(abi):
    """bf16 4096 x 8192 x 256: four k-steps and 1024 tiles, the regime AUTO hands to this variant; every
    workgroup walks two tiles and the second workgroup of each pair starts late.  Every element
    against the one-thread-per-output kernel, and sampled rows against the CPU oracle."""
    M, N, K = 4096, 8192, 256
    assert abi.mi355_gemm_select_variant(M, N, K, ac.BF16) == ac.ALTERNATE
    A, B = rand((M, K), 41, torch.bfloat16), rand((N, K), 42, torch.bfloat16)
    Ad, Bd = A.cuda(), B.cuda()
    S = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, S, 1.0, ac.SIMPLE) == 0
    for _ in range(3):
        C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert ac.gemm_tn(abi, Ad, Bd, C, 1.0, ac.AUTO) == 0
        torch.cuda.synchronize()
        d = (C.float() - S.float()).abs()
        bad = d > 2e-2 * S.float().abs() + 2e-2 * (K ** 0.5)
        assert not torch.isnan(C).any() and int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))
    rows = torch.arange(0, M, 97)
    assert oracle.rel_frobenius(C[rows.cuda()].cpu(), oracle.gemm_tn_fp32(A[rows], B)) <= 1e-2


@pytest.mark.parametrize("dt,M,N,K", [(torch.bfloat16, 4352, 4352, 1024), (torch.float16, 4352, 4100, 1032)])
def test_uneven_work_per_workgroup_every_element(abi, dt, M, N, K):
    """17 tile rows by 34 or 33 tile columns over 512 resident workgroups: some store a tile while
    their neighbour on the CU is in its k loop and others have already finished.  Every element
    against the one-thread-per-output kernel, three launches in a row."""
    A, B = rand((M, K), 70, dt), rand((N, K), 71, dt)
    Ad, Bd = A.cuda(), B.cuda()
    S = torch.empty((M, N), dtype=dt, device="cuda")
    assert ac.gemm_tn(abi, Ad, Bd, S, 1.0, ac.SIMPLE) == 0
    for _ in range(3):
        C = torch.full((M, N), float("nan"), dtype=dt, device="cuda")
        assert ac.gemm_tn(abi, Ad, Bd, C, 1.0, ac.ALTERNATE) == 0
        torch.cuda.synchronize()
        d = (C.float() - S.float()).abs()
        bad = d > 2e-2 * S.float().abs() + 2e-2 * (K ** 0.5)
        assert not torch.isnan(C).any() and int(bad.sum()) == 0, (int(bad.sum()), float(d.max()))


def test_config3_bf16_8192_full_size(abi):
    """The metric's own shape on this variant: sampled rows against the CPU oracle and the whole
    result bit for bit against the single-group kernel, which adds the same products in the same order."""
    from gemm_kernels import workloads
    A, B = workloads.bf16_8192(seed=0, device="cuda")
    C = torch.full((8192, 8192), float("nan"), dtype=torch.bfloat16, device="cuda")
    W = torch.full((8192, 8192), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, A, B, C, 1.0, ac.ALTERNATE) == 0 and ac.gemm_tn(abi, A, B, W, 1.0, ac.BASIC) == 0
    torch.cuda.synchronize()
    assert not torch.isnan(C.float()).any()
    assert torch.equal(C.view(torch.int16), W.view(torch.int16))
    rows = torch.arange(0, 8192, 171)
    ref = oracle.gemm_tn_fp32(A[rows.cuda()].cpu(), B.cpu())
    assert oracle.rel_frobenius(C[rows.cuda()].cpu(), ref) <= 1e-2


def test_fp8_is_refused(abi):
    A = torch.zeros(256, 128, device="cuda").to(torch.float8_e4m3fn)
    C = torch.full((256, 256), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn(abi, A, A, C, 1.0, ac.ALTERNATE) == ac.ERR_VARIANT
    torch.cuda.synchronize()
    assert torch.isnan(C.float()).all()
