"""mi355_gemm_tn_noalloc (the entry point that allocates nothing: its K-split partials, tail-split
tiles and repacked operands live in a buffer inside the library's code object) against
mi355_gemm_tn with a caller-allocated workspace, through the C ABI.  Both run the same plan and the
same kernels, so the outputs must agree bit for bit; the calls come in rows, each later one smaller
than the one before, so that the shared buffer still holds the larger problem's partial results.
No counterpart in the reference (its launcher has no workspace, gemm_test.cu:12-92)."""
import pytest
import torch

from oracle import oracle
from tests import abi_ctypes as ac

pytestmark = pytest.mark.gpu


def rand(shape, seed, dtype, std=1.0):
    x = torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * std
    return x.to(dtype)


def both(abi, A, B, variant=ac.AUTO, scale=1.0, out_dtype=torch.bfloat16):
    """(C from mi355_gemm_tn_noalloc, C from mi355_gemm_tn), each NaN-prefilled, on the device."""
    M, N = A.shape[0], B.shape[0]
    Ad, Bd = A.cuda(), B.cuda()
    C0 = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    C1 = torch.full((M, N), float("nan"), dtype=out_dtype, device="cuda")
    print("noalloc case", tuple(A.shape), tuple(B.shape), A.dtype, "variant", variant, flush=True)
    rc = ac.gemm_tn_noalloc(abi, Ad, Bd, C0, scale, variant)
    assert rc == ac.OK, abi.mi355_gemm_strerror(rc)
    rc = ac.gemm_tn(abi, Ad, Bd, C1, scale, variant)
    assert rc == ac.OK, abi.mi355_gemm_strerror(rc)
    torch.cuda.synchronize()
    return C0, C1


def same_bits(C0, C1):
    assert not torch.isnan(C0.float()).any(), "an element was left unwritten"
    return torch.equal(C0.view(torch.int16), C1.view(torch.int16))


# (M, N, K, dtype, what the plan puts into the workspace); every later case of a row is smaller
ROWS = {
    "streaming kernel, K split": [(64, 4096, 14336, torch.bfloat16), (16, 6144, 4096, torch.bfloat16),
                                  (16, 2048, 4096, torch.float16)],
    "tile kernel, uniform K split": [(256, 6144, 4096, torch.bfloat16), (256, 4096, 2048, torch.bfloat16),
                                     (130, 1024, 4096, torch.float16)],
    "tile kernel, tail split": [(4096, 6144, 4096, torch.bfloat16), (4352, 4352, 2048, torch.bfloat16)],
    "tile kernel, two launches, the second with a K split": [(8704, 4096, 2496, torch.bfloat16), (2048, 8448, 6912, torch.float16)],
    "fp8": [(256, 14336, 4096, torch.float8_e4m3fn), (16, 4096, 14336, torch.float8_e4m3fn)],
    "repacked misaligned problem": [(1001, 1003, 1001, torch.bfloat16), (515, 1003, 777, torch.bfloat16)],
}


@pytest.mark.parametrize("row", list(ROWS))
def test_noalloc_matches_the_workspace_entry_point(abi, row):
    wanted_scratch = 0
    for i, (M, N, K, dt) in enumerate(ROWS[row]):
        if dt == torch.float8_e4m3fn:
            A = rand((M, K), 100 + i, torch.float32).clamp_(-200, 200).to(dt)
            B = rand((N, K), 200 + i, torch.float32).clamp_(-200, 200).to(dt)
        else:
            A, B = rand((M, K), 100 + i, dt), rand((N, K), 200 + i, dt)
        need = abi.mi355_gemm_workspace_bytes(M, N, K, ac.torch_code(dt), ac.AUTO)
        assert need <= ac.NOALLOC_SCRATCH_BYTES
        wanted_scratch = max(wanted_scratch, need)
        out_dt = torch.bfloat16 if dt == torch.float8_e4m3fn else dt
        C0, C1 = both(abi, A, B, out_dtype=out_dt)
        assert same_bits(C0, C1), (row, M, N, K)
        # and the pair is not wrong together: sampled rows against the oracle
        rows = torch.arange(0, M, max(1, M // 16))
        ref = oracle.gemm_tn_fp32(A[rows], B)
        assert oracle.rel_frobenius(C0[rows.cuda()].cpu(), ref) <= (3e-2 if dt == torch.float8_e4m3fn else 1e-2)
    assert wanted_scratch > 0, "this row was meant to use the scratch buffer"


def test_noalloc_twice_in_a_row_second_call_smaller(abi):
    """Two calls back to back on one stream with nothing in between, the second on a smaller input
    whose partial planes overlap the first call's in the shared buffer."""
    A1, B1 = rand((64, 14336), 1, torch.bfloat16), rand((4096, 14336), 2, torch.bfloat16)
    A2, B2 = rand((16, 4096), 3, torch.bfloat16), rand((6144, 4096), 4, torch.bfloat16)
    assert abi.mi355_gemm_workspace_bytes(64, 4096, 14336, ac.BF16, ac.AUTO) > \
        abi.mi355_gemm_workspace_bytes(16, 6144, 4096, ac.BF16, ac.AUTO) > 0
    A1d, B1d, A2d, B2d = A1.cuda(), B1.cuda(), A2.cuda(), B2.cuda()
    C1 = torch.full((64, 4096), float("nan"), dtype=torch.bfloat16, device="cuda")
    C2 = torch.full((16, 6144), float("nan"), dtype=torch.bfloat16, device="cuda")
    print("noalloc back to back", flush=True)
    assert ac.gemm_tn_noalloc(abi, A1d, B1d, C1) == ac.OK
    assert ac.gemm_tn_noalloc(abi, A2d, B2d, C2) == ac.OK
    torch.cuda.synchronize()
    W1 = torch.full_like(C1, float("nan"))
    W2 = torch.full_like(C2, float("nan"))
    assert ac.gemm_tn(abi, A1d, B1d, W1) == ac.OK and ac.gemm_tn(abi, A2d, B2d, W2) == ac.OK
    torch.cuda.synchronize()
    assert same_bits(C1, W1) and same_bits(C2, W2)


def test_noalloc_without_scratch_use_has_no_size_limit(abi):
    """A problem whose plan wants no workspace runs whatever its size (here 4096^3: 32 MiB per operand)."""
    assert abi.mi355_gemm_workspace_bytes(4096, 4096, 4096, ac.BF16, ac.AUTO) == 0
    A, B = rand((4096, 4096), 5, torch.bfloat16), rand((4096, 4096), 6, torch.bfloat16)
    C0, C1 = both(abi, A, B)
    assert same_bits(C0, C1)


def test_noalloc_refuses_what_does_not_fit(abi):
    """Misaligned 8191 x 8193 x 8190: the repacked operands alone are 400 MB.  The call must say so
    (never run the slow generic kernel silently) and must leave C alone.  (Split partials never
    exceed the buffer: a plan has at most 256 split items of at most 256 x 256 floats.)"""
    M, N, K = 8191, 8193, 8190
    assert abi.mi355_gemm_workspace_bytes(M, N, K, ac.BF16, ac.AUTO) > ac.NOALLOC_SCRATCH_BYTES
    A = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    B = torch.zeros((N, K), dtype=torch.bfloat16, device="cuda")
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    assert ac.gemm_tn_noalloc(abi, A, B, C) == ac.ERR_SCRATCH
    torch.cuda.synchronize()
    assert torch.isnan(C.float()).all()


def test_noalloc_under_graph_capture_replays(abi):
    """What the entry point is for: one warm call outside any capture (the per-GPU scratch address is
    looked up on the first call), then two calls captured into one graph on one stream -- a K-split
    problem followed by a smaller one whose partial planes overlap the first one's in the shared
    buffer -- replayed with new operand contents, eager work in between, every replay bit for bit
    what mi355_gemm_tn gives.  A replay finds the previous replay's partial planes in the buffer."""
    shapes = [(64, 4096, 14336), (16, 6144, 4096)]
    for M, N, K in shapes:
        assert abi.mi355_gemm_workspace_bytes(M, N, K, ac.BF16, ac.AUTO) > 0
    ops = [(torch.empty(M, K, dtype=torch.bfloat16, device="cuda").normal_(),
            torch.empty(N, K, dtype=torch.bfloat16, device="cuda").normal_(),
            torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")) for M, N, K in shapes]

    def both_calls():
        for A, B, C in ops:
            assert ac.gemm_tn_noalloc(abi, A, B, C) == ac.OK

    print("noalloc graph capture", flush=True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        both_calls()                              # the warm call, outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        both_calls()
    for replay in range(3):
        for A, B, C in ops:
            A.normal_()
            B.normal_()
            C.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for A, B, C in ops:
            want = torch.full_like(C, float("nan"))
            assert ac.gemm_tn(abi, A, B, want) == ac.OK     # eager work between the replays
            torch.cuda.synchronize()
            assert same_bits(C, want), (replay, tuple(C.shape))
