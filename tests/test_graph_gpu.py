"""The library under HIP graph capture (torch.cuda.CUDAGraph): every entry point only enqueues
kernels on the caller's stream (no allocation, no memset node, no synchronisation), so a captured
sequence must replay with new operand contents and give what the eager calls give.  Each graph is
replayed several times with eager work and synchronisations in between, and every replay is
compared bit for bit with the eager result."""
import pytest
import torch

import gemm_kernels

pytestmark = pytest.mark.gpu


def _capture(fn):
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()                                   # warm-up outside the capture (workspace in the allocator's pool)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


@pytest.mark.parametrize("shape", [(512, 768, 1024), (16, 4096, 4096), (512, 6144, 4096), (4096, 6144, 4096), (8704, 4096, 2496)])
def test_bf16_gemm_replays(shape):
    """Tile kernel, streaming kernel with its K split, tile kernel with K split and with tail split, and a problem that
    runs as two launches, the second with a K split."""
    M, N, K = shape
    A = torch.randn(M, K, device="cuda").bfloat16()
    B = torch.randn(N, K, device="cuda").bfloat16()
    C = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    g = _capture(lambda: gemm_kernels.gemm_tn_test(A, B, C))
    for i in range(3):
        A.copy_(torch.randn(M, K, device="cuda").bfloat16())
        B.copy_(torch.randn(N, K, device="cuda").bfloat16())
        C.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        got = C.clone()
        want = torch.empty_like(C)
        gemm_kernels.gemm_tn_test(A, B, want)      # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), i


def test_quantise_and_fp8_gemms_replay():
    """Per-tensor and block-scaled pipelines: quantisers, scale shuffle, both fp8 GEMMs in one graph."""
    M, N, K = 512, 1024, 2048
    X = torch.randn(M, K, device="cuda").bfloat16()
    W = torch.randn(N, K, device="cuda").bfloat16()
    C1 = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    C2 = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)

    def pipeline(c1, c2):
        (xq, sx), (wq, sw) = gemm_kernels.quantize_e4m3(X), gemm_kernels.quantize_e4m3(W)
        gemm_kernels.gemm_tn_fp8(xq, wq, sx, sw, c1)
        (xm, bx), (wm, bw) = gemm_kernels.quantize_mxfp8(X), gemm_kernels.quantize_mxfp8(W)
        gemm_kernels.gemm_tn_mxfp8(xm, wm, bx, bw, c2)

    g = _capture(lambda: pipeline(C1, C2))
    for i in range(3):
        X.copy_((torch.randn(M, K, device="cuda") * (i + 1)).bfloat16())
        W.copy_(torch.randn(N, K, device="cuda").bfloat16())
        C1.fill_(float("nan"))
        C2.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        got1, got2 = C1.clone(), C2.clone()
        want1, want2 = torch.empty_like(C1), torch.empty_like(C2)
        pipeline(want1, want2)
        torch.cuda.synchronize()
        assert torch.equal(got1.view(torch.int16), want1.view(torch.int16)), i
        assert torch.equal(got2.view(torch.int16), want2.view(torch.int16)), i
        ref = X.float() @ W.float().t()
        assert float((got1.float() - ref).norm() / ref.norm()) < 6e-2
        assert float((got2.float() - ref).norm() / ref.norm()) < 6e-2


def test_host_threads_on_their_own_streams():
    """Four host threads, each on its own stream, issue different problems at the same time (tile
    kernel with a tail split, streaming kernel with a K split, fp8, block-scaled fp8): the library
    keeps no state between calls, so every result equals the one computed alone."""
    import threading
    torch.manual_seed(0)
    jobs = []
    for kind, (M, N, K) in (("bf16", (4096, 6144, 1024)), ("bf16", (16, 4096, 4096)), ("fp8", (512, 1024, 2048)),
                            ("mx", (768, 768, 2048))):
        X = torch.randn(M, K, device="cuda").bfloat16()
        W = torch.randn(N, K, device="cuda").bfloat16()
        jobs.append((kind, X, W))

    def run(kind, X, W, C):
        if kind == "bf16":
            gemm_kernels.gemm_tn_test(X, W, C)
        elif kind == "fp8":
            (xq, sx), (wq, sw) = gemm_kernels.quantize_e4m3(X), gemm_kernels.quantize_e4m3(W)
            gemm_kernels.gemm_tn_fp8(xq, wq, sx, sw, C)
        else:
            (xq, sx), (wq, sw) = gemm_kernels.quantize_mxfp8(X, True), gemm_kernels.quantize_mxfp8(W, True)
            gemm_kernels.gemm_tn_mxfp8(xq, wq, sx, sw, C, True)

    alone = []
    for kind, X, W in jobs:
        C = torch.empty(X.shape[0], W.shape[0], dtype=torch.bfloat16, device="cuda")
        run(kind, X, W, C)
        alone.append(C)
    torch.cuda.synchronize()

    results = [None] * len(jobs)
    errors = []

    def worker(i):
        try:
            kind, X, W = jobs[i]
            stream = torch.cuda.Stream()
            stream.wait_stream(torch.cuda.default_stream())
            outs = []
            with torch.cuda.stream(stream):
                for _ in range(20):
                    C = torch.full((X.shape[0], W.shape[0]), float("nan"), dtype=torch.bfloat16, device="cuda")
                    run(kind, X, W, C)
                    outs.append(C)
            stream.synchronize()
            results[i] = outs
        except Exception as e:  # surfaced below: an exception in a thread would otherwise be lost
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i, outs in enumerate(results):
        for C in outs:
            assert torch.equal(C.view(torch.int16), alone[i].view(torch.int16)), i
