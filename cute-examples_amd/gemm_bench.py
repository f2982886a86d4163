#!/usr/bin/env python3
"""Shape sweep of gemm_kernels.gemm_tn_test against torch.mm (hipBLASLt) on one MI355X.

Counterpart of the reference's kernels/tests/gemm_bench.py: same shape list (:616-623, where a
"shape" (s0, s1) means M = N = s0, K = s1, :502), same figure of merit (TFLOP/s = 2*M*N*K / t,
:502-506) and the same per-launch wall-clock protocol with fresh operands and a cache flush before
every timed launch (:53-62, :285-295) -- with the flush sized for the 256 MB Infinity Cache instead
of H100's L2, hipBLASLt through torch.mm as the comparator instead of the cuBLAS ctypes sweep
(:124-424, NVIDIA-only), and an MI355X entry in the peak table (:587-608).  A second column times
back-to-back launches with HIP events, which is what bench.py reports.  Every shape is also
cross-checked (relative Frobenius distance between the two results on the same operands), and the
run ends with the reference's summary table (:635-672) and, with --out, one JSON file.

    PYTHONPATH=cute-examples_amd python cute-examples_amd/gemm_bench.py [--dtype bf16|fp16] [--runs 100]
                                        [--shapes 1024x1024,8192x16384,4096x14336x4096] [--out sweep.json]
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))   # so that the script runs from any directory

import torch

from gemm_kernels import gemm_tn_test

SHAPES = [(1024, 1024), (2048, 2048), (4096, 4096), (8192, 16384), (8192, 8192), (16384, 4096)]
PEAK_TFLOPS = {"AMD Instinct MI355X": 2500.0}   # dense bf16/fp16 MFMA


def theoretical_peak_tflops():
    name = torch.cuda.get_device_name()
    for key, val in PEAK_TFLOPS.items():
        if key.lower() in name.lower() or "mi355" in name.lower():
            return val
    return 2500.0


def fresh_operands(M, N, K, dtype, flush):
    A = torch.randn(M, K, device="cuda", dtype=dtype)
    B = torch.randn(N, K, device="cuda", dtype=dtype)     # (N, K): already "transposed" for the TN kernel
    C = torch.empty(M, N, device="cuda", dtype=dtype)
    flush.mul_(1.0001)                                     # 512 MB read+written: evicts L2 and the Infinity Cache
    return A, B, C


def wall_clock_per_launch(fn, M, N, K, dtype, runs, flush):
    """The reference's protocol: synchronize, perf_counter, one launch, synchronize."""
    times = []
    for _ in range(runs):
        A, B, C = fresh_operands(M, N, K, dtype, flush)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn(A, B, C)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return sum(times) / len(times)


def events_back_to_back(fn, M, N, K, dtype, runs):
    A = torch.randn(M, K, device="cuda", dtype=dtype)
    B = torch.randn(N, K, device="cuda", dtype=dtype)
    C = torch.empty(M, N, device="cuda", dtype=dtype)
    for _ in range(5):
        fn(A, B, C)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(runs):
        fn(A, B, C)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / runs / 1e3


def cross_check(ours, blas, M, N, K, dtype):
    """||ours - torch.mm||_F / ||torch.mm||_F on one set of operands (both round to the output type,
    so ~2e-3 for bf16 and ~3e-4 for fp16 is rounding alone)."""
    A = torch.randn(M, K, device="cuda", dtype=dtype)
    B = torch.randn(N, K, device="cuda", dtype=dtype)
    C0 = torch.full((M, N), float("nan"), device="cuda", dtype=dtype)
    C1 = torch.empty(M, N, device="cuda", dtype=dtype)
    ours(A, B, C0)
    blas(A, B, C1)
    torch.cuda.synchronize()
    d = (C0.float() - C1.float()).norm() / C1.float().norm()
    return float(d)


def summary_table(rows, peak):
    """The reference's closing table (gemm_bench.py:635-672): one line per shape, time / TFLOP/s per
    implementation and the speed-up; the cuBLAS column of the reference has no counterpart here."""
    out = ["=" * 100, "PERFORMANCE SUMMARY (wall clock per launch, cold caches)", "=" * 100,
           f"{'Shape':<12} {'Custom':<18} {'PyTorch (hipBLASLt)':<20} {'vs PyTorch':<12} {'% of peak':<10} {'rel. diff':<10}",
           f"{'':12} {'(ms / TFLOPS)':<18} {'(ms / TFLOPS)':<20} {'(speedup)':<12} {'(custom)':<10} {'(Frobenius)':<10}",
           "-" * 100]
    for r in rows:
        shape = f"{r['M']}x{r['K']}" if r['M'] == r['N'] else f"{r['M']}x{r['N']}x{r['K']}"
        custom = f"{r['ours_wall_ms']:.3f} / {r['ours_wall_tflops']:.1f}"
        torch_s = f"{r['blas_wall_ms']:.3f} / {r['blas_wall_tflops']:.1f}"
        out.append(f"{shape:<12} {custom:<18} {torch_s:<20} {r['blas_wall_ms'] / r['ours_wall_ms']:<12.2f} "
                   f"{100 * r['ours_wall_tflops'] / peak:<10.1f} {r['rel_diff']:<10.2e}")
    return "\n".join(out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16"])
    ap.add_argument("--runs", type=int, default=100)
    ap.add_argument("--shapes", default=None, help="comma-separated s0xs1 (M = N = s0, K = s1, the reference's notation) or "
                                                   "MxNxK; default: the reference's six")
    ap.add_argument("--json", action="store_true", help="also print one JSON line per shape")
    ap.add_argument("--out", default=None, help="write all rows and the run's parameters to this JSON file")
    a = ap.parse_args()
    dtype = torch.bfloat16 if a.dtype == "bf16" else torch.float16
    shapes = SHAPES if not a.shapes else [tuple(int(x) for x in s.split("x")) for s in a.shapes.split(",")]
    peak = theoretical_peak_tflops()
    flush = torch.ones(128 * 1024 * 1024, device="cuda")   # 512 MB fp32

    ours = lambda A, B, C: gemm_tn_test(A, B, C)
    blas = lambda A, B, C: torch.mm(A, B.t(), out=C)

    rows = []
    print(f"{torch.cuda.get_device_name()}  dtype={a.dtype}  peak={peak:.0f} TFLOP/s  runs={a.runs}")
    hdr = f"{'M=N':>6} {'K':>6} | {'ours ms':>8} {'TF':>7} {'%pk':>5} | {'blas ms':>8} {'TF':>7} {'%pk':>5} | {'ours/blas':>9} || {'ours ev-ms':>10} {'TF':>7} | {'blas ev-ms':>10} {'TF':>7}"
    print(hdr)
    print("-" * len(hdr))
    for shape in shapes:
        if len(shape) not in (2, 3):
            raise SystemExit("a shape is s0xs1 or MxNxK, not %r" % (shape,))
        M, N, K = (shape[0], shape[0], shape[1]) if len(shape) == 2 else shape
        flops = 2.0 * M * N * K
        for fn in (ours, blas):                              # warm-up, as gemm_bench.py:473-481
            A, B, C = fresh_operands(M, N, K, dtype, flush)
            for _ in range(5):
                fn(A, B, C)
        rel = cross_check(ours, blas, M, N, K, dtype)
        t_ours = wall_clock_per_launch(ours, M, N, K, dtype, a.runs, flush)
        t_blas = wall_clock_per_launch(blas, M, N, K, dtype, a.runs, flush)
        e_ours = events_back_to_back(ours, M, N, K, dtype, a.runs)
        e_blas = events_back_to_back(blas, M, N, K, dtype, a.runs)
        tf = lambda t: flops / t / 1e12
        label = f"{M:>6}" if M == N else f"{M}x{N}"
        print(f"{label} {K:>6} | {t_ours*1e3:8.4f} {tf(t_ours):7.1f} {100*tf(t_ours)/peak:5.1f} | "
              f"{t_blas*1e3:8.4f} {tf(t_blas):7.1f} {100*tf(t_blas)/peak:5.1f} | {t_blas/t_ours:9.3f} || "
              f"{e_ours*1e3:10.4f} {tf(e_ours):7.1f} | {e_blas*1e3:10.4f} {tf(e_blas):7.1f}", flush=True)
        rows.append({"M": M, "N": N, "K": K, "dtype": a.dtype, "rel_diff": rel,
                     "ours_wall_ms": t_ours * 1e3, "blas_wall_ms": t_blas * 1e3,
                     "ours_wall_tflops": tf(t_ours), "blas_wall_tflops": tf(t_blas),
                     "ours_event_ms": e_ours * 1e3, "blas_event_ms": e_blas * 1e3,
                     "ours_tflops": tf(e_ours), "blas_tflops": tf(e_blas)})
    print()
    print(summary_table(rows, peak))
    if a.json:
        for r in rows:
            print(json.dumps(r))
    if a.out:
        with open(a.out, "w") as f:
            json.dump({"device": torch.cuda.get_device_name(), "dtype": a.dtype, "runs": a.runs,
                       "peak_tflops": peak, "comparator": "torch.mm (hipBLASLt)", "rows": rows}, f, indent=1)


if __name__ == "__main__":
    main()
