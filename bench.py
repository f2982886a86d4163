#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extras] [--no-cpu]
                    [--no-calibrate] [--no-fp8]

A step is one gemm launch over one set of synthetic operands already resident in HBM.  The
headline workload is bf16 M=N=K=8192, Normal(0,1) operands (the configuration the metric is
quoted on); fp8 8192^3 (per-tensor scales and MX block scales), bf16 4096^3, fp16 512^3 and the
skinny projection shapes are timed with fewer steps and reported under "extras".  The metric names
two configurations, so fp8 e4m3 8192^3 gets a block of its own ("fp8": value, roofline, cpu_baseline)
measured with the same protocol and the same K and W as the headline.  Prints ONE JSON line.

Clock settling.  The shader clock of an idle GPU needs tens of milliseconds of load to reach the
level it then sustains (an 8192^3 GEMM runs ~13 % slower in the first few milliseconds after an
idle period, ~5 % slower over the first 60 launches).  Every measurement therefore begins with a settle phase that is
not part of W or K: the same launch repeated, in batches timed with HIP events, for at least
150 ms and until three consecutive batches agree within 1 % (at most 2 s).  It is reported as
settle_launches / settle_ms; the W warm-up and K timed launches follow it back to back.

Calibration (on by default, --no-calibrate skips it): the library's MFMA-only kernel on the
workload's own operands and its plain read kernel give roofline.measured_mfma_ceiling and
roofline.measured_hbm_read, what this GPU sustains with nothing but matrix-core work / nothing but
loads.  roofline.frac stays against the published peak.

Protocol follows the reference's benchmark (kernels/tests/gemm_bench.py:285-295, :502-506):
warm-up, then timed launches, TFLOP/s = 2*M*N*K / t — with HIP events on the launch stream
instead of wall-clock around each launch, and operand sets rotated for the memory-bound shapes
so they are not served from the 256 MB Infinity Cache.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "cute-examples_amd"))

METRIC = "GEMM TFLOP/s and % of MI355X dense MFMA peak, bf16 8192^3 and fp8 8192^3"
PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "e4m3": 5000.0}   # dense MFMA, MI355X
PEAK_HBM_GBS = 8000.0
# HBM-side bytes per launch of the dominant kernel, from two rocprofv3 --pmc runs of this script
# (FETCH_SIZE, then WRITE_SIZE, each with --copy-calibration and scaled by what the same counter
# reads for the 1 GiB copy: x2.000 and x1.000).  Workloads without a counter run report null.
MEASURED_TRAFFIC_BYTES = {"bf16_8192": 1.747e9, "fp8_8192": 0.941e9, "mxfp8_8192": 0.975e9, "bf16_4096": 2.354e8,
                          "skinny_16_14336_4096": 1.190e8, "skinny_64_14336_4096": 1.236e8, "skinny_64_4096_14336": 1.527e8,
                          "skinny_256_14336_4096": 1.560e8, "skinny_256_6144_4096": 1.209e8, "skinny_128_8192_4096": 1.131e8}
TRAFFIC_PROFILE = {"bf16_8192": "profiles/gemm_tn_tile_ring__bf16_8192.md", "fp8_8192": "profiles/gemm_tn_tile_ring__fp8_8192.md",
                   "mxfp8_8192": "profiles/gemm_tn_tile_ring__mxfp8_8192.md", "bf16_4096": "profiles/gemm_tn_tile_ring__bf16_4096.md",
                   "skinny_16_14336_4096": "profiles/gemm_tn_stream__skinny_16_14336_4096.md",
                   "skinny_64_14336_4096": "profiles/gemm_tn_stream__skinny_64_14336_4096.md",
                   "skinny_64_4096_14336": "profiles/gemm_tn_stream__skinny_64_4096_14336.md",
                   "skinny_256_14336_4096": "profiles/gemm_tn_tile_ring__skinny_256_14336_4096.md",
                   "skinny_256_6144_4096": "profiles/gemm_tn_tile_ring__skinny_256_6144_4096.md",
                   "skinny_128_8192_4096": "profiles/gemm_tn_tile_ring__skinny_128_8192_4096.md"}
SETTLE_MIN_MS, SETTLE_MAX_MS, SETTLE_BATCH_MS = 150.0, 2000.0, 10.0
# Counter readings of the committed rocprofv3 profiles of this script (not re-measured in a plain
# run): the share of SIMD cycles with an MFMA in flight and the shader clock during the kernel
# (busy CU cycles / CUs / traced duration).
PROFILED = {
    "bf16_8192": {"mfma_busy": 0.906, "shader_clock_ghz": 1.71, "lds_bank_conflict_cycles": 0,
                  "source": "profiles/gemm_tn_tile_ring__bf16_8192.md"},
    "fp8_8192": {"mfma_busy": 0.870, "shader_clock_ghz": 1.78, "lds_bank_conflict_cycles": 0,
                 "source": "profiles/gemm_tn_tile_ring__fp8_8192.md"},
}


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    # The shader clock needs some tens of milliseconds of load to settle (the first ~60 launches of
    # an 8192^3 GEMM run about 5 % slower), hence the long default warm-up.
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=100)
    p.add_argument("--workload", default="bf16_8192")
    p.add_argument("--variant", default="auto")
    p.add_argument("--no-extras", action="store_true")
    p.add_argument("--no-cpu", action="store_true")
    p.add_argument("--no-fp8", action="store_true", help="skip the fp8 8192^3 block of the metric")
    p.add_argument("--calibrate", action="store_true", help="(default) measure the MFMA-only and plain-read ceilings")
    p.add_argument("--no-calibrate", action="store_true")
    p.add_argument("--no-vendor", action="store_true", help="skip torch.mm / torch._scaled_mm on the same operands")
    p.add_argument("--no-settle", action="store_true", help="skip the clock-settle phase in front of every measurement")
    p.add_argument("--copy-calibration", action="store_true",
                   help="also run three 1 GiB device-to-device copies (known traffic: 1 GiB read + 1 GiB "
                        "written each) so that a rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this "
                        "command can be scaled by what the same counter reads for a plain copy")
    return p.parse_args()


def settle(call, enabled=True):
    """Clock-settle phase: repeat the launch in event-timed batches of ~10 ms for at least
    SETTLE_MIN_MS and until three consecutive batches agree within 1 %, at most SETTLE_MAX_MS.
    Returns (launches, total ms, ms per launch of the last batch)."""
    import torch
    if not enabled:
        return 0, 0.0, None
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    call()
    e1.record()
    torch.cuda.synchronize()
    per = max(e0.elapsed_time(e1), 1e-3)
    batch = max(1, min(2000, int(SETTLE_BATCH_MS / per)))
    launches, total, history = 1, per, []
    while total < SETTLE_MAX_MS:
        e0.record()
        for _ in range(batch):
            call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        launches += batch
        total += ms
        history.append(ms / batch)
        if total >= SETTLE_MIN_MS and len(history) >= 3:
            last = history[-3:]
            if max(last) <= 1.01 * min(last):
                break
    return launches, total, history[-1] if history else per


def time_calls(call, steps, warmup, do_settle=True):
    """Settle phase, then `warmup` untimed launches, then HIP events on the current stream around
    `steps` back-to-back launches -> (ms per launch, wall ms per launch, settle launches, settle ms)."""
    import torch
    n_settle, settle_ms, _ = settle(call, do_settle)
    for _ in range(warmup):
        call()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        call()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    return e0.elapsed_time(e1) / steps, wall_ms, n_settle, settle_ms


def per_launch_ms(call, steps):
    """A second pass with an event pair around every launch -> (median, min) ms.  Includes the gap
    between launches, so it is not the figure `value` is computed from."""
    import torch
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        call()
        ev[i + 1].record()
    torch.cuda.synchronize()
    t = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    return t[len(t) // 2], t[0]


def build_case(name, variant, device="cuda", seed=0):
    import torch
    import gemm_kernels
    from gemm_kernels import workloads as w

    rot = 1
    if name == "bf16_8192":
        A, B = w.bf16_8192(seed, device)
        sets, tag, fp8 = [(A, B)], "bf16", None
    elif name == "bf16_4096":
        sets, tag, fp8 = [w.bf16_4096(seed + 10 * i, device) for i in range(4)], "bf16", None
    elif name == "fp16_512":
        sets, tag, fp8 = [w.fp16_512(seed, device)], "f16", None
    elif name == "fp8_8192":
        A, B, sa, sb = w.fp8_8192(seed, device)
        sets, tag, fp8 = [(A, B)], "e4m3", (float(sa), float(sb))
    elif name == "mxfp8_8192":
        A, sa, B, sb = w.mxfp8_8192(seed, device)
        # weights-style call: the block scales are re-laid once, outside the timed launches
        sets, tag, fp8 = [(A, B)], "e4m3", ("mx", gemm_kernels.shuffle_mx_scales(sa), gemm_kernels.shuffle_mx_scales(sb))
    elif name.startswith("bf16_shape_") or name.startswith("fp16_shape_"):
        # any shape: bf16_shape_M_N_K / fp16_shape_M_N_K, Normal(0,1) operands
        M, N, K = (int(x) for x in name.split("_")[2:])
        dt = torch.bfloat16 if name.startswith("bf16") else torch.float16
        gen = torch.Generator(device=device).manual_seed(seed)
        sets = [(torch.randn(M, K, device=device, generator=gen).to(dt), torch.randn(N, K, device=device, generator=gen).to(dt))]
        tag, fp8 = ("bf16" if dt == torch.bfloat16 else "f16"), None
    elif name.startswith("skinny_"):
        M, N, K = (int(x) for x in name.split("_")[1:])
        # rotate operand sets so weights come from HBM, not the Infinity Cache (256 MB)
        rot = max(2, int(600e6 // (N * K * 2)) + 1)
        sets, tag, fp8 = [w.skinny(M, N, K, seed + 10 * i, device) for i in range(rot)], "bf16", None
    elif name.startswith("skinnyfp8_") or name.startswith("skinnymx_"):
        # the same small-M shapes with e4m3 weights: unit per-tensor scales, or OCP MX block scales
        # quantised by the library into the layout the kernels read
        M, N, K = (int(x) for x in name.split("_")[1:])
        rot = max(2, int(600e6 // (N * K)) + 1)
        sets = []
        for i in range(rot):
            X, W = w.skinny(M, N, K, seed + 10 * i, device)
            if name.startswith("skinnymx_"):
                (xq, px), (wq, pw) = gemm_kernels.quantize_mxfp8(X, shuffled=True), gemm_kernels.quantize_mxfp8(W * 50.0, shuffled=True)
                sets.append((xq, wq, px, pw))
            else:
                sets.append((X.to(torch.float8_e4m3fn), (W * 50.0).to(torch.float8_e4m3fn)))
        tag, fp8 = "e4m3", (("mxsets",) if name.startswith("skinnymx_") else (1.0, 1.0))
    elif name.startswith("quant_e4m3_") or name.startswith("quant_mxfp8_"):
        # the quantisers in front of the fp8 GEMMs: bf16 (rows, K) -> e4m3 with one scale per tensor (two passes over
        # x: maximum, then cast) or with one E8M0 scale per 32 elements in the GEMM's layout (one pass)
        rows, K = (int(x) for x in name.split("_")[2:])
        x = torch.randn(rows, K, device=device, generator=torch.Generator(device=device).manual_seed(seed)).to(torch.bfloat16)
        per_tensor = name.startswith("quant_e4m3_")

        def call():
            if per_tensor:
                gemm_kernels.quantize_e4m3(x)
            else:
                gemm_kernels.quantize_mxfp8(x, shuffled=True)
        n = rows * K
        nbytes = (2 * 2 * n + n) if per_tensor else (2 * n + n + n // 32)
        return call, 0.0, nbytes, "bf16", (rows, 0, K), [(x, x)], None, None
    else:
        raise SystemExit("unknown workload " + name)
    M, K = sets[0][0].shape
    N = sets[0][1].shape[0]
    out_dt = torch.bfloat16 if fp8 else sets[0][0].dtype
    C = torch.empty((M, N), dtype=out_dt, device=device)
    state = {"i": 0}

    def call():
        A, B = sets[state["i"] % len(sets)][:2]
        state["i"] += 1
        if fp8 and fp8[0] == "mxsets":
            _, _, pa, pb = sets[(state["i"] - 1) % len(sets)]
            gemm_kernels.gemm_tn_mxfp8(A, B, pa, pb, C, True)
        elif fp8 and fp8[0] == "mx":
            gemm_kernels.gemm_tn_mxfp8(A, B, fp8[1], fp8[2], C, True)
        elif fp8:
            gemm_kernels.gemm_tn_fp8(A, B, fp8[0], fp8[1], C, variant)
        else:
            gemm_kernels.gemm_tn(A, B, C, variant)

    es = sets[0][0].element_size()
    nbytes = (M * K + N * K) * es + M * N * C.element_size()
    if fp8 and fp8[0] in ("mx", "mxsets"):
        nbytes += (M + N) * (K // 32)
    return call, 2.0 * M * N * K, nbytes, tag, (M, N, K), sets, C, fp8


def measure(name, variant, steps, warmup, do_settle=True):
    call, flops, nbytes, tag, mnk, sets, C, fp8 = build_case(name, variant)
    ms, wall_ms, n_settle, settle_ms = time_calls(call, steps, warmup, do_settle)
    med, mn = per_launch_ms(call, steps)
    tflops = flops / ms / 1e9
    row = {"workload": name, "M": mnk[0], "N": mnk[1], "K": mnk[2], "dtype": tag, "steps": steps, "warmup": warmup,
           "settle_launches": n_settle, "settle_ms": round(settle_ms, 1),
           "ms": round(ms, 5), "wall_ms": round(wall_ms, 5), "launch_ms_median": round(med, 5),
           "launch_ms_min": round(mn, 5), "tflops": round(tflops, 2),
           "pct_mfma_peak": round(100 * tflops / PEAK_TFLOPS[tag], 2),
           "gbs": round(nbytes / ms / 1e6, 1), "pct_hbm_peak": round(100 * nbytes / ms / 1e6 / PEAK_HBM_GBS, 2)}
    return row, (sets, C, fp8, flops, nbytes)


def roofline_of(row, workload, variant, sets, flops, nbytes):
    """The roofline object of one measured workload (the dominant kernel is its only GEMM kernel)."""
    import gemm_kernels
    traffic = MEASURED_TRAFFIC_BYTES.get(workload)
    if not workload.startswith(("skinny", "quant_")):
        roof = {"bound": "mfma", "achieved": row["tflops"], "peak": PEAK_TFLOPS[row["dtype"]],
                "unit": "TFLOP/s", "frac": round(row["tflops"] / PEAK_TFLOPS[row["dtype"]], 4), "traffic": traffic}
    else:
        roof = {"bound": "hbm", "achieved": row["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(row["gbs"] / PEAK_HBM_GBS, 4), "traffic": traffic}
    # the counters are not read in this run: the figure is the one of the committed profile of this command
    roof["traffic_source"] = (TRAFFIC_PROFILE[workload] + " (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this script; not re-measured)") if traffic else None
    if workload.startswith("quant_"):
        roof["kernel"] = "amax_kernel + quantize_kernel" if workload.startswith("quant_e4m3") else "mx_quantize_shuffled_kernel"
    else:
        roof["kernel"] = gemm_kernels.select_variant(row["M"], row["N"], row["K"], sets[0][0].dtype) \
            if variant == "auto" else variant
    roof["flops_per_launch"] = flops
    roof["algorithmic_bytes_per_launch"] = nbytes
    roof["avg_launch_ms"] = row["ms"]
    roof["launch_ms_median"], roof["launch_ms_min"] = row["launch_ms_median"], row["launch_ms_min"]
    return roof


MFMA_SHAPES = {"bf16": ("16x16x32", "32x32x16"), "f16": ("16x16x32", "32x32x16"), "e4m3": ("16x16x128", "32x32x64")}


def calibrate(A, B, do_settle=True, read=True):
    """The library's two ceiling kernels through its C ABI: matrix cores only, on the workload's own
    operands (dtype of A) -- on the MFMA shape the kernels use and on the 32-wide shape they do not --
    and a plain read of 1 GiB.  Returns the two roofline entries (the second None without `read`)."""
    import ctypes
    import torch
    lib = ctypes.CDLL(os.path.join(ROOT, "cute-examples_amd", "gemm_kernels", "libmi355gemm.so"))
    vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    lib.mi355_calibrate_sink_bytes.restype = sz
    lib.mi355_calibrate_mfma_shape.argtypes = [ci, ci, vp, sz, vp, sz, ci, vp, ctypes.POINTER(ctypes.c_double), vp]
    lib.mi355_calibrate_read.argtypes = [vp, sz, vp, vp]
    code = {torch.bfloat16: 0, torch.float16: 1, torch.float8_e4m3fn: 2}[A.dtype]
    tag = {0: "bf16", 1: "f16", 2: "e4m3"}[code]
    sink = torch.empty(lib.mi355_calibrate_sink_bytes(), dtype=torch.uint8, device=A.device)
    flops = ctypes.c_double()
    iters = 4000   # ~2 ms per launch
    stream = torch.cuda.current_stream().cuda_stream

    def mfma_on(a, b, wide):
        def run():
            rc = lib.mi355_calibrate_mfma_shape(code, wide, a.data_ptr(), a.numel() * a.element_size(), b.data_ptr(),
                                                b.numel() * b.element_size(), iters, sink.data_ptr(), ctypes.byref(flops), stream)
            assert rc == 0, rc
        return run
    ms, _, n_settle, settle_ms = time_calls(mfma_on(A, B, 0), 40, 5, do_settle)
    mfma_entry = {"value": round(flops.value / ms / 1e9, 1), "unit": "TFLOP/s", "ms_per_launch": round(ms, 4),
                  "settle_launches": n_settle, "settle_ms": round(settle_ms, 1), "mfma_shape": MFMA_SHAPES[tag][0],
                  "what": "mi355_calibrate_mfma_shape: 4 waves per CU, the tile kernel's MFMA pattern on fragments of this "
                          "workload's operands held in registers; no LDS, no copies, no barriers"}
    # The same loop on the 32-wide MFMA shape, which the kernels do not use: what the choice of shape
    # is worth on this GPU and this data.
    ms_wide, _, _, _ = time_calls(mfma_on(A, B, 1), 40, 5, do_settle)
    mfma_entry["by_shape"] = {MFMA_SHAPES[tag][0]: mfma_entry["value"],
                              MFMA_SHAPES[tag][1]: round(flops.value / ms_wide / 1e9, 1)}
    # The kernels' shape on all-zero operands: no data toggling, so the board power limit does not bind
    # and the clock stays near nominal.  The gap to the figure above is what the data costs in clock.
    zeros = torch.zeros(1 << 20, dtype=torch.uint8, device=A.device)
    ms0, _, _, _ = time_calls(mfma_on(zeros, zeros, 0), 40, 5, do_settle)
    mfma_entry["value_zero_operands"] = round(flops.value / ms0 / 1e9, 1)
    read_entry = None
    if read:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=A.device)
        src.view(torch.int32).random_()

        def read_all():
            rc = lib.mi355_calibrate_read(src.data_ptr(), src.numel(), sink.data_ptr(), stream)
            assert rc == 0, rc
        ms, _, n_settle, settle_ms = time_calls(read_all, 100, 10, do_settle)
        read_entry = {"value": round(src.numel() / ms / 1e6, 1), "unit": "GB/s", "ms_per_launch": round(ms, 4),
                      "settle_launches": n_settle, "settle_ms": round(settle_ms, 1),
                      "what": "mi355_calibrate_read: 16-byte loads over 1 GiB (four times the Infinity Cache), nothing else"}
        del src
    del sink
    torch.cuda.empty_cache()
    return mfma_entry, read_entry


def clock_under_load(sets, C, fp8, variant, flops, ms_hint, do_settle):
    """The shader clock while this workload's launches run, without a profiler: the library's clock probe (single
    waves that sleep and sample the cycle counter and the 100 MHz counter) runs on a second stream beside a train of
    launches long enough to outlast it.  Returns the clock (mean over the probe's waves, and by XCD), the time per
    launch meanwhile, and whether the probe really ended before the launches did."""
    import ctypes
    import torch
    import gemm_kernels
    lib = ctypes.CDLL(os.path.join(ROOT, "cute-examples_amd", "gemm_kernels", "libmi355gemm.so"))
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.mi355_clock_probe_bytes.restype = ctypes.c_size_t
    lib.mi355_clock_probe_bytes.argtypes = [ci, ci]
    lib.mi355_clock_probe.argtypes = [ci, ci, ci, vp, vp]
    A, B = sets[0][:2]
    if fp8:
        def call():
            gemm_kernels.gemm_tn_fp8(A, B, fp8[0], fp8[1], C, variant)
    else:
        def call():
            gemm_kernels.gemm_tn(A, B, C, variant)
    waves, samples, pause = 32, 100, 8                      # 800 sleeps of 8128 cycles: 2.7 ms at 2.4 GHz, 6.5 ms at 1 GHz
    launches = int(2 * 6.5 / max(ms_hint, 1e-3)) + 4        # twice the slowest probe
    out = torch.zeros(lib.mi355_clock_probe_bytes(waves, samples) // 8, dtype=torch.int64, device=A.device)
    side = torch.cuda.Stream()
    started, ended, probe_ended = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    # A stream's hardware queue is set up at its first launch, which disturbs whatever runs then: get that over with.
    assert lib.mi355_clock_probe(1, 2, 1, out.data_ptr(), side.cuda_stream) == 0
    torch.cuda.synchronize()
    settle(call, do_settle)
    for _ in range(3):
        call()
    started.record()
    for _ in range(launches):
        call()
    ended.record()
    side.wait_event(started)
    rc = lib.mi355_clock_probe(waves, samples, pause, out.data_ptr(), side.cuda_stream)
    assert rc == 0, rc
    probe_ended.record(side)
    torch.cuda.synchronize()
    got = out.view(waves, 2, samples + 1).cpu()
    cycles, ticks = got[:, 0, 1:].double(), got[:, 1, 1:].double()
    ghz = (cycles[:, -1] - cycles[:, 0]) / (ticks[:, -1] - ticks[:, 0]) / 10.0     # a tick is 10 ns
    by_xcd = {}
    for w in range(waves):
        by_xcd.setdefault(int(got[w, 0, 0]), []).append(float(ghz[w]))
    by_xcd = {str(k): round(sum(v) / len(v), 3) for k, v in sorted(by_xcd.items())}
    ms = started.elapsed_time(ended) / launches
    return {"value": round(float(ghz.mean()), 3), "unit": "GHz", "by_xcd": by_xcd,
            "min_xcd": min(by_xcd.values()), "max_xcd": max(by_xcd.values()),
            "ms_per_launch_meanwhile": round(ms, 5), "tflops_meanwhile": round(flops / ms / 1e9, 1),
            "launches": launches, "probe_ms": round(started.elapsed_time(probe_ended), 3),
            "probe_inside_launches": started.elapsed_time(probe_ended) < started.elapsed_time(ended),
            "what": "mi355_clock_probe: %d waves x %d samples of s_memtime (shader cycles) and s_memrealtime (100 MHz) on a "
                    "second stream beside the launches" % (waves, samples)}


def guarded(yardstick, *args):
    """A yardstick beside the measurement must not cost the measurement: None (and a line on stderr) if it fails."""
    try:
        return yardstick(*args)
    except Exception as e:   # noqa: BLE001
        print("bench.py: %s not available: %s: %s" % (yardstick.__name__, type(e).__name__, str(e)[:200]), file=sys.stderr)
        return None


def vendor_same_run(sets, C, fp8, flops, steps, warmup, do_settle):
    """The vendor library on the same operands, same protocol (settle, W warm-up, K timed launches):
    torch.mm (hipBLASLt) for the 16-bit types, torch._scaled_mm for e4m3 with per-tensor scales.
    A yardstick of what this GPU gives a tuned kernel today; None with the reason if torch refuses."""
    import torch
    A, B = sets[0][:2]
    Bt = B.t()
    try:
        if fp8:
            sa = torch.tensor(float(fp8[0]), dtype=torch.float32, device=A.device)
            sb = torch.tensor(float(fp8[1]), dtype=torch.float32, device=A.device)

            def call():
                torch._scaled_mm(A, Bt, scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16, out=C)
            what = "torch._scaled_mm(A_q, B_q.T, scale_a, scale_b, out_dtype=bf16) on the same operands"
        else:
            def call():
                torch.mm(A, Bt, out=C)
            what = "torch.mm(A, B.T) (hipBLASLt) on the same operands"
        call()
        torch.cuda.synchronize()
        ms, _, n_settle, settle_ms = time_calls(call, steps, warmup, do_settle)
    except Exception as e:   # noqa: BLE001  (a yardstick, not the product: report and go on)
        return {"value": None, "unit": "TFLOP/s", "what": "not available: %s: %s" % (type(e).__name__, str(e)[:160])}
    return {"value": round(flops / ms / 1e9, 2), "unit": "TFLOP/s", "ms_per_launch": round(ms, 5), "steps": steps,
            "warmup": warmup, "settle_launches": n_settle, "settle_ms": round(settle_ms, 1), "what": what}


def cpu_baseline(A, B, total_rows, scale=1.0, budget_s=12.0, native_budget_s=5.0):
    """The oracle's fp32 matmul (the reference's ground truth, gemm_test.py:36) timed on the host
    cores on a bounded sample: as many row blocks of A against all of B as fit the budget.  For fp8
    operands this is the fp32 product of the dequantised operands times scale_a * scale_b."""
    import torch
    from oracle import oracle
    Bc = B.cpu()
    N, K = Bc.shape
    rows = min(1024, A.shape[0])
    Ac = A[:rows].cpu()   # the caller may hand over just these rows (already on the host)
    oracle.gemm_tn_fp32(Ac[:64], Bc, scale)            # warm-up (thread pool, conversions)
    t0 = time.perf_counter()
    done = 0
    while True:
        oracle.gemm_tn_fp32(Ac, Bc, scale)
        done += rows
        el = time.perf_counter() - t0
        if el > budget_s or done >= 16 * total_rows:
            break
    tflops = 2.0 * done * N * K / el / 1e12
    # The same product in the operands' own 16-bit type, where torch has a CPU kernel for it.
    native = None
    if Ac.dtype in (torch.bfloat16, torch.float16) and native_budget_s > 0:
        try:
            torch.matmul(Ac[:64], Bc.T)
            t0, n_done = time.perf_counter(), 0
            while True:
                torch.matmul(Ac, Bc.T)
                n_done += rows
                el_n = time.perf_counter() - t0
                if el_n > native_budget_s or n_done >= 16 * total_rows:
                    break
            native = round(2.0 * n_done * N * K / el_n / 1e12, 4)
        except RuntimeError:
            native = None
    kind = "e4m3->fp32" if Ac.dtype == torch.float8_e4m3fn else "%s->fp32" % str(Ac.dtype).split(".")[-1]
    return {"value": round(tflops, 4), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "native_16bit_value": native,
            "sample": "%d rows in %.1f s: %d-row blocks of A x all of B (N=%d, K=%d), fp32 torch.matmul incl. %s casts; %d cpus"
                      % (done, el, rows, N, K, kind, os.cpu_count())}


def larger_shapes(steps, do_settle):
    """Two larger bf16 problems (twice the K; twice the M and N with half the K), this library and the vendor
    library one after the other on the same operands, same protocol.  {"M_N_K": {tflops, torch_mm_tflops, vs_torch_mm}}"""
    import torch
    out = {}
    for (M, N, K) in ((8192, 8192, 16384), (16384, 16384, 4096)):
        row, keep = measure("bf16_shape_%d_%d_%d" % (M, N, K), "auto", steps, steps, do_settle)
        sets, C, fp8, flops, _ = keep
        vendor = vendor_same_run(sets, C, fp8, flops, steps, steps, do_settle)
        out["%d_%d_%d" % (M, N, K)] = {
            "ms": row["ms"], "tflops": row["tflops"], "frac": round(row["tflops"] / PEAK_TFLOPS["bf16"], 4),
            "torch_mm_tflops": vendor["value"],
            "vs_torch_mm": round(row["tflops"] / vendor["value"], 4) if vendor["value"] else None}
        del sets, C, keep
        torch.cuda.empty_cache()
    return out


def other_configs(extras, mfma_ceiling, hbm_read):
    """The other configurations the baseline names (the nine small-M projection shapes, bf16 4096^3,
    fp16 512^3) in brief: time per launch, achieved rate, fraction of the published peak and of the
    ceiling measured in this run (MFMA-only loop on the headline's operands / plain read)."""
    wanted = ["bf16_4096", "fp16_512"] + ["skinny_%d_%d_%d" % (m, n, k) for (n, k) in ((14336, 4096), (4096, 14336), (6144, 4096))
                                          for m in (16, 64, 256)]
    out = {}
    for row in extras:
        name = row["workload"]
        if name not in wanted or "variant" in row:
            continue
        if name.startswith("skinny"):
            e = {"ms": row["ms"], "achieved": row["gbs"], "unit": "GB/s", "bound": "hbm",
                 "frac": round(row["gbs"] / PEAK_HBM_GBS, 4),
                 "frac_of_measured_ceiling": round(row["gbs"] / hbm_read["value"], 4) if hbm_read else None}
        else:
            e = {"ms": row["ms"], "achieved": row["tflops"], "unit": "TFLOP/s", "bound": "mfma",
                 "frac": round(row["tflops"] / PEAK_TFLOPS[row["dtype"]], 4),
                 "frac_of_measured_ceiling": round(row["tflops"] / mfma_ceiling["value"], 4) if mfma_ceiling else None}
        out[name] = e
    return out


def flatten_into(roof, fp8_block):
    """The nested entries of the roofline object once more as scalar fields of it (plain numbers under
    systematic names), for readers that keep only the scalar fields of this object."""
    def tag(shape):
        return shape.replace("x", "_")
    ceil = roof.get("measured_mfma_ceiling")
    if ceil:
        roof["measured_mfma_ceiling_tflops"] = ceil["value"]
        roof["mfma_ceiling_zero_operands_tflops"] = ceil.get("value_zero_operands")
        for shape, v in (ceil.get("by_shape") or {}).items():
            roof["mfma_ceiling_%s_tflops" % tag(shape)] = v
    if roof.get("measured_hbm_read"):
        roof["measured_hbm_read_gbs"] = roof["measured_hbm_read"]["value"]
    if roof.get("torch_mm_same_run"):
        roof["torch_mm_same_run_tflops"] = roof["torch_mm_same_run"]["value"]
    per_ghz = 256 * 4 * (2048 if roof["peak"] > 3000 else 1024) / 1e3     # TFLOP/s per GHz with an MFMA in every cycle
    clk = roof.get("shader_clock")
    if clk:
        # Measured in this run: the clock under this workload, an MFMA in every cycle of every SIMD at that clock, and
        # the share of that the launches beside the probe reached (= the share of cycles with an MFMA issued).
        roof["shader_clock_ghz_live"], roof["shader_clock_ghz_live_min_xcd"] = clk["value"], clk["min_xcd"]
        roof["shader_clock_ghz_live_max_xcd"], roof["shader_clock_probe_inside_launches"] = clk["max_xcd"], clk["probe_inside_launches"]
        roof["full_issue_at_live_clock_tflops"] = round(per_ghz * clk["value"], 1)
        roof["tflops_beside_clock_probe"] = clk["tflops_meanwhile"]
        roof["mfma_issue_share_live"] = round(clk["tflops_meanwhile"] / (per_ghz * clk["value"]), 4)
    prof = roof.get("profiled")
    if prof:
        roof["profiled_mfma_busy"], roof["profiled_shader_clock_ghz"] = prof["mfma_busy"], prof["shader_clock_ghz"]
        roof["profiled_source"] = prof["source"]
        # An MFMA in every cycle of every SIMD at the clock the profile shows for this kernel (256 CUs x 4 SIMDs x
        # 1024 flop per cycle for the 16-bit types, twice that for fp8), and the share of cycles the 0.70 / 0.60
        # target of the published peak would therefore need MFMAs to be issued in.
        roof["full_issue_at_profiled_clock_tflops"] = round(per_ghz * prof["shader_clock_ghz"], 1)
        target = 0.60 if roof["peak"] > 3000 else 0.70
        roof["mfma_busy_needed_for_target"] = round(target * roof["peak"] / roof["full_issue_at_profiled_clock_tflops"], 3)
    if fp8_block:
        r8 = fp8_block["roofline"]
        roof["fp8_value_tflops"], roof["fp8_ms_per_step"], roof["fp8_frac"] = fp8_block["value"], fp8_block["ms_per_step"], r8["frac"]
        c8 = r8.get("measured_mfma_ceiling")
        if c8:
            roof["fp8_measured_mfma_ceiling_tflops"] = c8["value"]
            roof["fp8_frac_of_measured_ceiling"] = r8.get("frac_of_measured_ceiling")
            for shape, v in (c8.get("by_shape") or {}).items():
                roof["fp8_mfma_ceiling_%s_tflops" % tag(shape)] = v
        if r8.get("torch_mm_same_run"):
            roof["fp8_torch_scaled_mm_same_run_tflops"] = r8["torch_mm_same_run"]["value"]
            roof["fp8_vs_torch_scaled_mm_same_run"] = r8.get("vs_torch_mm_same_run")
        if r8.get("shader_clock"):
            c8k = r8["shader_clock"]
            roof["fp8_shader_clock_ghz_live"] = c8k["value"]
            roof["fp8_full_issue_at_live_clock_tflops"] = round(256 * 4 * 2048 / 1e3 * c8k["value"], 1)
            roof["fp8_mfma_issue_share_live"] = round(c8k["tflops_meanwhile"] / (256 * 4 * 2048 / 1e3 * c8k["value"]), 4)
        if r8.get("profiled"):
            roof["fp8_profiled_mfma_busy"] = r8["profiled"]["mfma_busy"]
            roof["fp8_profiled_shader_clock_ghz"] = r8["profiled"]["shader_clock_ghz"]
        if fp8_block.get("cpu_baseline"):
            roof["fp8_cpu_baseline_tflops"] = fp8_block["cpu_baseline"]["value"]
    for shape, e in (roof.get("larger_shapes") or {}).items():
        for key, v in e.items():
            roof["bf16_%s_%s" % (shape, key)] = v
    for name, e in (roof.get("other_configs") or {}).items():
        unit = "tflops" if e["unit"] == "TFLOP/s" else "gbs"
        roof["cfg_%s_ms" % name] = e["ms"]
        roof["cfg_%s_%s" % (name, unit)] = e["achieved"]
        roof["cfg_%s_frac" % name] = e["frac"]
        roof["cfg_%s_frac_of_measured_ceiling" % name] = e["frac_of_measured_ceiling"]


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this library is a single-GPU GEMM; --gpus %d is not supported "
              "(run with --gpus 1)" % a.gpus, file=sys.stderr)
        raise SystemExit(2)
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    import gemm_kernels  # noqa: F401  (fails loudly when the extension is not built)

    if a.copy_calibration:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    do_settle = not a.no_settle
    if a.workload.startswith("quant_"):      # no GEMM: no CPU GEMM baseline, no second configuration
        a.no_cpu = a.no_fp8 = True
    head, keep = measure(a.workload, a.variant, a.steps, a.warmup, do_settle)
    sets, C, fp8, flops, nbytes = keep
    roof = roofline_of(head, a.workload, a.variant, sets, flops, nbytes)
    if not a.no_calibrate:
        roof["measured_mfma_ceiling"], roof["measured_hbm_read"] = calibrate(sets[0][0], sets[0][1], do_settle)
        if roof["bound"] == "mfma":
            roof["frac_of_measured_ceiling"] = round(head["tflops"] / roof["measured_mfma_ceiling"]["value"], 4)
        else:
            roof["frac_of_measured_ceiling"] = round(head["gbs"] / roof["measured_hbm_read"]["value"], 4)
    if roof["bound"] == "mfma" and not a.no_vendor:
        roof["torch_mm_same_run"] = vendor_same_run(sets, C, fp8, flops, a.steps, a.warmup, do_settle)
        if roof["torch_mm_same_run"]["value"]:
            roof["vs_torch_mm_same_run"] = round(head["tflops"] / roof["torch_mm_same_run"]["value"], 4)
    if roof["bound"] == "mfma" and not a.no_calibrate:
        roof["shader_clock"] = guarded(clock_under_load, sets, C, fp8, a.variant, flops, head["ms"], do_settle)
    if a.workload in PROFILED:
        roof["profiled"] = PROFILED[a.workload]

    head_scale = float(fp8[0]) * float(fp8[1]) if fp8 and isinstance(fp8[0], float) else 1.0
    cpu_operands = (sets[0][0][:1024].cpu(), sets[0][1].cpu(), sets[0][0].shape[0], head_scale) if not a.no_cpu else None
    del sets, C, keep
    torch.cuda.empty_cache()

    # The second configuration of the metric: fp8 e4m3 8192^3, same protocol, same K and W.
    fp8_block, fp8_cpu_operands = None, None
    if a.workload == "bf16_8192" and not a.no_fp8:
        row, keep = measure("fp8_8192", a.variant, a.steps, a.warmup, do_settle)
        sets8, C8, sc8, flops8, nbytes8 = keep
        roof8 = roofline_of(row, "fp8_8192", a.variant, sets8, flops8, nbytes8)
        if not a.no_calibrate:
            roof8["measured_mfma_ceiling"], _ = calibrate(sets8[0][0], sets8[0][1], do_settle, read=False)
            roof8["frac_of_measured_ceiling"] = round(row["tflops"] / roof8["measured_mfma_ceiling"]["value"], 4)
        if not a.no_vendor:
            roof8["torch_mm_same_run"] = vendor_same_run(sets8, C8, sc8, flops8, a.steps, a.warmup, do_settle)
            if roof8["torch_mm_same_run"]["value"]:
                roof8["vs_torch_mm_same_run"] = round(row["tflops"] / roof8["torch_mm_same_run"]["value"], 4)
        if not a.no_calibrate:
            roof8["shader_clock"] = guarded(clock_under_load, sets8, C8, sc8, a.variant, flops8, row["ms"], do_settle)
        roof8["profiled"] = PROFILED["fp8_8192"]
        fp8_block = {"value": row["tflops"], "unit": "TFLOP/s", "ms_per_step": row["ms"], "steps": a.steps,
                     "warmup": a.warmup, "settle_launches": row["settle_launches"], "settle_ms": row["settle_ms"],
                     "dtype": "e4m3", "pct_of_dense_mfma_peak": row["pct_mfma_peak"],
                     "config": {"workload": "fp8_8192: M=N=K=8192 e4m3 operands quantised from Normal(0,1) with per-tensor "
                                            "fp32 scales amax/448, fp32 accumulate, bf16 output after scale",
                                "variant": roof8["kernel"]},
                     "roofline": roof8, "cpu_baseline": None}
        if not a.no_cpu:
            fp8_cpu_operands = (sets8[0][0][:1024].cpu(), sets8[0][1].cpu(), sets8[0][0].shape[0], float(sc8[0]) * float(sc8[1]))
        del sets8, C8, keep
        torch.cuda.empty_cache()

    extras = []
    if not a.no_extras:
        names = ["bf16_8192", "fp8_8192", "mxfp8_8192", "bf16_4096", "fp16_512"] + \
                ["skinny_%d_%d_%d" % (m, n, k) for (n, k) in ((14336, 4096), (4096, 14336), (6144, 4096))
                 for m in (16, 64, 256)] + ["skinny_128_8192_4096", "skinnyfp8_16_14336_4096", "skinnymx_16_14336_4096",
                                            "quant_e4m3_8192_8192", "quant_mxfp8_8192_8192"]
        for n in names:
            if n == a.workload or (n == "fp8_8192" and fp8_block):
                continue
            steps = 60 if "8192" in n else 200
            row, keep = measure(n, "auto", steps, steps, do_settle)
            extras.append(row)
            del keep
            torch.cuda.empty_cache()
        if a.workload == "bf16_8192" and a.variant == "auto":
            for v in ("basic", "pingpong"):
                row, keep = measure("bf16_8192", v, 60, 60, do_settle)
                row["variant"] = v
                extras.append(row)
                del keep
                torch.cuda.empty_cache()

    if a.workload == "bf16_8192" and a.variant == "auto" and not a.no_extras and not a.no_vendor:
        roof["larger_shapes"] = guarded(larger_shapes, 40, do_settle)

    # Last, so that the GPU does not idle (and drop its clocks) in the middle of the measurements.
    cpu = cpu_baseline(*cpu_operands) if cpu_operands else None
    if fp8_block and fp8_cpu_operands:
        fp8_block["cpu_baseline"] = cpu_baseline(*fp8_cpu_operands, budget_s=8.0, native_budget_s=0.0)

    if fp8_block:
        # the second configuration of the metric in brief, beside the headline's roofline
        r8 = fp8_block["roofline"]
        roof["fp8_8192"] = {"value": fp8_block["value"], "unit": "TFLOP/s", "ms_per_step": fp8_block["ms_per_step"],
                            "peak": r8["peak"], "frac": r8["frac"], "traffic": r8["traffic"],
                            "measured_mfma_ceiling": (r8.get("measured_mfma_ceiling") or {}).get("value"),
                            "mfma_ceiling_by_shape": (r8.get("measured_mfma_ceiling") or {}).get("by_shape"),
                            "frac_of_measured_ceiling": r8.get("frac_of_measured_ceiling"),
                            "torch_mm_same_run": (r8.get("torch_mm_same_run") or {}).get("value"),
                            "vs_torch_mm_same_run": r8.get("vs_torch_mm_same_run"),
                            "profiled": r8.get("profiled"),
                            "cpu_baseline_value": (fp8_block["cpu_baseline"] or {}).get("value"),
                            "see": "the top-level \"fp8\" object of this line"}
    if extras:
        roof["other_configs"] = other_configs(extras, roof.get("measured_mfma_ceiling"), roof.get("measured_hbm_read"))
    flatten_into(roof, fp8_block)
    out = {
        "metric": METRIC, "value": head["tflops"], "unit": "TFLOP/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "settle_launches": head["settle_launches"], "settle_ms": head["settle_ms"],
        "ms_per_step": head["ms"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": "%s: M=%d N=%d K=%d, A (M,K) and B (N,K) K-contiguous, fp32 accumulate"
                               % (a.workload, head["M"], head["N"], head["K"]),
                   "variant": roof["kernel"], "parallelism": "single GPU",
                   "protocol": ("no settle; " if a.no_settle else "settle (>=%d ms, 3 batches within 1%%) precedes " % SETTLE_MIN_MS) +
                               "W warm-up + K timed launches, HIP events on the launch stream"},
        "pct_of_dense_mfma_peak": head["pct_mfma_peak"],
        "roofline": roof, "cpu_baseline": cpu, "extras": extras, "fp8": fp8_block,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
