"""The shape-sweep harness (cute-examples_amd/gemm_bench.py, the counterpart of the reference's
kernels/tests/gemm_bench.py) runs end to end on its two smallest shapes: both implementations are
timed with both protocols, they agree on the same operands, and the summary table and the JSON file
come out."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_gemm_bench_two_smallest_shapes(tmp_path):
    out = tmp_path / "sweep.json"
    env = dict(os.environ, PYTHONPATH=os.path.join(ROOT, "cute-examples_amd"))
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "cute-examples_amd", "gemm_bench.py"), "--runs", "3",
                           "--shapes", "1024x1024,2048x2048,512x1536x1024", "--out", str(out)],
                          capture_output=True, text=True, env=env, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "PERFORMANCE SUMMARY" in proc.stdout and "1024x1024" in proc.stdout and "2048x2048" in proc.stdout
    assert "512x1536x1024" in proc.stdout       # a shape with M != N, which the reference's notation cannot name
    data = json.loads(out.read_text())
    assert data["comparator"].startswith("torch.mm") and len(data["rows"]) == 3
    assert (data["rows"][2]["M"], data["rows"][2]["N"], data["rows"][2]["K"]) == (512, 1536, 1024)
    for row in data["rows"]:
        assert row["rel_diff"] <= 1e-2, row                     # ours and torch.mm on the same operands
        for key in ("ours_wall_ms", "blas_wall_ms", "ours_event_ms", "blas_event_ms"):
            assert 0.0 < row[key] < 1e3, (key, row)
        assert row["ours_tflops"] > 1.0 and row["blas_tflops"] > 1.0


def test_calibration_kernels_run_and_report_plausible_ceilings(abi):
    """mi355_calibrate_mfma / mi355_calibrate_read through the C ABI: they launch, write their sink,
    and the rates they give are those of a GPU (above 100 TFLOP/s and 1 TB/s) and below the published
    peaks.  Argument errors come back before any launch."""
    import ctypes
    import torch
    from tests import abi_ctypes as ac

    sink = torch.zeros(abi.mi355_calibrate_sink_bytes(), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    flops = ctypes.c_double()
    assert abi.mi355_calibrate_mfma(ac.BF16, None, 4096, None, 4096, 10, sink.data_ptr(), ctypes.byref(flops), stream) == ac.ERR_NULL
    assert abi.mi355_calibrate_mfma_shape(ac.BF16, 2, sink.data_ptr(), 4096, sink.data_ptr(), 4096, 10, sink.data_ptr(),
                                          ctypes.byref(flops), stream) == ac.ERR_VARIANT
    for code, dt, peak in ((ac.BF16, torch.bfloat16, 2500.0), (ac.F16, torch.float16, 2500.0), (ac.E4M3, torch.float8_e4m3fn, 5000.0)):
        A = torch.randn(1024, 1024, device="cuda").to(dt)
        B = torch.randn(1024, 1024, device="cuda").to(dt)
        nbytes = A.numel() * A.element_size()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        flop_counts = []
        for wide in (None, 0, 1):      # the plain entry point, then both MFMA shapes by name
            for timed in (False, True):
                e0.record()
                if wide is None:
                    rc = abi.mi355_calibrate_mfma(code, A.data_ptr(), nbytes, B.data_ptr(), nbytes, 2000, sink.data_ptr(),
                                                  ctypes.byref(flops), stream)
                else:
                    rc = abi.mi355_calibrate_mfma_shape(code, wide, A.data_ptr(), nbytes, B.data_ptr(), nbytes, 2000,
                                                        sink.data_ptr(), ctypes.byref(flops), stream)
                e1.record()
                assert rc == ac.OK
                torch.cuda.synchronize()
            tflops = flops.value / e0.elapsed_time(e1) / 1e9
            assert 100.0 < tflops <= 1.02 * peak, (code, wide, tflops)
            flop_counts.append(flops.value)
        # 2000 passes over 128 x 128 outputs per wave: the narrow shapes span twice the K of the wide ones
        assert flop_counts[0] == flop_counts[1] == 2 * flop_counts[2]
    src = torch.empty(1 << 28, dtype=torch.uint8, device="cuda")
    src.view(torch.int32).random_()
    for timed in (False, True):
        e0.record()
        assert abi.mi355_calibrate_read(src.data_ptr(), src.numel(), sink.data_ptr(), stream) == ac.OK
        e1.record()
        torch.cuda.synchronize()
    gbs = src.numel() / e0.elapsed_time(e1) / 1e6
    assert 1000.0 < gbs, gbs


def test_clock_probe_reads_a_plausible_shader_clock_beside_a_gemm(abi):
    """mi355_clock_probe on a second stream while GEMMs run on the first: every wave's cycle and 10 ns counters
    rise from sample to sample, the clock they give lies between 0.5 and 2.6 GHz, the waves report XCDs 0..7,
    and the GEMM's result is what it is without the probe.  Argument errors come back before any launch."""
    import torch
    from tests import abi_ctypes as ac
    import gemm_kernels

    assert abi.mi355_clock_probe_bytes(0, 10) == 0 and abi.mi355_clock_probe_bytes(8, 1) == 0
    assert abi.mi355_clock_probe_bytes(8, 4097) == 0 and abi.mi355_clock_probe_bytes(1025, 10) == 0
    waves, samples, pause = 16, 40, 4
    assert abi.mi355_clock_probe_bytes(waves, samples) == waves * (samples + 1) * 16
    out = torch.zeros((waves, 2, samples + 1), dtype=torch.int64, device="cuda")
    assert abi.mi355_clock_probe(waves, samples, pause, None, None) == ac.ERR_NULL
    assert abi.mi355_clock_probe(waves, samples, 0, out.data_ptr(), None) == ac.ERR_SHAPE
    assert abi.mi355_clock_probe(waves, 4096, 17, out.data_ptr(), None) == ac.ERR_SHAPE
    assert abi.mi355_clock_probe(waves, samples, pause, out.data_ptr() + 4, None) == ac.ERR_ALIGN
    A = torch.randn(4096, 4096, device="cuda").to(torch.bfloat16)
    B = torch.randn(4096, 4096, device="cuda").to(torch.bfloat16)
    alone = gemm_kernels.gemm_tn(A, B, torch.empty(4096, 4096, dtype=torch.bfloat16, device="cuda"))
    torch.cuda.synchronize()
    C = torch.empty_like(alone)
    side = torch.cuda.Stream()
    started = torch.cuda.Event()
    gemm_kernels.gemm_tn(A, B, C)
    started.record()
    for _ in range(12):
        gemm_kernels.gemm_tn(A, B, C)
    side.wait_event(started)
    assert abi.mi355_clock_probe(waves, samples, pause, out.data_ptr(), side.cuda_stream) == ac.OK
    torch.cuda.synchronize()
    assert torch.equal(C, alone)
    got = out.cpu()
    assert set(got[:, 0, 0].tolist()) <= set(range(8)) and (got[:, 1, 0] == 0).all()
    cycles, ticks = got[:, 0, 1:], got[:, 1, 1:]
    assert (cycles[:, 1:] > cycles[:, :-1]).all() and (ticks[:, 1:] > ticks[:, :-1]).all()
    ghz = (cycles[:, -1] - cycles[:, 0]).double() / (ticks[:, -1] - ticks[:, 0]).double() / 10.0
    assert (ghz > 0.5).all() and (ghz < 2.6).all(), ghz
