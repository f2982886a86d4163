"""bench.py's JSON assembly without a GPU: the other configurations of the baseline and the
yardsticks must appear inside `roofline` both nested and as scalar fields under systematic names
(a reader that keeps only the scalar fields of that object still sees every figure)."""
import importlib.util
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("_bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def row(name, ms, tflops, gbs, dtype="bf16", **extra):
    r = {"workload": name, "ms": ms, "tflops": tflops, "gbs": gbs, "dtype": dtype}
    r.update(extra)
    return r


def test_other_configs_cover_the_eleven_configurations_and_nothing_else():
    b = load_bench()
    names = ["bf16_4096", "fp16_512"] + ["skinny_%d_%d_%d" % (m, n, k) for (n, k) in ((14336, 4096), (4096, 14336), (6144, 4096))
                                         for m in (16, 64, 256)]
    extras = [row(n, 0.05, 1000.0, 4000.0, "f16" if n == "fp16_512" else "bf16") for n in names]
    extras += [row("skinny_128_8192_4096", 0.02, 1.0, 3000.0), row("mxfp8_8192", 0.3, 3000.0, 1.0, "e4m3"),
               row("bf16_8192", 0.7, 1500.0, 500.0, variant="pingpong")]
    out = b.other_configs(extras, {"value": 2000.0}, {"value": 6800.0})
    assert sorted(out) == sorted(names)
    assert out["bf16_4096"] == {"ms": 0.05, "achieved": 1000.0, "unit": "TFLOP/s", "bound": "mfma", "frac": 0.4,
                                "frac_of_measured_ceiling": 0.5}
    assert out["skinny_16_14336_4096"] == {"ms": 0.05, "achieved": 4000.0, "unit": "GB/s", "bound": "hbm", "frac": 0.5,
                                           "frac_of_measured_ceiling": round(4000.0 / 6800.0, 4)}
    assert b.other_configs(extras, None, None)["fp16_512"]["frac_of_measured_ceiling"] is None


def test_roofline_carries_every_yardstick_as_a_scalar_field():
    b = load_bench()
    roof = {"bound": "mfma", "peak": 2500.0,
            "measured_mfma_ceiling": {"value": 2000.0, "value_zero_operands": 2400.0, "by_shape": {"16x16x32": 2000.0, "32x32x16": 1800.0}},
            "measured_hbm_read": {"value": 6800.0}, "torch_mm_same_run": {"value": 1660.0}, "profiled": b.PROFILED["bf16_8192"],
            "shader_clock": {"value": 1.7, "min_xcd": 1.66, "max_xcd": 1.73, "probe_inside_launches": True, "tflops_meanwhile": 1600.0},
            "larger_shapes": {"8192_8192_16384": {"ms": 1.42, "tflops": 1550.0, "frac": 0.62, "torch_mm_tflops": 1540.0, "vs_torch_mm": 1.0065}},
            "other_configs": b.other_configs([row("bf16_4096", 0.09, 1500.0, 1.0), row("skinny_64_6144_4096", 0.017, 1.0, 3000.0)],
                                             {"value": 2000.0}, {"value": 6800.0})}
    fp8 = {"value": 3200.0, "ms_per_step": 0.34, "cpu_baseline": {"value": 1.3},
           "roofline": {"frac": 0.64, "frac_of_measured_ceiling": 0.73, "vs_torch_mm_same_run": 0.99,
                        "measured_mfma_ceiling": {"value": 4400.0, "by_shape": {"16x16x128": 4400.0, "32x32x64": 4100.0}},
                        "torch_mm_same_run": {"value": 3230.0}, "profiled": b.PROFILED["fp8_8192"]}}
    b.flatten_into(roof, fp8)
    flat = {k: v for k, v in roof.items() if not isinstance(v, (dict, list))}
    for key, want in [("measured_mfma_ceiling_tflops", 2000.0), ("mfma_ceiling_16_16_32_tflops", 2000.0),
                      ("mfma_ceiling_32_32_16_tflops", 1800.0), ("mfma_ceiling_zero_operands_tflops", 2400.0),
                      ("measured_hbm_read_gbs", 6800.0), ("torch_mm_same_run_tflops", 1660.0),
                      ("profiled_mfma_busy", b.PROFILED["bf16_8192"]["mfma_busy"]),
                      ("fp8_value_tflops", 3200.0), ("fp8_frac", 0.64), ("fp8_mfma_ceiling_32_32_64_tflops", 4100.0),
                      ("fp8_torch_scaled_mm_same_run_tflops", 3230.0), ("fp8_vs_torch_scaled_mm_same_run", 0.99),
                      ("fp8_cpu_baseline_tflops", 1.3), ("cfg_bf16_4096_tflops", 1500.0), ("cfg_bf16_4096_frac", 0.6),
                      ("cfg_skinny_64_6144_4096_gbs", 3000.0),
                      ("shader_clock_ghz_live", 1.7), ("shader_clock_ghz_live_min_xcd", 1.66), ("shader_clock_probe_inside_launches", True),
                      ("full_issue_at_live_clock_tflops", round(1048.576 * 1.7, 1)), ("mfma_issue_share_live", round(1600.0 / (1048.576 * 1.7), 4)),
                      ("bf16_8192_8192_16384_tflops", 1550.0), ("bf16_8192_8192_16384_torch_mm_tflops", 1540.0),
                      ("bf16_8192_8192_16384_vs_torch_mm", 1.0065), ("cfg_skinny_64_6144_4096_frac", 0.375)]:
        assert flat[key] == want, key
    # an MFMA in every cycle at the profiled clock, and the issue share the 0.70 target would need at that clock
    assert flat["full_issue_at_profiled_clock_tflops"] == round(1048.576 * b.PROFILED["bf16_8192"]["shader_clock_ghz"], 1)
    # (above 1 when the target is out of reach at that clock whatever the schedule)
    assert 0.9 < flat["mfma_busy_needed_for_target"] < 1.1
    json.dumps(roof)                                     # everything stays serialisable
    assert all(len(v) <= 120 for v in flat.values() if isinstance(v, str))    # survives a reader that cuts long strings


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True)
    assert proc.returncode == 2 and "single-GPU" in proc.stderr and proc.stdout.strip() == ""
