"""CPU checks of bench.py's output contract: the result line (last line of stdout) must stay short enough for a
harness that keeps only the tail of stdout, whatever the number of per-layer rows measured before it."""
import json
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _fake_row(layer, op):
    par = {"vs": "fp64 CPU oracle", "subset": "images [0, 1, 2, 3, 63] of 64, all channels", "checked": 4014080, "tol_rel": 1e-4,
           "tol_abs": 1.23e-05, "max_err_ratio": 0.4123, "max_err_ratio_at_abs_1e-5": 27.5123, "max_abs_err": 1.23e-05,
           "rms_expected": 301.1234, "samePercentRelative_1e-4": 0.999876, "samePercentRelative_1e-5": 0.987654, "ok": True,
           "bit_reproducible_run_to_run": True}
    roof = {"bound": "mfma", "achieved": 133.123, "peak": 157.3, "unit": "TFLOP/s", "kernel_ms": 0.11123, "traffic": 134506496,
            "frac": 0.8463, "flop_per_byte": 143.87, "mfma_frac": 0.8463, "hbm_frac": 0.1157, "touched_MB": 38.6,
            "hbm_frac_touched": 0.3612, "note": "x" * 120, "executed_mfma_frac": 0.3761}
    return {"layer": layer, "op": op, "ms_per_step": 0.11812, "event_ms_per_step": 0.11799, "tflops": 125.312, "gflop": 14.798,
            "algorithmic_MB": 102.91, "GridZ": 128, "roofline": roof, "parity": par}


def _fake_head():
    row = _fake_row("c3a", "fwd")
    cpu = {"value": 0.423123, "unit": "TFLOP/s", "cores": 16, "kind": "port", "sample": "c3a fwd, 64 of 64 images x 3 repeats, 12.9 s; " + "y" * 80}
    return {"metric": "conv fwd/bwd TFLOP/s (fp32) + % of MI355X fp32 MFMA peak, 1 GPU", "value": 125.3, "unit": "TFLOP/s", "n_gpus": 1,
            "steps": 50, "warmup": 10, "ms_per_step": 0.118, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
            "data": "synthetic", "config": {"workload": "w" * 160, "layer": "c3a", "op": "fwd", "gflop_per_step": 14.798,
                                            "algorithmic_MB_per_step": 102.91, "frac_of_fp32_mfma_peak": 0.7966, "tolerance": "t" * 70,
                                            "clock_ramp_ms": 40.0, "device": {"name": "AMD Instinct MI355X", "cus": 256, "clock_ghz": 2.4,
                                                                              "fp32_mfma_peak_from_device_tflops": 157.3}},
            "roofline": row["roofline"], "parity": bench.compact_parity(row["parity"]),
            "winograd": {"value": 220.1, "unit": "TFLOP/s (direct-conv-equivalent)", "ms_per_step": 0.0671, "kernel_ms": 0.061,
                         "kernel_tflops": 242.6, "direct_equivalent_over_fp32_mfma_peak": 1.54, "executed_flop_frac_of_fp32_mfma_peak": 0.68,
                         "parity": bench.compact_parity(row["parity"])},
            "parity_summary": {"rows": 51, "rows_ok": 51, "worst_max_err_ratio": 0.41, "worst_max_err_ratio_at_abs_1e-5": 27.5,
                               "least_samePercentRelative_1e-4": 0.9983},
            "cpu_baseline": cpu, "cpu_baseline_dx": cpu, "cpu_baseline_dw": cpu, "cpu_baseline_c1_1core": cpu}


def test_result_line_with_every_row_stays_under_the_limit():
    rows = [_fake_row(layer, op) for layer in sorted(bench.LAYERS) for op in bench.layer_ops(layer)]
    assert len(rows) >= 51
    line = bench.result_line(_fake_head(), rows)
    assert "\n" not in line
    assert len(line.encode()) <= bench.FINAL_LINE_LIMIT <= 4096
    got = json.loads(line)
    for key in ("metric", "value", "unit", "ms_per_step", "roofline", "cpu_baseline", "parity_summary", "layers_min", "config"):
        assert key in got, key
    assert len(got["layers_min"]) == len(rows)
    assert got["layers_min"]["c5a/dw"] == [0.846, 0.1181, 1]
    assert got["roofline"]["frac"] == 0.8463 and got["cpu_baseline"]["cores"] == 16


def test_result_line_sheds_optional_parts_before_it_overflows():
    rows = [_fake_row("c3a", "op%04d" % i) for i in range(400)]   # far more rows than the configs have
    line = bench.result_line(_fake_head(), rows)
    assert len(line.encode()) <= bench.FINAL_LINE_LIMIT
    got = json.loads(line)
    assert "layers_min" not in got
    for key in ("metric", "value", "ms_per_step", "roofline", "cpu_baseline", "parity_summary"):
        assert key in got, key


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr
