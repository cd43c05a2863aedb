"""bench.py end to end on a small workload: the JSON line's contract fields, the vendor baselines beside it (dense
MIOpen convolution and CSR x im2col through torch, the counterparts of Tetris/cuda_utils.cc:6-132 and
Tetris/cusparse_test.cc:147-173) and the refusal of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.gpu
def test_bench_line_with_vendor_baselines():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--suite", "single", "--batch", "1", "--steps", "3",
                        "--warmup", "2", "--layer-repeat", "3", "--no-suites", "--dense-baseline", "--csr-baseline"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = r.stdout.strip().splitlines()[-1]
    assert len(line) < 4096, len(line)
    d = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["dtype"] == "f32" and d["vs_baseline"] is None
    assert d["check"]["ok"] and d["check"]["all_workloads_ok"]
    assert d["value"] > 0 and d["ms_per_step"] > 0
    rl = d["roofline"]
    assert rl["bound"] in ("hbm", "mfma") and 0 < rl["frac"] < 1 and rl["peak"] in (8000.0, 157.3)
    cpu = d["cpu_baseline"]
    assert cpu["value"] > 0 and cpu["cores"] >= 1 and cpu["kind"] == "port"
    full = json.load(open(os.path.join(ROOT, d["details"])))  # the side file: per-layer tables and everything else
    assert full["cpu_baseline"]["gpu_vs_this_cpu_output_max_rel_err"] <= 1e-4  # reference-layout decode == device
    assert len(full["layers"]) == 1 and full["layers"][0]["us"] > 0 and full["check"]["layers_checked"] == 1
    ctx = d["context"]
    assert ctx["vendor_dense_fp32_ms_per_step"] > 0 and ctx["vendor_csr_im2col_ms_per_step"] > 0, ctx


@pytest.mark.gpu
def test_default_command_prints_one_short_line():
    """The command the round's end runs (every workload of the metric, the chained network pass and the CPU baseline
    on): stdout's last line is one JSON object under 4 KB that carries `roofline`, `cpu_baseline` and `check` whole --
    a reader that keeps only the tail of stdout still gets all of it."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "5", "--warmup", "2"],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = r.stdout.strip().splitlines()
    assert len(lines) == 1, [ln[:80] for ln in lines]
    line = lines[-1]
    assert len(line) < 2000, len(line)  # a reader that keeps the last 2000 characters of stdout holds the whole line
    d = json.loads(line)
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["config"]["suite"] == "vgg19"
    assert d["config"]["batch"] == 16 and d["check"]["ok"] and d["check"]["all_workloads_ok"], d["check"]
    rl, cpu = d["roofline"], d["cpu_baseline"]
    assert rl["bound"] in ("hbm", "mfma") and 0 < rl["frac"] < 1 and abs(rl["frac"] - rl["achieved"] / rl["peak"]) < 1e-3
    assert cpu["value"] > 0 and cpu["cores"] >= 1 and cpu["kind"] in ("port", "reference") and cpu["sample"]
    assert len(d["suites"]) == 7 and all(row[-1] is True for row in d["suites"]), d["suites"]
    assert d["chain"]["check_ok"] is True
    full = json.load(open(os.path.join(ROOT, d["details"])))
    assert len(full["layers"]) == 16 and sum(len(s["layers"]) for s in full["suites"]) == 190


def test_summary_line_stays_short():
    """summary_line() on a record of the default run's shape (seven other workloads, chain, CPU baseline): under 4 KB,
    the contract's keys present, no list of per-layer rows in it."""
    sys.path.insert(0, ROOT)
    import bench

    suites = [{"suite": s, "batch": b, "ms_per_step_device": 12.3456, "bound": "valu_fp32", "roofline_frac": 0.1234,
               "min_layer_roofline_frac": 0.0432, "traffic": 1049550000.0, "algorithmic_bytes_per_launch": 689550000.0,
               "check": {"ok": True}, "layers": [{"layer": "x" * 20, "us": 1.0}] * 75} for s, b in bench.OTHER_WORKLOADS]
    full = {"metric": "m", "value": 298123.4, "unit": "GFLOP/s", "n_gpus": 1, "steps": 20, "warmup": 5,
            "settle_ms": 30.0, "ms_per_step": 2.0912, "ms_per_step_device": 2.0907, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": "w" * 100, "suite": "vgg19", "batch": 16, "layers": 16, "tensor_seed": "t" * 200},
            "check": {"ok": True, "layers_checked": 16, "max_rel_err": 3.8123456789e-05, "tolerance": 1e-4,
                      "failed_layers": [], "all_workloads_ok": True, "failed_workloads": [], "against": "a" * 100},
            "roofline": {"bound": "mfma", "note": "n" * 100, "achieved": 30.712, "peak": 157.3, "unit": "TFLOP/s",
                         "frac": 0.1953, "kernel": "spconv2d_kernel", "launches_per_step": 16, "avg_launch_us": 130.67,
                         "algorithmic_flops_per_launch": 4016738304.0, "algorithmic_bytes_per_launch": 101912345.5,
                         "traffic": 161600000.0, "traffic_source": {"file": "f" * 100}},
            "cpu_baseline": {"value": 81.65, "unit": "GFLOP/s", "cores": 16, "kind": "port", "sample": "s" * 220,
                             "dense_host_conv2d": {"sample": "d" * 100}},
            "min_layer_roofline_frac": 0.0712, "layers": [{"layer": "y" * 20}] * 16,
            "context": {"measured_copy_gbs": 5301.2, "measured_fma_tflops": 71.61, "roofline_frac_of_measured": 0.4288,
                        "peaks_note": "p" * 300},
            "suites": suites, "chain": {"ms_per_pass": 2.0845, "check": {"ok": True}, "workload": "c" * 300}}
    line = json.dumps(bench.summary_line(full, os.path.join(ROOT, "gpurun_out", "bench_layers.json")))
    assert len(line) < 2400, len(line)
    d = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "check"):
        assert key in d, key
    assert "layers" not in d and all(not isinstance(v, dict) for row in d["suites"] for v in row)
    assert d["details"] == os.path.join("gpurun_out", "bench_layers.json")


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr
