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
    d = json.loads(r.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["dtype"] == "f32" and d["vs_baseline"] is None
    assert d["check"]["ok"] and d["check"]["layers_checked"] == 1
    assert d["value"] > 0 and d["ms_per_step"] > 0
    rl = d["roofline"]
    assert rl["bound"] in ("hbm", "valu_fp32") and 0 < rl["frac"] < 1 and rl["peak"] in (8000.0, 157.3)
    cpu = d["cpu_baseline"]
    assert cpu["value"] > 0 and cpu["cores"] >= 1 and cpu["kind"] == "port"
    assert cpu["gpu_vs_this_cpu_output_max_rel_err"] <= 1e-4  # the reference-layout decode agrees with the device
    ctx = d["context"]
    assert ctx["vendor_dense_fp32_ms_per_step"] > 0 and ctx["vendor_csr_im2col_ms_per_step"] > 0, ctx


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr
