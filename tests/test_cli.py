"""The per-layer command-line drivers (counterparts of the reference's spconv2d_test.o / spf_test.o mains,
Tetris/spconv2d.cc:369-450 and Tetris/spf.cc:95-176): stdout lines in the reference's format, and the tensors
they compute checked against the CPU oracle."""
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import ROOT
from helpers import max_rel_err, sparse_filter

BIN = os.path.join(ROOT, "tetris-artifact-evalution_amd", "bin")


def write_weight_file(path, w, H, W, pad, stride):
    K, C, ks, _ = w.shape
    with open(path, "w") as f:  # header order of Tetris/tensor_utils.cc:66
        f.write("%d %d %d %d %d %d %d 1\n" % (H, W, C, K, ks, pad, stride))
        f.write(" ".join(repr(float(v)) for v in w.reshape(-1)) + "\n")


ALL_CLIS = ["spconv2d_test", "para_test", "spf_test", "bank_sr_test", "filter_gr_test", "wo_bank_sr_test",
            "wi_bank_sr_test", "baseline_test"]  # evalution/script/build_all.sh:14, build_ablation.sh:12-18


@pytest.mark.parametrize("exe", ALL_CLIS)
def test_cli_is_built_and_explains_itself(exe):
    p = subprocess.run([os.path.join(BIN, exe)], capture_output=True, text=True, timeout=60)
    assert p.returncode == 2 and "usage" in p.stderr
    assert p.stdout.startswith("args : 1 ")  # the reference's first line


@pytest.mark.gpu
@pytest.mark.parametrize("exe,shape", [
    ("spconv2d_test", (3, 24, 20, 20, 40, 3, 1, 1)),
    ("spconv2d_test", (2, 16, 15, 15, 33, 1, 2, 0)),
    ("spf_test", (2, 24, 20, 20, 40, 3, 1, 1)),
    ("bank_sr_test", (2, 24, 20, 20, 40, 3, 1, 1)),
    ("filter_gr_test", (2, 24, 20, 20, 40, 3, 1, 1)),
    ("wo_bank_sr_test", (3, 20, 14, 14, 70, 3, 2, 1)),
    ("baseline_test", (2, 24, 20, 20, 40, 3, 1, 1)),
    ("baseline_test", (1, 40, 9, 9, 33, 1, 1, 0)),
    ("para_test", (2, 24, 20, 20, 40, 3, 1, 1)),
])
def test_cli_output_and_tensors(oracle, tmp_path, exe, shape):
    N, C, H, W, K, ks, stride, pad = shape
    rng = np.random.default_rng(3)
    w = sparse_filter(rng, K, C, ks, 0.8)
    wf, dump = str(tmp_path / "layer.txt"), str(tmp_path / "dump.bin")
    write_weight_file(wf, w, H, W, pad, stride)
    p = subprocess.run([os.path.join(BIN, exe), wf, str(N), "--seed", "7", "--dump", dump], capture_output=True,
                       text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    out = p.stdout
    nnz = int((w != 0).sum())
    m = re.search(r"\[Config\] sparsity = ([0-9.e-]+), nnz = (\d+), batch_size = (\d+), img_h = (\d+), img_w = (\d+), "
                  r"in_channel = (\d+), out_channel = (\d+), kernel_size = (\d+), padding = (\d+), stride = (\d+)", out)
    assert m and [int(v) for v in m.groups()[1:]] == [nnz, N, H, W, C, K, ks, pad, stride]
    assert abs(float(m.group(1)) - (1.0 - nnz / w.size)) < 1e-5
    if exe in ("spconv2d_test", "para_test", "baseline_test"):  # the lines evalution/conv2d_timing.py:51-79 parses
        who = "Baseline" if exe == "baseline_test" else "Spconv2d"  # Tetris/baseline.cc:82-83, spconv2d.cc:357-358
        t = re.search(r"Time of %s :([0-9.e-]+)ms" % who, out)
        fl = re.search(r"FLOPS of %s :([0-9.e+-]+)T" % who, out)
        assert t and fl and float(t.group(1)) > 0
        oh, ow = (H + 2 * pad - ks) // stride + 1, (W + 2 * pad - ks) // stride + 1
        want = oh * ow * N * K * C * ks * ks * 2 * 1000 / float(t.group(1)) / 1024 ** 4
        assert abs(float(fl.group(1)) - want) <= 2e-2 * want  # both numbers are printed with six digits
    else:
        assert re.search(r"Time of Ablation :([0-9.e-]+)ms", out)
    oh, ow = (H + 2 * pad - ks) // stride + 1, (W + 2 * pad - ks) // stride + 1
    raw = np.fromfile(dump, dtype=np.float32)
    assert raw.size == N * C * H * W + N * K * oh * ow
    x = raw[: N * C * H * W].reshape(N, C, H, W)
    y = raw[N * C * H * W:].reshape(N, K, oh, ow)
    assert -1.0 <= x.min() and x.max() < 1.0 and x.std() > 0.5  # uniform on [-1, 1)
    assert max_rel_err(y, oracle.host_conv2d(x, w, stride, pad, threads=4)) <= 1e-4


@pytest.mark.gpu
def test_cli_check_option_prints_the_reference_verdict(tmp_path):
    rng = np.random.default_rng(4)
    w = sparse_filter(rng, 24, 16, 3, 0.8)
    wf = str(tmp_path / "layer.txt")
    write_weight_file(wf, w, 12, 12, 1, 1)
    p = subprocess.run([os.path.join(BIN, "spconv2d_test"), wf, "2", "--check"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stderr
    lines = p.stdout.splitlines()
    assert lines.index("HostConv2d begin") < lines.index("HostConv2d end") < lines.index("Sparse Pass.")
    assert "Sparse Error." not in p.stdout


@pytest.mark.gpu
def test_cli_missing_file_behaves_like_the_reference():
    p = subprocess.run([os.path.join(BIN, "spconv2d_test"), "/nonexistent/layer", "1"], capture_output=True, text=True,
                       timeout=60)
    assert p.returncode == 1 and "Open file error." in p.stdout  # Tetris/tensor_utils.cc:61-64


CANNED = """args : 3 ./spconv2d_test.o layer 4

GPU Device 0: "AMD Instinct MI355X" (gfx950, 256 compute units)

[Config] sparsity = 0.899902, nnz = 7380, batch_size = 4, img_h = 56, img_w = 56, in_channel = 64, out_channel = 128, kernel_size = 3, padding = 1, stride = 1
Time of Spconv2d :0.012345ms
FLOPS of Spconv2d :136.5T
"""


def test_timing_driver_parses_and_writes_the_reference_csv(tmp_path):
    # host logic of the per-folder timing loop (counterpart of evalution/conv2d_timing.py), with a stand-in binary
    from tetris_amd import timing

    cfg, ms, tf = timing.parse_output(CANNED)
    assert (ms, tf) == (0.012345, 136.5) and cfg["kernel_size"] == "3" and cfg["nnz"] == "7380" and cfg["stride"] == "1"
    assert timing.parse_output("nothing useful\n") == ({}, -1.0, -1.0)
    folder = tmp_path / "net-90-acc-1.0"
    folder.mkdir()
    rng = np.random.default_rng(0)
    for i in range(3):
        w = sparse_filter(rng, 8, 4, 3, 0.5)
        timing.write_weight_file(str(folder / ("conv_%d" % i)), w, 9, 9, 1, 1)
    import tetris_amd as T
    hdr, w2 = T.ReadConfigAndDataFromFile(str(folder / "conv_2"))[:2]
    assert np.array_equal(w2.reshape(w.shape), w)  # nine significant digits round-trip fp32
    fake = tmp_path / "fake_bin"
    fake.write_text("#!/bin/sh\ncat <<'EOT'\n" + CANNED + "EOT\n")
    fake.chmod(0o755)
    csv, rows = timing.time_folder(str(fake), str(folder), 4, str(tmp_path / "logs"))
    assert os.path.basename(csv) == "net-90-acc-1.0_batch_4.csv"
    assert open(csv).read().splitlines() == [",op_name,spconv2d"] + ["%d,conv_%d,%.5f" % (i, i, 0.012345) for i in range(3)]
    log = open(str(tmp_path / "logs" / "net-90-acc-1.0_batch_4.log")).read()
    assert log.count("# Run[") == 3 and "spconv2d: time = 0.0123" in log
    bad = tmp_path / "bad_bin"
    bad.write_text("#!/bin/sh\nexit 3\n")
    bad.chmod(0o755)
    with pytest.raises(RuntimeError):
        timing.time_layer(str(bad), str(folder / "conv_0"), 1)


def test_ablation_driver_writes_the_reference_csv(tmp_path):
    # host logic of the ladder loop (counterpart of evalution/ablation_timing.py), with stand-in binaries
    from tetris_amd import timing

    folder = tmp_path / "vgg19-90-acc"
    folder.mkdir()
    rng = np.random.default_rng(1)
    for i in range(2):
        timing.write_weight_file(str(folder / ("conv_%d" % i)), sparse_filter(rng, 8, 4, 3, 0.5), 9, 9, 1, 1)
    bins = tmp_path / "bin"
    bins.mkdir()
    lines = {"baseline_test": "Time of Baseline :0.5ms\nFLOPS of Baseline :1.5T\n", "spf_test": "Time of Ablation :0.4ms\n",
             "bank_sr_test": "Time of Ablation :0.3ms\n", "filter_gr_test": "Time of Ablation :0.25ms\n",
             "para_test": "Time of Spconv2d :0.125ms\nFLOPS of Spconv2d :6T\n"}
    for name, text in lines.items():
        f = bins / name
        f.write_text("#!/bin/sh\ncat <<'EOT'\n[Config] sparsity = 0.5, nnz = 144, batch_size = 4, kernel_size = 3\n" + text + "EOT\n")
        f.chmod(0o755)
    csv, rows = timing.ablation_folder(str(bins), str(folder), 4, str(tmp_path / "logs"))
    assert os.path.basename(csv) == "ablation_a.csv"
    assert open(csv).read().splitlines() == [",op_name,Baseline,SPF,Bank-SR,Filter-GR,Para",
                                             "0,conv_0,0.50000,0.40000,0.30000,0.25000,0.12500",
                                             "1,conv_1,0.50000,0.40000,0.30000,0.25000,0.12500"]
    log = open(str(tmp_path / "logs" / "ablation_a.log")).read()
    assert log.count("# Run[") == 2 and "Bank-SR: time = 0.30000ms" in log and "'kernel_size': '3'" in log
    (bins / "para_test").unlink()
    with pytest.raises(SystemExit):
        timing.main(["--ablation", "--weights", str(folder), "--bin-dir", str(bins), "--log-dir", str(tmp_path / "l2")])


@pytest.mark.gpu
def test_ablation_driver_on_the_real_binaries(tmp_path):
    from tetris_amd import timing

    folder = tmp_path / "net-80"
    folder.mkdir()
    rng = np.random.default_rng(2)
    timing.write_weight_file(str(folder / "a_3x3"), sparse_filter(rng, 64, 32, 3, 0.8), 28, 28, 1, 1)
    timing.write_weight_file(str(folder / "b_1x1"), sparse_filter(rng, 48, 64, 1, 0.8), 14, 14, 0, 1)
    csv, rows = timing.ablation_folder(BIN, str(folder), 4, str(tmp_path / "logs"))
    assert [op for op, _ in rows] == ["a_3x3", "b_1x1"]
    assert all(len(t) == 5 and all(0 < v < 50 for v in t) for _, t in rows)
    # every rung computes the convolution: the reference's own check, through each binary
    for exe in [b for b, _ in timing.LADDER]:
        p = subprocess.run([os.path.join(BIN, exe), str(folder / "a_3x3"), "2", "--check"], capture_output=True, text=True,
                           timeout=120)
        assert p.returncode == 0 and "Sparse Pass." in p.stdout, (exe, p.stdout[-500:], p.stderr[-500:])


@pytest.mark.gpu
def test_timing_driver_on_the_real_binary(tmp_path):
    from tetris_amd import timing
    from tetris_amd import workloads as W

    layers = [W.Layer("tiny", i, "l%d" % i, c, hw, hw, k, ks, st, ks // 2, 0.8)
              for i, (c, hw, k, ks, st) in enumerate([(16, 14, 32, 3, 1), (24, 10, 20, 1, 1), (8, 21, 16, 3, 2)])]
    folder = str(tmp_path / "tiny-80")
    assert timing.write_layers(layers, folder) == 3
    csv, rows = timing.time_folder(os.path.join(BIN, "spconv2d_test"), folder, 2, str(tmp_path / "logs"))
    assert len(rows) == 3 and all(0 < ms < 50 for _, ms in rows)
    lines = open(csv).read().splitlines()
    assert lines[0] == ",op_name,spconv2d" and len(lines) == 4 and lines[1].startswith("0,000_l0_H_14_W_14_IC_16_OC_32_KS_3")


def _counter_csv(path, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        f.write('"Correlation_Id","Dispatch_Id","Agent_Id","Kernel_Name","Counter_Name","Counter_Value"\n')
        for did, kernel, counter, value in rows:
            f.write('%d,%d,"Agent 4","%s","%s",%s\n' % (did, did, kernel, counter, value))


def test_memory_metric_reads_counters_and_writes_the_table(tmp_path):
    # host logic of the conflict-counter loop (counterpart of evalution/script/memory_metric.sh and the checks of
    # evalution/draw_ablation_b.py:36-41), on counter files in rocprofv3's csv layout
    from tetris_amd import memory_metric as M

    conv = "void tetris::(anonymous namespace)::spconv2d_kernel<1, 1>(float const*, float*)"
    _counter_csv(str(tmp_path / "wo" / "x" / "1_counter_collection.csv"), [
        (1, "decode_kernel", "SQ_INSTS_LDS", 99), (2, conv, "SQ_INSTS_LDS", 1000), (2, conv, "SQ_LDS_BANK_CONFLICT", 300),
        (2, conv, "SQ_LDS_IDX_ACTIVE", 600), (3, conv, "SQ_INSTS_LDS", 1000), (3, conv, "SQ_LDS_BANK_CONFLICT", 300),
        (3, conv, "SQ_LDS_IDX_ACTIVE", 600), (3, conv, "GRBM_GUI_ACTIVE", 5)])
    s = M.conv_counter_sums(str(tmp_path / "wo"))
    assert s == {"SQ_INSTS_LDS": 2000.0, "SQ_LDS_BANK_CONFLICT": 600.0, "SQ_LDS_IDX_ACTIVE": 1200.0, "dispatches": 2}
    with pytest.raises(RuntimeError):
        M.conv_counter_sums(str(tmp_path / "nothing"))
    wi = {"SQ_INSTS_LDS": 2000.0, "SQ_LDS_BANK_CONFLICT": 0.0, "SQ_LDS_IDX_ACTIVE": 640.0, "dispatches": 2}
    M.write_table(str(tmp_path / "t.csv"), [("conv_a", {"wo": s, "wi": wi})])
    assert open(str(tmp_path / "t.csv")).read().splitlines()[1] == "0,conv_a,2000,2000,600,0,1200,640,0.5000,0.0000"
    with pytest.raises(SystemExit):
        M.main(["--weights", str(tmp_path), "--bin-dir", str(tmp_path / "no_bin")])


@pytest.mark.gpu
def test_memory_metric_on_the_real_binaries(tmp_path):
    # the pitch rule is what keeps the kernel's LDS reads free of bank conflicts: on a layer whose fixed tile needs a
    # padded pitch the binary without the rule shows conflict cycles, the one with it none
    import shutil
    from tetris_amd import memory_metric as M
    from tetris_amd import timing

    if not shutil.which("rocprofv3"):
        pytest.skip("rocprofv3 not on PATH")
    rng = np.random.default_rng(5)
    wf = str(tmp_path / "conv_H_28")
    timing.write_weight_file(wf, sparse_filter(rng, 64, 32, 3, 0.8), 28, 28, 1, 1)
    try:
        r = M.profile_layer(BIN, wf, 4, str(tmp_path / "prof"), timeout=150)
    except (RuntimeError, subprocess.TimeoutExpired) as e:  # the profiler, not the library: nothing to assert here
        pytest.skip("rocprofv3 gave no counters on this machine: %s" % str(e)[-300:])
    for v in ("wo", "wi"):
        assert r[v]["dispatches"] == 130 and r[v]["SQ_INSTS_LDS"] > 0 and r[v]["SQ_LDS_IDX_ACTIVE"] > 0  # 30 warm + 100 timed
    assert r["wi"]["SQ_LDS_BANK_CONFLICT"] <= 0.01 * r["wi"]["SQ_LDS_IDX_ACTIVE"]
    assert r["wo"]["SQ_LDS_BANK_CONFLICT"] >= r["wi"]["SQ_LDS_BANK_CONFLICT"]


def test_timing_driver_vendor_columns(tmp_path, monkeypatch):
    # --vendors: the reference's cudnn / cusparse columns of conv2d_timing.py, here miopen / rocsparse, before the
    # library's own column; the children are stand-ins
    from tetris_amd import timing

    folder = tmp_path / "net-90"
    folder.mkdir()
    rng = np.random.default_rng(3)
    timing.write_weight_file(str(folder / "conv_0"), sparse_filter(rng, 8, 4, 3, 0.5), 9, 9, 1, 1)
    fake = tmp_path / "fake_bin"
    fake.write_text("#!/bin/sh\ncat <<'EOT'\n" + CANNED + "EOT\n")
    fake.chmod(0o755)
    monkeypatch.setattr(timing, "time_vendor", lambda kind, path, batch: ({}, 0.5 if kind == "dense" else 7.25, 1.0))
    csv, rows = timing.time_folder(str(fake), str(folder), 4, str(tmp_path / "logs"), vendors=True)
    assert open(csv).read().splitlines() == [",op_name,miopen,rocsparse,spconv2d", "0,conv_0,0.50000,7.25000,%.5f" % 0.012345]
    log = open(str(tmp_path / "logs" / "net-90_batch_4.log")).read()
    assert "miopen: time = 0.50000ms" in log and "rocsparse: time = 7.25000ms" in log and "spconv2d: time = 0.0123" in log
    sp = dict(timing.geo_mean_speedups(rows + [("conv_1", 0.25, [1.0, 1.0])]))  # evalution/overall_speedup.py:45-51
    assert abs(sp["miopen"] - (0.5 / 0.012345 * 4.0) ** 0.5) < 1e-9 and abs(sp["rocsparse"] - (7.25 / 0.012345 * 4.0) ** 0.5) < 1e-9


def test_vendor_driver_explains_itself(capsys):
    from tetris_amd import vendor_test

    assert vendor_test.main(["dense"]) == 2
    assert capsys.readouterr().out.startswith("args : 2 vendor_test dense")


@pytest.mark.gpu
@pytest.mark.parametrize("kind,label", [("dense", "MIOpen"), ("csr", "Rocsparse")])
def test_vendor_driver_on_the_gpu(tmp_path, kind, label):
    # one child process per layer and vendor, the reference's stdout lines, the result checked against a dense conv
    import sys
    from tetris_amd import timing

    rng = np.random.default_rng(6)
    wf = str(tmp_path / "layer")
    timing.write_weight_file(wf, sparse_filter(rng, 24, 16, 3, 0.8), 14, 14, 1, 1)
    env = dict(os.environ, PYTHONPATH=os.path.join(ROOT, "tetris-artifact-evalution_amd"))
    p = subprocess.run([sys.executable, "-m", "tetris_amd.vendor_test", kind, wf, "2", "--check"], capture_output=True,
                       text=True, timeout=300, env=env)
    assert p.returncode == 0, p.stdout[-800:] + p.stderr[-800:]
    cfg, ms, tf = timing.parse_output(p.stdout)
    assert cfg["out_channel"] == "24" and cfg["batch_size"] == "2" and ms > 0 and tf > 0
    assert "Time of %s :" % label in p.stdout and "Sparse Pass." in p.stdout
    assert timing.time_vendor(kind, wf, 2)[1] > 0
