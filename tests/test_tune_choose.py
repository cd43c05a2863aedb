"""tetris_amd/tune.py --choose on made-up counter files: the dispatch matching (a conv kernel, optionally followed by
its reduce kernel, per shortlisted tile) and the selection rules (fewest bytes within the slack for HBM-bound layers,
fastest tile for layers bound by the vector units, the incumbent kept unless it wastes bytes)."""
import csv
import json
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "tetris-artifact-evalution_amd")
HEAD = ["Correlation_Id", "Dispatch_Id", "Agent_Id", "Queue_Id", "Process_Id", "Thread_Id", "Grid_Size", "Kernel_Id",
        "Kernel_Name", "Workgroup_Size", "LDS_Block_Size", "Scratch_Size", "VGPR_Count", "Accum_VGPR_Count", "SGPR_Count",
        "Counter_Name", "Counter_Value", "Start_Timestamp", "End_Timestamp"]


def _counters(path, name, per_launch):
    """per_launch: [(conv value, reduce value or None), ...]; other kernels are sprinkled in between"""
    os.makedirs(os.path.join(path, "vm"))
    with open(os.path.join(path, "vm", "1_counter_collection.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(HEAD)
        did = 0

        def row(kernel, value):
            nonlocal did
            did += 1
            w.writerow([did, did, "Agent 1", 1, 1, 1, 64, 1, kernel, 256, 0, 0, 8, 0, 16, name, value, 0, 1])

        for conv, red in per_launch:
            row("tetris::(anonymous namespace)::bind_kernel(int const*, float const*)", 1e9)  # not a conv launch
            row("void tetris::(anonymous namespace)::spconv2d_flat6<1>(float const*, float*)", conv)
            if red is not None:
                row("tetris::(anonymous namespace)::reduce_kernel(float const*, float*, long long, int)", red)


def _run(args):
    env = dict(os.environ, PYTHONPATH=PKG + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, "-m", "tetris_amd.tune"] + args, capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stderr


def _rows(path):
    pat = re.compile(r"\s*\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), \{(\d+), (\d+), (\d+), (\d+), (\d+)\}\},\s*// (.*)")
    out = {}
    for ln in open(path):
        m = pat.match(ln)
        if m:
            v = [int(x) for x in m.groups()[:13]]
            out[tuple(v[:8])] = (v[8:], m.group(14))
    return out


def test_choose_takes_fewest_bytes_within_the_slack_only_for_hbm_bound_layers(tmp_path):
    sys.path.insert(0, PKG)
    from tetris_amd import workloads as W

    mob = W.SUITES["mobilenet"]()[2]   # 128->128 56x56 pointwise: HBM-bound
    vgg = W.SUITES["vgg19"]()[5]       # 256->256 56x56 3x3: bound by the vector units
    assert W.work(mob, 16)["bound"] == "hbm" and W.work(vgg, 16)["bound"] == "fp32"
    items = []
    for L in (mob, vgg):
        items.append({"key": [16, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad], "suite": L.suite, "name": L.name,
                      "index": L.index, "sparsity": L.sparsity,
                      "candidates": [{"tile": [64, 1, 8, 16, 64], "ms": 0.0200}, {"tile": [64, 1, 4, 16, 64], "ms": 0.0203},
                                     {"tile": [64, 2, 8, 8, 32], "ms": 0.0230}]})
    short = tmp_path / "short.json"
    short.write_text(json.dumps(items))
    # KiB per launch: the second tile moves fewer bytes (its reduce kernel included), the third fewest but is too slow
    fetch = [(1000, 200), (700, None), (100, None)] * 2
    write = [(1000, None), (800, None), (100, None)] * 2
    _counters(str(tmp_path / "fetch"), "FETCH_SIZE", fetch)
    _counters(str(tmp_path / "write"), "WRITE_SIZE", write)
    out = tmp_path / "t.inc"
    msg = _run(["--choose", str(short), "--fetch", str(tmp_path / "fetch"), "--write", str(tmp_path / "write"),
                "--out", str(out)])
    rows = _rows(str(out))
    assert "1 of 2 shapes took a tile other than the fastest" in msg
    k_mob, k_vgg = tuple(items[0]["key"]), tuple(items[1]["key"])
    assert rows[k_mob][0] == [64, 1, 4, 16, 64]   # within 2 % of the fastest and fewer bytes
    assert rows[k_vgg][0] == [64, 1, 8, 16, 64]   # compute-bound: the fastest
    # bytes = FETCH KiB * 1024 * 2 + WRITE KiB * 1024, the reduce kernel's share added to its conv launch
    assert "%.2f MB moved" % ((700 * 2 + 800) * 1024 / 1e6) in rows[k_mob][1]
    assert "%.2f MB moved" % ((1200 * 2 + 1000) * 1024 / 1e6) in rows[k_vgg][1]
    # slack for compute-bound layers too: now both switch
    _run(["--choose", str(short), "--fetch", str(tmp_path / "fetch"), "--write", str(tmp_path / "write"),
          "--within-compute", "0.02", "--out", str(out)])
    assert _rows(str(out))[k_vgg][0] == [64, 1, 4, 16, 64]
    # --base: the incumbent stays unless it moves more than --waste times the algorithmic bytes
    base = tmp_path / "base.inc"
    base.write_text("".join("    {%d, %d, %d, %d, %d, %d, %d, %d, {64, 1, 8, 16, 64}},  // kept\n" % tuple(it["key"]) for it in items))
    _run(["--choose", str(short), "--fetch", str(tmp_path / "fetch"), "--write", str(tmp_path / "write"),
          "--base", str(base), "--out", str(out)])
    rows = _rows(str(out))
    assert rows[k_mob] == ([64, 1, 8, 16, 64], "kept") and rows[k_vgg] == ([64, 1, 8, 16, 64], "kept")  # 3.4 MB is no waste
    _run(["--choose", str(short), "--fetch", str(tmp_path / "fetch"), "--write", str(tmp_path / "write"),
          "--base", str(base), "--waste", "0.01", "--out", str(out)])
    assert _rows(str(out))[k_mob][0] == [64, 1, 4, 16, 64]


def test_choose_refuses_counter_files_that_do_not_match_the_shortlist(tmp_path):
    items = [{"key": [16, 56, 56, 128, 128, 1, 1, 0], "suite": "mobilenet", "name": "x", "index": 2, "sparsity": 0.7,
              "candidates": [{"tile": [64, 1, 8, 16, 64], "ms": 0.02}, {"tile": [64, 1, 4, 16, 64], "ms": 0.021}]}]
    short = tmp_path / "short.json"
    short.write_text(json.dumps(items))
    _counters(str(tmp_path / "fetch"), "FETCH_SIZE", [(1, None)])
    _counters(str(tmp_path / "write"), "WRITE_SIZE", [(1, None), (1, None)])
    env = dict(os.environ, PYTHONPATH=PKG)
    r = subprocess.run([sys.executable, "-m", "tetris_amd.tune", "--choose", str(short), "--fetch", str(tmp_path / "fetch"),
                        "--write", str(tmp_path / "write"), "--out", str(tmp_path / "t.inc")], capture_output=True, text=True,
                       env=env, timeout=120)
    assert r.returncode != 0 and "conv launches" in r.stderr


def test_table_rows_with_and_without_csplit(tmp_path):
    """A table row's tile has five numbers, or six when it fixes csplit: the tuner's writer and reader agree on both,
    and the library's own loader (tetris_tile_table_load) reads what the tuner writes."""
    sys.path.insert(0, PKG)
    import tetris_amd as T
    from tetris_amd import tune

    rows = [((2, 13, 13, 512, 256, 1, 1, 0), (64, 1, 1, 16, 64, 4), "with csplit"),
            ((16, 56, 56, 256, 256, 3, 1, 1), (14, 2, 8, 16, 16), "rule")]
    path = tmp_path / "t.inc"
    tune.write_table(str(path), rows)
    pat = re.compile(tune.ROW + r",\s*// (.*)")
    got = []
    for ln in open(path):
        m = pat.match(ln)
        if m:
            g = m.groups()
            got.append((tuple(int(x) for x in g[:8]), tune.row_tile(g), g[14]))
    assert got == rows
    n = T.tile_table_load(str(path))
    assert n == 2
    t = T.tile_select(2, 13, 13, 512, 256, 1, 1, 0)
    assert t.as_list() == [64, 1, 1, 16, 64, 4] and "csplit=4" in repr(t)
    t = T.tile_select(16, 56, 56, 256, 256, 3, 1, 1)
    assert t.as_list() == [14, 2, 8, 16, 16] and t.csplit == 0
