#!/usr/bin/env python3
"""Benchmark of the gfx950 filter-sparse conv2d path on one MI355X.

A "step" is one pass of the hot path over one synthetic batch: every conv layer of the chosen suite
(default: the VGG19-shaped stack at batch 16) launched once, back to back on one stream, inputs and
packed weights already resident in HBM.  Prints ONE short JSON line (under 4 KB): whole-step dense-equivalent
GFLOP/s (the reference's "FLOPS" figure, Tetris/spconv2d.cc:358, in decimal giga), the roofline of the conv
kernel, a CPU baseline measured on this box's cores, and one row of scalars for each other workload of the
metric (the single layer at batch 1, VGG19 at batch 1/4/8, ResNet-50, MobileNet and YOLOv3 at batch 16).
Per-layer microseconds and roofline fractions of every workload go to the file --details names.  Every layer
of every timed workload is compared with the CPU oracle on the whole batch; a mismatch beyond 1e-4 makes
the exit status non-zero.  Before the W warm-up steps of a workload, untimed passes of the same workload run for
--settle-ms (30 ms): the shader clock idles near 2.1 GHz and needs 10-25 ms of unbroken work to reach the 2.3-2.4 GHz
it holds under load, which short workloads would otherwise be timed without (`settle_ms` in the output).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms 30] [--suite vgg19|resnet50|mobilenet|yolov3|single]
                  [--batch N] [--no-cpu] [--no-check] [--no-suites] [--details FILE]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tetris-artifact-evalution_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))

PEAK_HBM_GBS = 8000.0        # MI355X published HBM3E bandwidth
PEAK_FP32_TFLOPS = 157.3     # MI355X published vector/matrix fp32 peak


OTHER_WORKLOADS = [("single", 1), ("vgg19", 1), ("vgg19", 4), ("vgg19", 8), ("resnet50", 16), ("mobilenet", 16),
                   ("yolov3", 16)]
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
CSRC = os.path.join(ROOT, "tetris-artifact-evalution_amd", "csrc")


def csrc_digest():
    """Short digest of the kernel sources, to tell whether a recorded counter figure was taken on this code."""
    import hashlib
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".h", ".inc", ".cpp")):
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:12]


def measured_traffic(workload):
    """HBM bytes per layer launch (conv kernel plus, for split layers, the reduce kernel; average over a step) from the
    rocprofv3 FETCH_SIZE / WRITE_SIZE summaries: one text line per workload, stamped with the commit and the digest of
    the kernel sources it was measured on.  None for a workload without a line."""
    try:
        lines = open(TRAFFIC_FILE).read().splitlines()
    except OSError:
        return None
    for ln in lines:
        f = ln.split()
        if len(f) >= 6 and f[0] == workload:
            return {"bytes_per_launch": float(f[1]) + float(f[2]), "read": float(f[1]), "written": float(f[2]),
                    "commit": f[3], "csrc_digest": f[4], "measured": f[5], "file": "profiles/hbm_traffic.txt",
                    "stale": f[4] != csrc_digest()}
    return None


def run_workload(T, W, torch, np, O, args, suite, N, steps, warmup, layer_repeat, masks=None, loaded=None, keep=False):
    """Pack, time and check one (suite, batch): K steps of every layer back to back on the null stream, a per-layer
    table, and every layer's output compared with the CPU oracle's packed-format convolution of the same tensors."""
    dev = torch.device("cuda:0")
    layers = W.pruned_suite(masks) if masks else W.SUITES[suite]()
    if masks:
        suite = layers[0].suite
    if loaded is not None and (loaded["suite"], loaded["batch"], len(loaded["tiles"])) != (suite, N, len(layers)):
        sys.exit("bench.py: %s was written for another workload" % args.load_tiles)
    packs, tiles, xs, ys, works, ws = [], [], [], [], [], []
    t_pack = 0.0
    for li, L in enumerate(layers):
        w = W.make_weights(L)
        if loaded is not None:
            tile = T.Tile(*loaded["tiles"][li])
        elif args.tile == "autotune":
            tile, _ = T.tile_autotune(w, N, L.H, L.W, L.stride, L.pad, args.candidates)
        else:
            tile = T.tile_select(N, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
        t0 = time.perf_counter()
        pk = T.G950Filter.for_tile(w, tile, oc_order=args.oc_order)
        torch.cuda.synchronize()
        t_pack += time.perf_counter() - t0
        x = torch.from_numpy(W.make_activations(L, N)).to(dev)
        oh, ow = W.out_hw(L)
        y = torch.full((N, L.K, oh, ow), float("nan"), dtype=torch.float32, device=dev)
        packs.append(pk); tiles.append(tile); xs.append(x); ys.append(y); works.append(W.work(L, N)); ws.append(w)
    torch.cuda.synchronize()
    if keep and args.save_tiles:
        with open(args.save_tiles, "w") as f:
            json.dump({"suite": suite, "batch": N,
                       "tiles": [t.as_list() for t in tiles]}, f)

    def step():
        for L, pk, tile, x, y in zip(layers, packs, tiles, xs, ys):
            pk.launch(x.data_ptr(), y.data_ptr(), N, L.H, L.W, L.stride, L.pad, tile)

    def settle():
        """The shader clock idles near 2.1 GHz and needs 10-25 ms of unbroken work to reach the 2.3-2.4 GHz it holds
        under load: untimed passes for --settle-ms before anything is timed, so that short workloads are not measured
        on the ramp (a tenth in time)."""
        t_s = time.perf_counter()
        while (time.perf_counter() - t_s) * 1e3 < args.settle_ms:
            for _ in range(4):
                step()
            torch.cuda.synchronize()

    settle()
    for _ in range(warmup):
        step()
    # The launches go to the null stream, which is torch's current stream here, so torch's events bracket them.
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    ms_per_step_dev = ev0.elapsed_time(ev1) / steps  # device-side span of the same K steps

    # every layer of the timed stack, whole batch, against the CPU oracle (not timed); the outputs started as NaN
    check = None
    if not args.no_check:
        threads = min(16, O.max_threads())
        worst, bad, strict, big = (0.0, None), [], 0.0, 0.0
        for L, w, x, y in zip(layers, ws, xs, ys):
            ref = O.G950Pack(w, 32, 8).conv(x.cpu().numpy(), L.stride, L.pad, threads=threads)
            got = y.cpu().numpy()
            diff = np.abs(got - ref)
            floor = max(1e-3, 1e-2 * float(np.max(np.abs(ref))))  # same measure as tests/helpers.max_rel_err
            err = float(np.max(diff / np.maximum(np.abs(ref), floor)))
            # the same errors under stricter denominators: an absolute floor of 1e-3 alone, and the largest |ref| alone
            strict = max(strict, float(np.max(diff / np.maximum(np.abs(ref), 1e-3))))
            big = max(big, float(np.max(diff)) / float(np.max(np.abs(ref))))
            if not err <= 1e-4:  # also catches NaN
                bad.append(L.name)
            if err > worst[0] or err != err:
                worst = (err, L.name)
        check = {"ok": not bad, "layers_checked": len(layers), "of": len(layers), "batch_checked": N,
                 "max_rel_err": worst[0], "worst_layer": worst[1], "tolerance": 1e-4, "failed_layers": bad,
                 "max_rel_err_floor_1e-3_only": strict, "max_abs_err_over_max_abs_ref": big,
                 "against": "CPU oracle, packed-format convolution of the same seeded tensors"}

    # per-layer table: events on the launch stream around back-to-back launches (reference protocol,
    # Tetris/spconv2d.cc:44-68, with fewer repetitions so the default run stays short)
    table, t_layers = [], 0.0
    if layer_repeat > 0:
        settle()  # the check above left the GPU idle
    for L, pk, tile, x, y, wk in zip(layers, packs, tiles, xs, ys, works):
        if layer_repeat <= 0:
            break
        ms = pk.time(x.data_ptr(), y.data_ptr(), N, L.H, L.W, L.stride, L.pad, tile, warm=5, repeat=layer_repeat)
        t = ms * 1e-3
        t_layers += t
        table.append({"layer": L.name, "us": round(ms * 1e3, 2),
                      "gflops_dense_equiv": round(wk["flops_dense"] / t / 1e9, 1),
                      "bound": wk["bound"], "roofline_frac": round(wk["t_roof"] / t, 4),
                      "tile": tile.as_list()})
    for pk in packs:
        pk.close()
    fl_dense = sum(w["flops_dense"] for w in works)
    fl_sparse = sum(w["flops_sparse"] for w in works)
    bytes_alg = sum(w["bytes"] for w in works)
    t_step = ms_per_step_dev * 1e-3
    t_hbm, t_fp32 = bytes_alg / (PEAK_HBM_GBS * 1e9), fl_sparse / (PEAK_FP32_TFLOPS * 1e12)
    out = {"suite": suite, "batch": N, "layers_per_step": len(layers), "steps": steps, "warmup": warmup,
           "ms_per_step": round(ms_per_step, 4), "ms_per_step_device": round(ms_per_step_dev, 4),
           "gflops_dense_equiv": round(fl_dense / (ms_per_step * 1e-3) / 1e9, 1),
           "bound": "valu_fp32" if t_fp32 >= t_hbm else "hbm",
           "roofline_frac": round(max(t_hbm, t_fp32) / t_step, 4),
           "sum_of_layer_roofs_frac": round(sum(w["t_roof"] for w in works) / t_step, 4),
           "algorithmic_bytes_per_launch": bytes_alg / len(layers),
           "sum_layer_us": round(t_layers * 1e6, 1) if table else None,
           "min_layer_roofline_frac": min((r["roofline_frac"] for r in table), default=None),
           "pack_ms_total": round(t_pack * 1e3, 2), "check": check, "layers": table}
    if keep:
        out.update({"_layers": layers, "_xs": xs, "_ys": ys, "_works": works})
    return out


def run_chain(T, W, torch, np, O, args, N, steps, warmup):
    """The VGG19-shaped stack as a network: every convolution reads the activation of the layer before -- ReLU, and
    2x2 max-pooling where the next layer's image is half as large -- instead of its own synthetic tensor.  Only the
    first layer's input is synthetic.  Timed like the stack, twice: with the activation applied by the layer's own
    kernels (tetris_spconv2d_launch_act; the figure reported) and as a second pass per layer (tetris_relu_maxpool).
    The last activation and every layer's input are checked against the same chain on the CPU (oracle convolutions,
    numpy ReLU and pooling)."""
    dev = torch.device("cuda:0")
    layers = W.SUITES["vgg19"]()
    packs, tiles, ws, convs, acts, pools = [], [], [], [], [], []
    x0 = torch.from_numpy(W.make_activations(layers[0], N)).to(dev)
    for li, L in enumerate(layers):
        w = W.make_weights(L)
        tile = T.tile_select(N, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
        packs.append(T.G950Filter.for_tile(w, tile, oc_order=args.oc_order)); tiles.append(tile); ws.append(w)
        pool = 2 if (li + 1 == len(layers) or layers[li + 1].H * 2 == L.H) else 1
        pools.append(pool)
        convs.append(torch.empty((N, L.K, L.H, L.W), dtype=torch.float32, device=dev))
        acts.append(torch.full((N, L.K, L.H // pool, L.W // pool), float("nan"), dtype=torch.float32, device=dev))

    fused = [pk.act_supported(N, L.H, L.W, L.stride, L.pad, tile, pool)
             for L, pk, tile, pool in zip(layers, packs, tiles, pools)]

    def step_two_pass():  # every activation as a second pass over the layer's output
        x = x0
        for L, pk, tile, y, a, pool in zip(layers, packs, tiles, convs, acts, pools):
            pk.launch(x.data_ptr(), y.data_ptr(), N, L.H, L.W, L.stride, L.pad, tile)
            T.relu_maxpool(y.data_ptr(), a.data_ptr(), N, L.K, L.H, L.W, pool)
            x = a

    def step():  # activations written by the layer's own kernels where its tile can (tetris_spconv2d_launch_act)
        x = x0
        for L, pk, tile, y, a, pool, f in zip(layers, packs, tiles, convs, acts, pools, fused):
            if f:
                pk.launch_act(x.data_ptr(), a.data_ptr(), N, L.H, L.W, L.stride, L.pad, tile, pool)
            else:
                pk.launch_act(x.data_ptr(), y.data_ptr(), N, L.H, L.W, L.stride, L.pad, tile, T.ACT_RELU)
                T.relu_maxpool(y.data_ptr(), a.data_ptr(), N, L.K, L.H, L.W, pool)
            x = a

    def timed(fn):
        t_s = time.perf_counter()  # untimed passes until the shader clock has settled (see run_workload)
        while (time.perf_counter() - t_s) * 1e3 < args.settle_ms:
            fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    ms_two = timed(step_two_pass)
    for a in acts:
        a.fill_(float("nan"))
    ms = timed(step)  # last, so that the activations checked below are the fused pass's
    out = {"workload": "vgg19-shaped network pass, batch %d: 16 sparse convolutions, each followed by ReLU (2x2 max-pooling "
           "after layers 1, 3, 7, 11 and 15); every layer's input is the previous activation; the activation is applied "
           "by the layer's own kernels as they write (tetris_spconv2d_launch_act)" % N,
           "ms_per_pass": round(ms, 4), "steps": steps, "warmup": warmup,
           "launches_per_pass": len(layers) + sum(not f for f in fused),
           "layers_with_the_activation_as_a_second_pass": [L.name for L, f in zip(layers, fused) if not f],
           "ms_per_pass_activations_as_second_passes": round(ms_two, 4),
           "gflops_dense_equiv": round(sum(W.work(L, N)["flops_dense"] for L in layers) / (ms * 1e-3) / 1e9, 1)}
    if not args.no_check:
        threads = min(16, O.max_threads())
        ref, worst, bad = x0.cpu().numpy(), (0.0, None), []
        for L, w, a, pool in zip(layers, ws, acts, pools):
            ref = np.maximum(O.G950Pack(w, 32, 8).conv(np.ascontiguousarray(ref), L.stride, L.pad, threads=threads), 0.0)
            if pool == 2:
                n, c, h, wd = ref.shape
                ref = ref.reshape(n, c, h // 2, 2, wd // 2, 2).max(axis=(3, 5))
            got = a.cpu().numpy()
            floor = max(1e-3, 1e-2 * float(np.max(np.abs(ref))))
            err = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))
            if not err <= 1e-4:
                bad.append(L.name)
            if err > worst[0] or err != err:
                worst = (err, L.name)
            ref = got  # the next layer is checked on the activation the device produced (errors do not pile up)
        out["check"] = {"ok": not bad, "activations_checked": len(layers), "max_rel_err": worst[0], "worst_layer": worst[1],
                        "tolerance": 1e-4, "failed_layers": bad,
                        "against": "CPU oracle convolution + numpy ReLU / pooling of the device's previous activation"}
    if args.dense_baseline:
        import torch.nn.functional as F
        wd = [torch.from_numpy(w).to(dev) for w in ws]

        def dense_step():
            x = x0
            for L, w, pool in zip(layers, wd, pools):
                x = F.relu(F.conv2d(x, w, None, L.stride, L.pad))
                if pool == 2:
                    x = F.max_pool2d(x, 2)

        for _ in range(3):
            dense_step()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(steps):
            dense_step()
        e1.record()
        torch.cuda.synchronize()
        out["vendor_dense_fp32_ms_per_pass"] = round(e0.elapsed_time(e1) / steps, 4)
    for pk in packs:
        pk.close()
    return out


def summary_line(full, details):
    """The one JSON line of stdout: the contract's fields, `roofline`, `cpu_baseline`, `check` and one row of scalars per
    other workload.  Kept well under 4 KB (a test holds it to that): per-layer tables live in the side file."""
    def pick(d, keys):
        return {k: d[k] for k in keys if d is not None and k in d}

    rl = full["roofline"]
    line = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "settle_ms", "ms_per_step",
                                 "ms_per_step_device", "higher_is_better", "scaling", "vs_baseline", "dtype", "data")}
    line["metric"] = "effective GFLOP/s (dense-equivalent), sparse conv stack"
    line["config"] = pick(full["config"], ("workload", "suite", "batch", "layers"))
    line["check"] = None if full["check"] is None else pick(full["check"], (
        "ok", "max_rel_err", "tolerance", "all_workloads_ok") + (() if full["check"]["all_workloads_ok"] else ("failed_workloads",)))
    line["roofline"] = pick(rl, ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "avg_launch_us",
                                 "launches_per_step", "algorithmic_flops_per_launch", "algorithmic_bytes_per_launch"))
    for k in ("algorithmic_flops_per_launch", "algorithmic_bytes_per_launch", "traffic"):
        if line["roofline"].get(k) is not None:
            line["roofline"][k] = int(round(line["roofline"][k]))
    line["roofline"]["note"] = rl.get("note")
    cpu = full["cpu_baseline"]
    line["cpu_baseline"] = None if cpu is None else pick(cpu, ("value", "unit", "cores", "kind", "sample"))
    line["min_layer_roofline_frac"] = full["min_layer_roofline_frac"]
    ctx = full["context"] or {}
    line["context"] = pick(ctx, ("measured_copy_gbs", "measured_fma_tflops", "vendor_dense_fp32_ms_per_step",
                                 "vendor_csr_im2col_ms_per_step"))
    # other workloads: [suite, batch, ms per pass, bound, fraction of the binding roof, smallest layer fraction,
    #                   counter bytes / algorithmic bytes, check ok]
    line["suites_cols"] = "suite,batch,ms,bound,frac,min_layer_frac,traffic_ratio,ok"
    line["suites"] = [[r["suite"], r["batch"], r["ms_per_step_device"], r["bound"].replace("valu_", ""), r["roofline_frac"],
                       r["min_layer_roofline_frac"],
                       round(r["traffic"] / r["algorithmic_bytes_per_launch"], 3) if r.get("traffic") else None,
                       None if r["check"] is None else r["check"]["ok"]] for r in full["suites"]]
    ch = full["chain"]
    line["chain"] = None if ch is None else {"ms_per_pass": ch["ms_per_pass"],
                                             "check_ok": ch.get("check", {}).get("ok") if ch.get("check") else None}
    line["details"] = os.path.relpath(details, ROOT) if details else None
    if line["check"] and isinstance(line["check"].get("max_rel_err"), float):
        line["check"]["max_rel_err"] = float("%.3g" % line["check"]["max_rel_err"])
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--settle-ms", type=float, default=30.0, help="untimed passes for this long before the warm-up steps "
                    "of every timed workload, so that the shader clock is where it stays under load (0: none)")
    ap.add_argument("--suite", default="vgg19")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--masks", metavar="NPZ", help="run the layers of a pruned network instead of --suite: a mask file "
                    "as tests/golden/masks_*.npz (zero patterns of shipped pruned weight files, seeded values)")
    ap.add_argument("--oc-order", choices=("balanced", "file", "reference"), default="balanced",
                    help="output-channel order of the packs: balanced over the waves of a workgroup, as in the filter, or "
                         "the order of the reference's ReorderOutChannel pass")
    ap.add_argument("--no-suites", action="store_true",
                    help="time only --suite at --batch, not the other workloads of the `suites` block")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-chain", action="store_true",
                    help="skip the whole-network pass of the vgg19 suite (layers chained through ReLU and max-pooling)")
    ap.add_argument("--no-check", action="store_true", help="skip the check of every layer against the CPU oracle")
    ap.add_argument("--layer-repeat", type=int, default=30, help="timed launches per layer for the per-layer table")
    ap.add_argument("--tile", choices=("autotune", "select"), default="select",
                    help="select: the library's own choice (its built-in table of tiles measured on MI355X, else its cycle "
                         "model); autotune: time the model's best candidates per layer during set-up, as the reference's "
                         "driver does with its 185-entry table")
    ap.add_argument("--candidates", type=int, default=24)
    ap.add_argument("--save-tiles", metavar="FILE", help="write the tile chosen for every layer to FILE (JSON)")
    ap.add_argument("--load-tiles", metavar="FILE", help="use the tiles a previous --save-tiles run wrote (so that a "
                    "profiled run launches nothing but packing and the timed convolutions)")
    ap.add_argument("--dense-baseline", action="store_true",
                    help="also time the vendor's dense fp32 convolution (MIOpen through torch) on the same layers, as "
                         "context (the reference compares with cuDNN the same way, Tetris/cuda_utils.cc:6-132)")
    ap.add_argument("--csr-baseline", action="store_true",
                    help="also time the vendor sparse-library path on the same tensors: im2col (torch unfold) + CSR x "
                    "dense product (torch.sparse.mm, rocSPARSE), the counterpart of the reference's cusparse_test")
    ap.add_argument("--details", metavar="FILE", default=os.path.join(ROOT, "gpurun_out", "bench_layers.json"),
                    help="where the full record goes (per-layer tables of every workload, chain, context); stdout "
                         "carries one short JSON line")
    ap.add_argument("--calibrate-copy", type=int, metavar="MIB", default=0,
                    help="instead of the benchmark, run one elementwise copy kernel over MIB MiB (reads MIB, writes MIB): "
                         "the known-size dispatch that scales the FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this engine runs on one GPU (no collectives or sharding are part of the path); "
                 "--gpus %d is not supported" % args.gpus)

    import numpy as np
    import torch

    import tetris_amd as T
    from tetris_amd import workloads as W

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        n = args.calibrate_copy * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(4):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_mib": args.calibrate_copy, "dispatches": 4,
                          "bytes_read_per_dispatch": 4 * n, "bytes_written_per_dispatch": 4 * n}))
        return
    T.G950Filter(np.ones((8, 8, 1, 1), np.float32), 8, 8).close()  # loads the device code, so pack times exclude it
    O = None
    if not (args.no_check and args.no_cpu):
        import oracle_py as O
    loaded = json.load(open(args.load_tiles)) if args.load_tiles else None
    main_run = run_workload(T, W, torch, np, O, args, args.suite, args.batch, args.steps, args.warmup, args.layer_repeat,
                            masks=args.masks, loaded=loaded, keep=True)
    layers, N = main_run.pop("_layers"), args.batch
    xs, ys, works = main_run.pop("_xs"), main_run.pop("_ys"), main_run.pop("_works")
    if args.masks:
        args.suite = layers[0].suite
    ms_per_step, ms_per_step_dev, table = main_run["ms_per_step"], main_run["ms_per_step_device"], main_run["layers"]
    check = main_run["check"]
    failed = [] if check is None or check["ok"] else ["%s/%d" % (args.suite, N)]

    fl_dense = sum(w["flops_dense"] for w in works)
    fl_sparse = sum(w["flops_sparse"] for w in works)
    bytes_alg = sum(w["bytes"] for w in works)
    t_roof = sum(w["t_roof"] for w in works)
    n_launch = len(layers)
    # Average launch duration of the conv kernel over the timed region: the device-side span of the K steps
    # (events on the launch stream) divided by the launches in it; nothing else runs on the stream in between.
    t_step = ms_per_step_dev * 1e-3
    t_hbm, t_fp32 = bytes_alg / (PEAK_HBM_GBS * 1e9), fl_sparse / (PEAK_FP32_TFLOPS * 1e12)
    if t_fp32 >= t_hbm:
        achieved = fl_sparse / t_step / 1e12
        # the contract's label for the compute roof is "mfma"; the work here is vector fp32 FMA on the VALU, no MFMA
        roofline = {"bound": "mfma", "bound_detail": "valu_fp32",
                    "note": "VALU fp32 FMA, no MFMA; peak needs packed fp32 (off here: 78.6 reachable)",
                    "achieved": round(achieved, 3), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / PEAK_FP32_TFLOPS, 4)}
    else:
        achieved = bytes_alg / t_step / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(achieved / PEAK_HBM_GBS, 4)}
    traffic = measured_traffic("%s/%d" % (args.suite, N))
    roofline.update({"kernel": "spconv2d_kernel", "launches_per_step": n_launch,
                     "avg_launch_us": round(t_step / n_launch * 1e6, 2),
                     "algorithmic_flops_per_launch": fl_sparse / n_launch,
                     "algorithmic_bytes_per_launch": bytes_alg / n_launch,
                     "sum_of_layer_roofs_frac": round(t_roof / t_step, 4),
                     "traffic": traffic["bytes_per_launch"] if traffic else None,
                     "traffic_source": traffic})

    # the other workloads of the metric ("batch 1-16" over the four suites and the single layer), each timed and
    # checked the same way with fewer steps
    suites = []
    if not (args.no_suites or args.masks):
        for suite, n in OTHER_WORKLOADS:
            if (suite, n) == (args.suite, N):
                continue
            r = run_workload(T, W, torch, np, O, args, suite, n, max(5, args.steps // 2), max(3, args.warmup // 3),
                             min(args.layer_repeat, 10))
            t = measured_traffic("%s/%d" % (suite, n))
            r["traffic"] = t["bytes_per_launch"] if t else None
            if r["check"] is not None and not r["check"]["ok"]:
                failed.append("%s/%d" % (suite, n))
            suites.append(r)

    chain = None
    if args.suite == "vgg19" and not (args.no_chain or args.masks):
        chain = run_chain(T, W, torch, np, O, args, N, max(5, args.steps // 2), max(3, args.warmup // 3))
        if chain.get("check") is not None and not chain["check"]["ok"]:
            failed.append("vgg19/%d chained" % N)

    cpu = None
    if not args.no_cpu:
        threads = min(O.max_threads(), 16)
        # The same workload (every layer at the benchmark's batch) once through the reference's own packed layout and its
        # CPU decode -- SparseFilter arrays built with Bank-SR and ReorderOutChannel, vectorised, TILE_IC 32, walked by the
        # restatement of HostReorderSpconv2d -- cut short after about 25 s of wall time: a few hundred core-seconds.
        budget_s, done_fl, t_cpu, t_cpu_pack, used, agree = 25.0, 0.0, 0.0, 0.0, 0, 0.0
        for L, x, y in zip(layers, xs, ys):
            w = W.make_weights(L)
            xn = x.cpu().numpy()
            t0 = time.perf_counter()
            pk = O.SpfPack(w, 32, apply_reorder=True, apply_vectorize=True, bank_optimize=True, reorder_out_channel=True)
            t_cpu_pack += time.perf_counter() - t0
            t0 = time.perf_counter()
            ref = pk.conv(xn, L.stride, L.pad, threads=threads)
            t_cpu += time.perf_counter() - t0
            done_fl += W.work(L, N)["flops_dense"]
            used += 1
            if not args.no_check:
                floor = max(1e-3, 1e-2 * float(np.max(np.abs(ref))))
                agree = max(agree, float(np.max(np.abs(y.cpu().numpy() - ref) / np.maximum(np.abs(ref), floor))))
            if t_cpu > budget_s:
                break
        cpu = {"value": round(done_fl / t_cpu / 1e9, 2), "unit": "GFLOP/s", "cores": threads,
               "kind": "port", "sample": "%d of %d %s layers, batch %d, one pass: reference SparseFilter layout (TILE_IC 32, "
               "Bank-SR + ReorderOutChannel, vec4) decoded by the oracle's HostReorderSpconv2d, OpenMP over (n, oc), %.1f s"
               % (used, len(layers), args.suite, N, t_cpu),
               "pack_s": round(t_cpu_pack, 2),
               "gpu_vs_this_cpu_output_max_rel_err": None if args.no_check else agree}
        if not args.no_check and not agree <= 1e-4:
            failed.append("%s/%d vs reference-layout CPU decode" % (args.suite, N))
        # the dense CPU convolution of the same path (restates HostConv2d, tensor_utils.cc:136-170), OpenMP over (n, oc)
        L = W.single_layer()[0]
        w1, x4 = W.make_weights(L), W.make_activations(L, 4)
        t0 = time.perf_counter()
        O.host_conv2d(x4, w1, L.stride, L.pad, threads=threads)
        dt = time.perf_counter() - t0
        cpu["dense_host_conv2d"] = {"value": round(W.work(L, 4)["flops_dense"] / dt / 1e9, 2), "unit": "GFLOP/s",
                                    "cores": threads, "kind": "port",
                                    "sample": "single 64->128 56x56 3x3 layer, batch 4, %.2f s" % dt}
        if O.ref_available():
            L = W.single_layer()[0]
            w, x1 = W.make_weights(L), W.make_activations(L, 1)
            t0 = time.perf_counter()
            O.ref_host_conv2d(x1, w, L.stride, L.pad)
            dt = time.perf_counter() - t0
            cpu["reference_HostConv2d"] = {"value": round(W.work(L, 1)["flops_dense"] / dt / 1e9, 3),
                                           "unit": "GFLOP/s", "cores": 1, "kind": "reference",
                                           "sample": "single 64->128 56x56 3x3 layer, batch 1, %.2f s" % dt}

    # what this box delivers to a plain copy and to a loop of independent FMAs, next to the nominal peaks
    copy_gbs, fma_tflops = T.measure_peaks()
    context = {"measured_copy_gbs": round(copy_gbs, 1), "measured_fma_tflops": round(fma_tflops, 2),
               "peaks_note": "tetris_measure_peaks: device copy of 256 MiB (read + write bytes) and sixteen independent "
                             "non-packed fp32 FMA chains per lane; nominal peaks 8000 GB/s and 157.3 TFLOP/s (packed)",
               "roofline_frac_of_measured": round((fl_sparse / t_step / 1e12) / fma_tflops, 4) if t_fp32 >= t_hbm
               else round((bytes_alg / t_step / 1e9) / copy_gbs, 4)}
    if args.dense_baseline:
        import torch.nn.functional as F
        ws = [torch.from_numpy(W.make_weights(L)).to(dev) for L in layers]

        def dense_step():
            for L, x, w in zip(layers, xs, ws):
                F.conv2d(x, w, None, L.stride, L.pad)

        for _ in range(3):
            dense_step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            dense_step()
        e1.record()
        torch.cuda.synchronize()
        dense_ms = e0.elapsed_time(e1) / args.steps
        context.update({"vendor_dense_fp32_ms_per_step": round(dense_ms, 4),
                   "vendor_dense_fp32_gflops": round(fl_dense / (dense_ms * 1e-3) / 1e9, 1),
                   "speedup_over_vendor_dense": round(dense_ms / ms_per_step, 3),
                   "note": "torch.nn.functional.conv2d (MIOpen) on the same tensors, weights dense with the zeros in"})

    if args.csr_baseline:
        import torch.nn.functional as F
        try:
            csr = [torch.from_numpy(W.make_weights(L).reshape(L.K, -1)).to(dev).to_sparse_csr() for L in layers]

            def csr_step():
                for L, x, a in zip(layers, xs, csr):
                    for n in range(N):  # one image at a time keeps the unfolded matrix small (C*ks*ks x OH*OW)
                        torch.sparse.mm(a, F.unfold(x[n:n + 1], L.ks, padding=L.pad, stride=L.stride)[0])

            csr_step()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            csr_step()
            e1.record()
            torch.cuda.synchronize()
            csr_ms = e0.elapsed_time(e1)
            context.update({"vendor_csr_im2col_ms_per_step": round(csr_ms, 3),
                            "speedup_over_vendor_csr": round(csr_ms / ms_per_step, 2),
                            "csr_note": "per image: torch unfold (im2col) + torch.sparse.mm (CSR weights x dense "
                                        "columns, rocSPARSE); one pass, outputs discarded"})
        except Exception as e:  # the sparse library path is context, not the product
            context.update({"vendor_csr_im2col_ms_per_step": None, "csr_note": "failed: %r" % (e,)})

    full = {
        "metric": "effective GFLOP/s (dense-equivalent) over the layer stack; per-layer us and roofline in `layers`",
        "value": round(fl_dense / (ms_per_step * 1e-3) / 1e9, 1),
        "unit": "GFLOP/s",
        "check": dict(check or {}, all_workloads_ok=not failed, failed_workloads=failed) if not args.no_check else None,
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_device": round(ms_per_step_dev, 4),
        # untimed passes of the same workload before the W warm-up steps, until the shader clock has settled
        "settle_ms": args.settle_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s-shaped sparse conv stack, %d layers, batch %d, fp32 NCHW, seeded masks"
                   % (args.suite, len(layers), N), "suite": args.suite, "batch": N, "layers": len(layers),
                   "base_seed": W.BASE_SEED,
                   "tensor_seed": "base_seed ^ crc32('<suite>/<layer index>/<w|x>'), splitmix64 streams "
                                  "(tetris_amd/workloads.py)"},
        "sparse_gflops": round(fl_sparse / (ms_per_step * 1e-3) / 1e9, 1),
        "sum_layer_us": main_run["sum_layer_us"],
        "min_layer_roofline_frac": main_run["min_layer_roofline_frac"],
        "pack_ms_total": main_run["pack_ms_total"],
        "tile_selection": args.tile,
        "oc_order": args.oc_order,
        "csrc_digest": csrc_digest(),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "context": context,
        "layers": table,
        "suites": suites,
        "chain": chain,
    }
    # Everything measured (per-layer tables of every workload included) goes to a side file; stdout carries ONE short
    # line, like the reference's two-line report (Tetris/spconv2d.cc:357-358): scalars only, a few hundred bytes per block.
    details = args.details
    try:
        os.makedirs(os.path.dirname(details) or ".", exist_ok=True)
        with open(details, "w") as f:
            json.dump(full, f)
    except OSError as e:
        print("bench.py: could not write %s: %s" % (details, e), file=sys.stderr)
        details = None
    print(json.dumps(summary_line(full, details)))
    if failed:
        sys.exit("bench.py: outputs differ from the CPU oracle beyond 1e-4 on: %s" % ", ".join(failed))


if __name__ == "__main__":
    main()
