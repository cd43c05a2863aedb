"""Per-layer timing over a folder of weight files: the counterpart of the reference's evalution/conv2d_timing.py
(its Tetris column) on this library's command-line driver.

    python -m tetris_amd.timing --weights DIR [--batch 1 4 8 16] [--log-dir DIR] [--bin PATH] [--vendors]
    python -m tetris_amd.timing --ablation --weights DIR [--batch 4] [--log-dir DIR] [--bin-dir DIR]
    python -m tetris_amd.timing --write-suite vgg19 DIR        # the synthetic suite as weight files
    python -m tetris_amd.timing --write-masks MASKS.npz DIR    # a pruned network's layers (seeded values)

For every weight file (the reference's text format: eight header ints `H W IC OC KS PAD STRIDE GROUPS`, then the
OIHW values, Tetris/tensor_utils.cc:55-82) and batch size it starts `bin/spconv2d_test <file> <batch>` as a child
process and reads the lines the reference's harness reads (conv2d_timing.py:51-79): `[Config] k = v, ...`,
`Time of Spconv2d :<ms>ms`, `FLOPS of Spconv2d :<x>T`.  Per batch size it writes, like the reference
(conv2d_timing.py:101-198), `<folder>_batch_<N>.csv` (columns: row index, op_name, spconv2d in ms with five decimals)
and `<folder>_batch_<N>.log`.  --vendors adds the columns `miopen` and `rocsparse` before it, the counterparts on this
machine of the reference's `cudnn` and `cusparse` columns (tetris_amd.vendor_test, one child process per layer and
column like the reference's cudnn_test.o / cusparse_test.o); the Sputnik columns have no counterpart here.

--ablation is the counterpart of evalution/ablation_timing.py: every layer goes through the five binaries of the
reference's ladder (ablation_timing.py:109-115: baseline_test, spf_test, bank_sr_test, filter_gr_test, para_test, built
by this package's Makefile with the switches of evalution/script/build_ablation.sh:12-16) and the times land in
`ablation_a.csv` (columns: row index, op_name, Baseline, SPF, Bank-SR, Filter-GR, Para) and `ablation_a.log`, as there
(:79-80, :143-144).
"""
import argparse
import os
import subprocess
import sys

VENDOR = "spconv2d"


def parse_output(text):
    """-> (config dict, milliseconds, TFLOPS) from the driver's stdout; -1.0 where a line is missing."""
    config, ms, tflops = {}, -1.0, -1.0
    for line in text.splitlines():
        line = line.strip()
        if "FLOPS of" in line:
            tflops = float(line.split(" :")[1][:-1])
        if "Time of" in line:
            ms = float(line.split(" :")[1][:-2])
        if "[Config]" in line:
            for item in line.split("[Config] ")[1].split(", "):
                k, v = item.split(" = ")
                config[k] = v
    return config, ms, tflops


def time_layer(binary, weight_file, batch, timeout=600):
    p = subprocess.run([binary, weight_file, str(batch)], capture_output=True, text=True, timeout=timeout)
    if p.returncode != 0:
        raise RuntimeError("%s %s %d: exit %d\n%s%s" % (binary, weight_file, batch, p.returncode, p.stdout[-2000:],
                                                      p.stderr[-2000:]))
    return parse_output(p.stdout)


VENDORS = [("dense", "miopen"), ("csr", "rocsparse")]  # the reference's cudnn and cusparse columns (conv2d_timing.py:24-28)


def time_vendor(kind, weight_file, batch, timeout=1200):
    """One vendor baseline of one layer, in a child process like every other column (tetris_amd.vendor_test)."""
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=here + os.pathsep + os.environ.get("PYTHONPATH", ""))
    cmd = [sys.executable, "-m", "tetris_amd.vendor_test", kind, weight_file, str(batch)]
    p = subprocess.run(cmd, capture_output=True, text=True, timeout=timeout, env=env)
    if p.returncode != 0:
        raise RuntimeError("%s: exit %d\n%s%s" % (" ".join(cmd), p.returncode, p.stdout[-2000:], p.stderr[-2000:]))
    return parse_output(p.stdout)


def geo_mean_speedups(rows):
    """Geometric mean over the layers of vendor time / library time, per vendor column, as the reference's summary
    prints it (evalution/overall_speedup.py:45-51); rows as time_folder returns them with vendors=True."""
    import math
    out = []
    for k, (_, name) in enumerate(VENDORS):
        ratios = [r[2][k] / r[1] for r in rows if r[1] > 0 and r[2][k] > 0]
        out.append((name, math.exp(sum(math.log(v) for v in ratios) / len(ratios)) if ratios else float("nan")))
    return out


def time_folder(binary, folder, batch, log_dir, vendors=False):
    folder = folder.rstrip("/")
    tag = "%s_batch_%d" % (os.path.basename(folder), batch)
    os.makedirs(log_dir, exist_ok=True)
    rows = []
    with open(os.path.join(log_dir, tag + ".log"), "w") as log:
        for idx, op in enumerate(sorted(os.listdir(folder))):
            path = os.path.join(folder, op)
            if not os.path.isfile(path):
                continue
            log.write("# Run[%d]: %s\n" % (idx, path))
            others = [(name,) + time_vendor(kind, path, batch)[1:] for kind, name in VENDORS] if vendors else []
            config, ms, tflops = time_layer(binary, path, batch)
            log.write("%r\n" % (config,))
            for name, vms, vtf in others:
                log.write("%s: time = %.5fms, FLOPS = %.5fT\n" % (name, vms, vtf))
            log.write("%s: time = %.5fms, FLOPS = %.5fT\n%s\n\n" % (VENDOR, ms, tflops, "-" * 84))
            log.flush()
            rows.append((op, ms) if not vendors else (op, ms, [v[1] for v in others]))
    csv = os.path.join(log_dir, tag + ".csv")
    with open(csv, "w") as f:
        f.write(",op_name,%s%s\n" % ("".join(name + "," for _, name in VENDORS) if vendors else "", VENDOR))
        for i, row in enumerate(rows):
            f.write("%d,%s,%s%.5f\n" % (i, row[0], "".join("%.5f," % v for v in row[2]) if vendors else "", row[1]))
    return csv, rows


LADDER = [("baseline_test", "Baseline"), ("spf_test", "SPF"), ("bank_sr_test", "Bank-SR"),
          ("filter_gr_test", "Filter-GR"), ("para_test", "Para")]  # evalution/ablation_timing.py:109-115


def ablation_folder(bin_dir, folder, batch, log_dir):
    """One row per weight file, one column per rung of the ladder; -> (csv path, rows of (op, [ms per rung]))."""
    folder = folder.rstrip("/")
    os.makedirs(log_dir, exist_ok=True)
    rows = []
    with open(os.path.join(log_dir, "ablation_a.log"), "w") as log:
        for idx, op in enumerate(sorted(os.listdir(folder))):
            path = os.path.join(folder, op)
            if not os.path.isfile(path):
                continue
            log.write("# Run[%d]: %s\n" % (idx, path))
            times = []
            for k, (binary, name) in enumerate(LADDER):
                config, ms, tflops = time_layer(os.path.join(bin_dir, binary), path, batch)
                if k == 0:
                    log.write("%r\n" % (config,))
                log.write("%s: time = %.5fms\n" % (name, ms))
                times.append(ms)
            log.write("-" * 84 + "\n\n")
            log.flush()
            rows.append((op, times))
    csv = os.path.join(log_dir, "ablation_a.csv")
    with open(csv, "w") as f:
        f.write(",op_name,%s\n" % ",".join(name for _, name in LADDER))
        for i, (op, times) in enumerate(rows):
            f.write("%d,%s,%s\n" % (i, op, ",".join("%.5f" % t for t in times)))
    return csv, rows


def write_weight_file(path, w, H, W, pad, stride, groups=1):
    K, C, ks, _ = w.shape
    with open(path, "w") as f:
        f.write("%d %d %d %d %d %d %d %d\n" % (H, W, C, K, ks, pad, stride, groups))
        f.write(" ".join("%.9g" % v for v in w.reshape(-1).tolist()))
        f.write("\n")


def write_layers(layers, out_dir):
    from tetris_amd import workloads as W
    os.makedirs(out_dir, exist_ok=True)
    for L in layers:
        name = "%03d_%s_H_%d_W_%d_IC_%d_OC_%d_KS_%d_Pad_%d_S_%d_G_1" % (L.index, L.name.split("_H_")[0], L.H, L.W, L.C,
                                                                        L.K, L.ks, L.pad, L.stride)
        write_weight_file(os.path.join(out_dir, name), W.make_weights(L), L.H, L.W, L.pad, L.stride)
    return len(layers)


def main(argv=None):
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--weights", metavar="DIR", help="folder of weight files to time")
    ap.add_argument("--batch", nargs="+", type=int, default=[1])
    ap.add_argument("--log-dir", default="timing_out")
    ap.add_argument("--bin", default=os.path.join(here, "bin", "spconv2d_test"))
    ap.add_argument("--vendors", action="store_true", help="also time the vendor's dense convolution and CSR product per "
                    "layer (columns miopen, rocsparse: the reference's cudnn and cusparse columns)")
    ap.add_argument("--ablation", action="store_true", help="time the five binaries of the ablation ladder instead")
    ap.add_argument("--bin-dir", default=os.path.join(here, "bin"), help="where the ladder's binaries are (--ablation)")
    ap.add_argument("--write-suite", nargs=2, metavar=("SUITE", "DIR"))
    ap.add_argument("--write-masks", nargs=2, metavar=("NPZ", "DIR"))
    args = ap.parse_args(argv)
    if args.write_suite or args.write_masks:
        from tetris_amd import workloads as W
        layers = W.SUITES[args.write_suite[0]]() if args.write_suite else W.pruned_suite(args.write_masks[0])
        out_dir = (args.write_suite or args.write_masks)[1]
        print("wrote %d weight files to %s" % (write_layers(layers, out_dir), out_dir))
    if args.weights and args.ablation:
        missing = [b for b, _ in LADDER if not os.path.isfile(os.path.join(args.bin_dir, b))]
        if missing:
            sys.exit("timing: %s not built in %s (make -C %s)" % (", ".join(missing), args.bin_dir, here))
        for n in args.batch:
            log_dir = args.log_dir if len(args.batch) == 1 else os.path.join(args.log_dir, "batch_%d" % n)
            csv, rows = ablation_folder(args.bin_dir, args.weights, n, log_dir)
            sums = [sum(t[k] for _, t in rows) for k in range(len(LADDER))]
            print("batch %d: %d layers; %s -> %s" % (n, len(rows), ", ".join("%s %.3f ms" % (name, v) for (_, name), v in
                                                                          zip(LADDER, sums)), csv), flush=True)
    elif args.weights:
        if not os.path.isfile(args.bin):
            sys.exit("timing: %s is not built (make -C %s)" % (args.bin, here))
        for n in args.batch:
            csv, rows = time_folder(args.bin, args.weights, n, args.log_dir, vendors=args.vendors)
            print("batch %d: %d layers, %.3f ms in total -> %s" % (n, len(rows), sum(r[1] for r in rows), csv), flush=True)
            if args.vendors:
                for name, sp in geo_mean_speedups(rows):
                    print("# Compare to %s : Geo Mean Speedup = %.2fx" % (name, sp), flush=True)
    elif not (args.write_suite or args.write_masks):
        ap.error("nothing to do: give --weights, --write-suite or --write-masks")


if __name__ == "__main__":
    main()
