"""LDS bank-conflict counters of the conv kernel with and without its conflict-avoidance rule, per layer: the
counterpart of the reference's evalution/script/memory_metric.sh (which runs `ncu --metrics group:memory__chart` on
wo_bank_sr_test.o and wi_bank_sr_test.o for every weight file of a folder, :9-16) and of the checks and ratios
evalution/draw_ablation_b.py:36-41 makes on those files.

    python -m tetris_amd.memory_metric --weights DIR [--batch 4] [--out DIR] [--bin-dir DIR]

For every weight file it starts

    rocprofv3 --pmc SQ_INSTS_LDS SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE --output-format csv -d OUT/<variant>/<file> --
        bin/<variant>_bank_sr_test <file> <batch>

for <variant> = wo, wi (the driver is the program after `--`; nothing else sits between the profiler and it), sums
the counters over the conv kernel's dispatches and writes OUT/memory_metric.csv with one row per layer:
LDS instructions (the reference's "requests"), cycles the LDS spent on bank conflicts and cycles it was busy, each
without and with the rule, and the two conflict rates.  As in the reference's plot script, a layer whose binaries
disagree on the work done is reported: here the rule may pick another lane arrangement for a tile, which changes the
LDS instruction count by the share of idle lane positions, so the counts are printed, not required to be equal.
"""
import argparse
import csv
import glob
import os
import subprocess
import sys

COUNTERS = ["SQ_INSTS_LDS", "SQ_LDS_BANK_CONFLICT", "SQ_LDS_IDX_ACTIVE"]
VARIANTS = [("wo", "wo_bank_sr_test"), ("wi", "wi_bank_sr_test")]  # evalution/script/build_ablation.sh:17-18


def conv_counter_sums(directory):
    """Sum of every counter over the dispatches of the conv kernels in a rocprofv3 output folder."""
    files = glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True)
    if not files:
        raise RuntimeError("no counter_collection.csv under %s" % directory)
    sums = dict.fromkeys(COUNTERS, 0.0)
    dispatches = set()
    for path in files:
        with open(path) as f:
            for r in csv.DictReader(f):
                if "spconv2d_" in r["Kernel_Name"] and r["Counter_Name"] in sums:
                    sums[r["Counter_Name"]] += float(r["Counter_Value"])
                    dispatches.add((path, r["Dispatch_Id"]))
    sums["dispatches"] = len(dispatches)
    return sums


def profile_layer(bin_dir, weight_file, batch, out_dir, timeout=600):
    """Runs both binaries on one weight file under the profiler; -> {variant: counter sums}."""
    res = {}
    for variant, binary in VARIANTS:
        d = os.path.join(out_dir, variant, os.path.basename(weight_file))
        os.makedirs(d, exist_ok=True)
        cmd = ["rocprofv3", "--pmc"] + COUNTERS + ["--output-format", "csv", "-d", d, "--",
                                                   os.path.join(bin_dir, binary), weight_file, str(batch)]
        p = subprocess.run(cmd, capture_output=True, text=True, timeout=timeout)
        if p.returncode != 0:
            raise RuntimeError("%s: exit %d\n%s%s" % (" ".join(cmd), p.returncode, p.stdout[-2000:], p.stderr[-2000:]))
        res[variant] = conv_counter_sums(d)
    return res


def write_table(path, rows):
    with open(path, "w") as f:
        f.write(",op_name,lds_insts_wo,lds_insts_wi,conflict_cycles_wo,conflict_cycles_wi,busy_cycles_wo,busy_cycles_wi,"
                "conflict_rate_wo,conflict_rate_wi\n")
        for i, (op, r) in enumerate(rows):
            wo, wi = r["wo"], r["wi"]
            rate = [v["SQ_LDS_BANK_CONFLICT"] / v["SQ_LDS_IDX_ACTIVE"] if v["SQ_LDS_IDX_ACTIVE"] else 0.0 for v in (wo, wi)]
            f.write("%d,%s,%d,%d,%d,%d,%d,%d,%.4f,%.4f\n" % (
                i, op, wo["SQ_INSTS_LDS"], wi["SQ_INSTS_LDS"], wo["SQ_LDS_BANK_CONFLICT"], wi["SQ_LDS_BANK_CONFLICT"],
                wo["SQ_LDS_IDX_ACTIVE"], wi["SQ_LDS_IDX_ACTIVE"], rate[0], rate[1]))


def main(argv=None):
    here = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--weights", metavar="DIR", required=True, help="folder of weight files")
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--out", default="memory_metric_out")
    ap.add_argument("--bin-dir", default=os.path.join(here, "bin"))
    args = ap.parse_args(argv)
    missing = [b for _, b in VARIANTS if not os.path.isfile(os.path.join(args.bin_dir, b))]
    if missing:
        sys.exit("memory_metric: %s not built in %s (make -C %s)" % (", ".join(missing), args.bin_dir, here))
    rows = []
    for op in sorted(os.listdir(args.weights)):
        path = os.path.join(args.weights, op)
        if not os.path.isfile(path):
            continue
        r = profile_layer(args.bin_dir, path, args.batch, args.out)
        rows.append((op, r))
        wo, wi = r["wo"], r["wi"]
        note = "" if wo["SQ_INSTS_LDS"] == wi["SQ_INSTS_LDS"] else "  (LDS instruction counts differ)"
        print("%s: conflict cycles %d -> %d of %d -> %d busy%s" % (op, wo["SQ_LDS_BANK_CONFLICT"], wi["SQ_LDS_BANK_CONFLICT"],
                                                                   wo["SQ_LDS_IDX_ACTIVE"], wi["SQ_LDS_IDX_ACTIVE"], note),
              flush=True)
    table = os.path.join(args.out, "memory_metric.csv")
    write_table(table, rows)
    print("%d layers -> %s" % (len(rows), table))


if __name__ == "__main__":
    main()
