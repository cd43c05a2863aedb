"""Where a workgroup's time goes: per-layer breakdown from time stamps compiled into the conv kernels.

    make -C tetris-artifact-evalution_amd stamps            # builds build_stamps/libtetris_spconv2d.so (-DTETRIS_STAMPS)
    TETRIS_SPCONV2D_LIB=tetris-artifact-evalution_amd/build_stamps/libtetris_spconv2d.so \
        python -m tetris_amd.stamps --suite resnet50 --batch 16 [--worst 10 | --layers NAME ...] [--cold] [--waterfall]

Loads the stamped build of the library (not the product build: the stamps cost a few stores per workgroup), launches
every chosen layer with the library's tile and the balanced channel order, and prints one markdown row per layer:
the launch time by events, then the mean over the layer's workgroups of the phases wave 0 stamps (csrc/spconv2d_kernel.hip,
TETRIS_STAMP) in microseconds -- kernel arguments, staging plan and first stage's loads issued, stream offsets and first
batch, first stage landed and barrier, stage loop (with the share of it that the busiest wave, and the average wave,
spent inside the walk), output stores issued, stores acknowledged -- plus when the last workgroup entered and the
device span of the conv kernel (first entry to last exit; the rest of the launch time is the gap before the kernel
and, for a split layer, the kernel that adds the slices).
--worst N lists only the N layers furthest below their roof (the waterfall's `all` row stays over every layer).
--waterfall prints, per layer and for the whole selection, the chain of factors from the vector units' rate to the
measured time: FMA-only time at the measured shader clock -> x loop (cycles per entry over FMA cycles per entry) ->
x lanes (lanes that own pixels) -> x workgroup slots filled -> x share of the stage loop the busiest wave spends
walking (a SIMD works at the loop's rate while that wave walks) -> x stage loop's share of the kernel
-> x kernel's share of the launch.  The stamped build reads the clock around every walk call, which makes a pass
some 2 % longer than the product build's.  Every layer is launched for about 30 ms before it is timed, so that the
shader clock is where a whole pass holds it.
"""
import argparse
import ctypes as C
import sys

import numpy as np

import tetris_amd as T
from tetris_amd import workloads as W

SLOTS, MAX_WGS = 16, 8192
# shader cycles of a SIMD per entry at four / two waves per SIMD, measured on the loop alone in a kernel that runs long
# enough for the clock to settle near the nominal 2.4 GHz its time is divided by (quads -> cycles); an entry's FMAs
# alone take 16 cycles per quad
LOOP_CYCLES = {True: {1: 26.2, 2: 43.5}, False: {1: 30.0, 2: 50.0, 4: 85.2}}


def read_stamps():
    buf = np.zeros((MAX_WGS, SLOTS), np.int64)
    fn = T._lib.tetris_stamps_read
    fn.argtypes = [C.c_void_p, C.c_int]
    T._check(fn(buf.ctypes.data_as(C.c_void_p), MAX_WGS))
    return buf[buf[:, 0] != 0]


def breakdown(torch, L, batch, cold):
    w, x = W.make_weights(L), W.make_activations(L, batch)
    tile = T.tile_select(batch, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    shape = pk.launch_shape(batch, L.H, L.W, L.stride, L.pad, tile)
    oh, ow = W.out_hw(L)
    dx = torch.from_numpy(x).cuda()
    dy = torch.empty((batch, L.K, oh, ow), device="cuda")
    args = (dx.data_ptr(), dy.data_ptr(), batch, L.H, L.W, L.stride, L.pad, tile)
    # The shader clock idles at about 2.1 GHz and takes 10-25 ms of unbroken work to reach the 2.3-2.4 GHz that a
    # whole pass runs at: launch some 30 ms' worth before the timed launches; the stamped launch follows at once (the
    # clock does not fall back during the fraction of a millisecond that clearing the stamps takes).
    ms = pk.time(*args, warm=2, repeat=5)
    ms = pk.time(*args, warm=max(5, min(3000, int(30.0 / ms))), repeat=20)
    read_stamps()  # clears what the timed launches left (the walk's cycle counts add up from launch to launch)
    if cold:
        torch.empty(128 << 20, dtype=torch.float32, device="cuda").fill_(1.0)  # 512 MiB: evicts the caches
        torch.cuda.synchronize()
    pk.launch(*args)
    s = read_stamps().astype(np.float64)
    nnz = pk.host_arrays()["nnz"]
    pk.close()
    mhz = 100.0 * float((s[:, 7] - s[:, 0]).sum()) / max(float((s[:, 10] - s[:, 9]).sum()), 1.0)  # shader clock in MHz (cycles per 100 MHz tick x 100)
    us = lambda a: float(np.mean(a)) / mhz  # noqa: E731
    loop = s[:, 5] - s[:, 4]
    four = tile.waves == 16 or (tile.waves == 8 and tile.oc_per_wave * 4 * tile.quads <= 64 and tile.quads <= 2)
    # workgroups the 256 CUs hold at once: one of 16 waves, or of 8 waves with 128 accumulators; else two (by LDS)
    slots = 256 * (1 if tile.waves == 16 or (tile.waves == 8 and not four) else 2)
    rounds = -(-shape.workgroups // slots)
    wk = W.work(L, batch)
    lanes = shape.lanes_used / 64.0
    if tile.lanes_w == 64:  # flat tile: 64 consecutive quads of the batch per unit, the last unit of the batch part empty
        quads = batch * -(-(oh * ow) // 4)
        lanes = quads / (64.0 * -(-quads // 64))
    loop_cycles = LOOP_CYCLES[four].get(tile.quads, 16.0 * tile.quads)
    # entries a SIMD walks in the stage loop: a workgroup's share of the non-zeros, a quarter of it per SIMD, times the
    # workgroups that share the CU
    simd_entries = nnz / float(shape.channel_blocks * shape.csplit) / 4.0 * (slots // 256)
    return {"layer": L.name, "tile": tile.as_list(), "wgs": len(s), "launch_us": ms * 1e3, "csplit": shape.csplit,
            "args": us(s[:, 1] - s[:, 0]), "issued": us(s[:, 2] - s[:, 1]), "head": us(s[:, 3] - s[:, 2]),
            "landed": us(s[:, 4] - s[:, 3]), "loop": us(loop),
            "walk_max": float(s[:, 12].sum() / max(loop.sum(), 1.0)),
            "walk_mean": float(s[:, 13].sum() / tile.waves / max(loop.sum(), 1.0)),
            "stores": us(s[:, 6] - s[:, 5]), "acked": us(s[:, 7] - s[:, 6]),
            "last_entry": float(s[:, 9].max() - s[:, 9].min()) / 100.0, "span": float(s[:, 10].max() - s[:, 9].min()) / 100.0,
            "kernel": us(s[:, 7] - s[:, 0]), "mhz": mhz, "roof_us": wk["t_roof"] * 1e6, "flops": wk["flops_sparse"],
            "lanes": lanes, "fill": shape.workgroups / float(rounds * slots), "rounds": rounds,
            "loop_eff": 16.0 * tile.quads / loop_cycles, "loop_cycles": loop_cycles,
            # what the SIMD spends per entry if it is busy whenever the busiest wave walks: to set beside loop_cycles
            "seen_cycles": float(np.mean(loop)) * float(s[:, 12].sum() / max(loop.sum(), 1.0)) / max(simd_entries, 1.0)}


def waterfall(rows, shown):
    """Per layer (those of `shown`) and in total (all of `rows`): the time the FMAs alone would take on 256 CUs x 4 SIMDs
    x 16 lanes at the measured clock, and the factors that lead from there to the measured launch time."""
    print("\n| layer | FMA-only us | loop | lanes | slots filled | busiest wave walking | stage loop / kernel | kernel / "
          "launch | product | measured us | FMA-only / measured | SIMD cycles per entry while the busiest wave walks (loop alone) |")
    print("|" + "---|" * 12)
    tot = dict(ideal=0.0, meas=0.0)
    acc = {k: 0.0 for k in ("loop_eff", "lanes", "fill", "walk_max", "loop_share", "kern_share")}
    for r in rows:
        ideal = r["flops"] / 2.0 / (256 * 4 * 16) / r["mhz"]  # FMAs / (lanes of the GPU) / MHz = microseconds
        loop_share = r["loop"] / r["kernel"]
        # one round of workgroups: the launch is a workgroup's life plus what lies around the kernel; several rounds: a
        # CU starts its next workgroup as one ends, the launch is the sum of lives (the idle slots are under "filled")
        kern_share = min(1.0, r["rounds"] * r["kernel"] / r["launch_us"])
        prod = r["loop_eff"] * r["lanes"] * r["fill"] * r["walk_max"] * loop_share * kern_share
        if any(r is x for x in shown):
            print("| %s | %.1f | %.2f | %.2f | %.2f | %.2f | %.2f | %.2f | %.3f | %.1f | %.3f | %.1f (%.1f) |" % (
                r["layer"], ideal, r["loop_eff"], r["lanes"], r["fill"], r["walk_max"], loop_share, kern_share, prod,
                r["launch_us"], ideal / r["launch_us"], r["seen_cycles"], r["loop_cycles"]))
        tot["ideal"] += ideal
        tot["meas"] += r["launch_us"]
        for k, v in (("loop_eff", r["loop_eff"]), ("lanes", r["lanes"]), ("fill", r["fill"]), ("walk_max", r["walk_max"]),
                     ("loop_share", loop_share), ("kern_share", kern_share)):
            acc[k] += v * r["launch_us"]  # weighted by where the time is spent
    w = {k: v / tot["meas"] for k, v in acc.items()}
    print("| all (time-weighted) | %.1f | %.2f | %.2f | %.2f | %.2f | %.2f | %.2f | %.3f | %.1f | %.3f | |" % (
        tot["ideal"], w["loop_eff"], w["lanes"], w["fill"], w["walk_max"], w["loop_share"], w["kern_share"],
        w["loop_eff"] * w["lanes"] * w["fill"] * w["walk_max"] * w["loop_share"] * w["kern_share"], tot["meas"],
        tot["ideal"] / tot["meas"]))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--suite", default="vgg19")
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--layers", nargs="*", help="layer names (substrings); default: all")
    ap.add_argument("--worst", type=int, default=0, help="list only the N layers furthest below their roof")
    ap.add_argument("--cold", action="store_true", help="evict the caches before the stamped launch")
    ap.add_argument("--waterfall", action="store_true", help="also print the chain of factors from the FMA rate to the time")
    args = ap.parse_args()
    import torch

    if not hasattr(T._lib, "tetris_stamps_read"):
        sys.exit("stamps.py: %s has no stamps compiled in: make -C tetris-artifact-evalution_amd stamps, then set "
                 "TETRIS_SPCONV2D_LIB to build_stamps/libtetris_spconv2d.so" % T.LIB_PATH)
    layers = [L for L in W.SUITES[args.suite]() if not args.layers or any(n in L.name for n in args.layers)]
    rows = [breakdown(torch, L, args.batch, args.cold) for L in layers]
    shown = sorted(rows, key=lambda r: r["roof_us"] / r["launch_us"])[:args.worst] if args.worst else rows
    print("%s at batch %d%s; shader clock %.0f MHz; microseconds, mean over a layer's workgroups\n" %
          (args.suite, args.batch, ", caches evicted before the stamped launch" if args.cold else "",
           float(np.mean([r["mhz"] for r in rows]))))
    print("| layer | tile | workgroups (slices per tile) | launch (events) | fraction of roof | arguments | plan + first "
          "stage issued | offsets + first batch | first stage landed + barrier | stage loop (walking: busiest wave, mean "
          "wave) | stores issued | stores acknowledged | last workgroup enters after | conv kernel span |")
    print("|" + "---|" * 14)
    for r in shown:
        print("| %s | %s | %d (%d) | %.1f | %.3f | %.2f | %.2f | %.2f | %.2f | %.1f (%.2f, %.2f) | %.2f | %.2f | %.2f | %.1f |" % (
            r["layer"], r["tile"], r["wgs"], r["csplit"], r["launch_us"], r["roof_us"] / r["launch_us"], r["args"],
            r["issued"], r["head"], r["landed"], r["loop"], r["walk_max"], r["walk_mean"], r["stores"], r["acked"],
            r["last_entry"], r["span"]))
    if args.waterfall:
        waterfall(rows, shown)


if __name__ == "__main__":
    main()
