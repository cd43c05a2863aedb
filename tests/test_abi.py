"""CPU-side checks of the shipped library: it loads, exports what include/tetris_spconv2d.h declares,
rejects bad arguments with a message, and its host packer equals the oracle byte for byte."""
import ctypes
import os
import re

import numpy as np
import pytest

from conftest import GOLDEN, ROOT, golden_weights
from helpers import sparse_filter

T = pytest.importorskip("tetris_amd")


def test_every_declared_symbol_is_exported():
    hdr = open(os.path.join(ROOT, "include", "tetris_spconv2d.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    names = set(re.findall(r"\b(tetris_[a-z0-9_]+)\s*\(", hdr))
    assert len(names) >= 20
    lib = ctypes.CDLL(T.LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing


def test_version_and_errors():
    assert "gfx950" in T.version()
    w = np.zeros((4, 4, 9, 9), np.float32)
    with pytest.raises(T.TetrisError) as e:
        T.SparseFilter(w, 4, 4, 9)  # 3-bit row/column fields: kernel_size <= 7
    assert e.value.code == T.EINVAL and "ks" in str(e.value)
    with pytest.raises(T.TetrisError) as e:
        T.ReadConfigAndDataFromFile("/nonexistent/weights")
    assert e.value.code == T.EIO and "Open file error" in str(e.value)


CASES = [(40, 20, 3, 8, 0.8), (64, 48, 1, 32, 0.7), (33, 7, 3, 32, 0.5), (70, 70, 1, 32, 0.9), (16, 3, 7, 32, 0.85),
         (96, 40, 3, 16, 0.95), (8, 64, 3, 64, 0.9), (255, 64, 1, 128, 0.75)]
MODES = [(0, 1, 0), (1, 0, 0), (1, 1, 0), (1, 1, T.BANK_OPTIMIZE), (1, 1, T.REORDER_OUT_CHANNEL),
         (1, 1, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL), (1, 0, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL)]


@pytest.mark.parametrize("case", CASES)
def test_sparse_filter_equals_oracle_bytes(oracle, case):
    K, C, ks, tic, sp = case
    w = sparse_filter(np.random.default_rng(K * 1000 + C + ks), K, C, ks, sp)
    for reorder, vec, flags in MODES:
        o = oracle.SpfPack(w, tic, bool(reorder), bool(vec), bool(flags & 1), bool(flags & 2))
        assert o.bank_oob == 0
        p = T.SparseFilter(w, C, K, ks, tic, bool(reorder), bool(vec), flags)
        for a, b in zip(o.arrays(), p.arrays()):
            assert a.dtype == b.dtype and a.tobytes() == b.tobytes()
        assert p.nnz_ == o.nnz_counted and p.GetTileIC() == tic
        p.close()


@pytest.mark.parametrize("name", ["rn90_3x3", "rn90_stem", "rn98_1x1", "vgg_64x128", "yolo_255"])
def test_sparse_filter_on_shipped_layers(oracle, name):
    import json
    rows = [r for r in json.load(open(os.path.join(GOLDEN, "spf_known_answers.json")))["rows"] if r["layer"] == name]
    hdr, w, _ = golden_weights(name)
    for r in rows:
        flags = (T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL) if r["flags"] == "BR" else 0
        p = T.SparseFilter(w, hdr["IC"], hdr["OC"], hdr["KS"], r["tile_ic"], True, True, flags)
        assert "%016x" % oracle.fnv1a(*p.arrays()) == r["fnv_all"]
        assert "%016x" % oracle.fnv1a(p.oc_permutation_) == r["fnv_perm"]
        p.close()


def test_reader_and_tolerance_match_oracle(oracle, tmp_path):
    vals = np.array([0.0, -0.0, 1.5, -2.25e-3, 7, 1e-8, 0.0, 3.25], np.float32)
    p = tmp_path / "w.txt"
    p.write_text("5 6 2 4 1 0 1 1\n" + " ".join(repr(float(v)) for v in vals) + "\n")
    hdr, w, nnz = T.ReadConfigAndDataFromFile(str(p))
    hdr_o, w_o, nnz_o = oracle.read_weight_file(str(p))
    assert hdr == hdr_o and nnz == nnz_o == 5 and w.tobytes() == w_o.tobytes()
    (tmp_path / "short.txt").write_text("5 6 2 4 1 0 1 1\n0.5 0.25\n")
    with pytest.raises(T.TetrisError) as e:
        T.ReadConfigAndDataFromFile(str(tmp_path / "short.txt"))
    assert e.value.code == T.EIO
    for a, b in [(0.0, 1e-5), (0.0, 1.01e-5), (1.0, 1.00003), (1.0, 1.00002), (1e6, 1e6 + 25), (1.0, -1.0)]:
        assert T.FloatEqual(a, b) == oracle.float_equal(a, b)
    x = np.arange(8, dtype=np.float32)
    assert T.TensorEqual(x, x.copy()) and not T.TensorEqual(x, x + 1)


def test_tile_select_is_sane():
    for shape in [(1, 56, 56, 64, 128, 3, 1, 1), (16, 224, 224, 3, 64, 3, 1, 1), (16, 7, 7, 1024, 1024, 1, 1, 0),
                  (4, 224, 224, 3, 64, 7, 2, 3), (16, 13, 13, 1024, 255, 1, 1, 0), (1, 14, 14, 512, 512, 3, 1, 1)]:
        t = T.tile_select(*shape)
        flat = t.lanes_w == 64  # flat tiles: pointwise layers only, 8 or 16 waves
        assert (1 <= t.lanes_w <= 62 or (flat and shape[5:] == (1, 1, 0) and t.waves in (8, 16)))
        assert t.quads in (1, 2, 4) and t.oc_per_wave in (1, 2, 4, 8, 16, 32)
        assert t.oc_per_wave * 4 * t.quads <= (64 if t.waves == 16 else 128) and t.waves in (1, 2, 4, 8, 16) and t.tile_ic >= 1
    with pytest.raises(T.TetrisError):
        T.tile_select(0, 5, 5, 3, 3, 3, 1, 1)


def test_tile_select_answers_from_the_measured_table():
    # shapes of the benchmark suites are answered from csrc/tuned_tiles.inc (as long as the kernel accepts the entry)
    import re

    import tetris_amd as T
    from conftest import ROOT

    rows = {}
    with open(os.path.join(ROOT, "tetris-artifact-evalution_amd", "csrc", "tuned_tiles.inc")) as f:
        for line in f:
            m = re.match(r"\s*\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), \{(\d+), (\d+), (\d+), (\d+), (\d+)\}\}", line)
            if m:
                v = [int(x) for x in m.groups()]
                rows.setdefault(tuple(v[:8]), tuple(v[8:]))  # the first entry of a shape wins, as in the library
    assert len(rows) >= 100
    hits = 0
    for key, tile in list(rows.items())[::7]:
        n, h, w, c, k, ks, stride, pad = key
        t = T.tile_select(n, h, w, c, k, ks, stride, pad)
        got = (t.lanes_w, t.quads, t.oc_per_wave, t.waves, t.tile_ic)
        hits += got == tile
    assert hits >= len(list(rows.items())[::7]) - 2  # an entry the current geometry checks refuse falls back to the model


def _busiest_wave_cost(w, order, g, waves, tile_ic):
    """Sum over workgroup blocks and input-channel stages of the busiest wave's entry count (what the waves of a
    workgroup wait for at their per-stage barrier), and the per-block sums."""
    K, C = w.shape[:2]
    stages = -(-C // tile_ic)
    per = np.zeros((K, stages), np.int64)
    for s in range(stages):
        per[:, s] = (w[:, s * tile_ic:(s + 1) * tile_ic] != 0).reshape(K, -1).sum(1)
    block = g * waves
    padded = np.zeros((-(-K // block) * block, stages), np.int64)
    padded[:K] = per[order]
    by_block = padded.reshape(-1, waves, g, stages).sum(2).max(1).sum(1)
    return int(by_block.sum()), by_block


@pytest.mark.parametrize("K,C,ks,g,waves,tile_ic", [(128, 64, 3, 4, 16, 16), (255, 96, 1, 8, 8, 32), (64, 48, 3, 8, 8, 64),
                                                   (40, 24, 3, 16, 2, 8), (7, 5, 7, 4, 4, 3)])
def test_balanced_order_is_a_permutation_that_lowers_the_busiest_wave(K, C, ks, g, waves, tile_ic):
    rng = np.random.default_rng(K + C)
    # channels of very different density, some empty, as pruned networks have
    density = np.clip(rng.lognormal(np.log(0.12), 0.8, K), 0, 0.9)
    density[rng.random(K) < 0.1] = 0
    w = (rng.standard_normal((K, C, ks, ks)) * (rng.random((K, C, ks, ks)) < density[:, None, None, None])).astype(np.float32)
    tile = T.Tile(7, 2, g, waves, tile_ic)
    order = T.oc_order_balanced(w, tile)
    assert order.dtype == np.int32 and sorted(order.tolist()) == list(range(K))
    ident, _ = _busiest_wave_cost(w, np.arange(K), g, waves, tile_ic)
    bal, by_block = _busiest_wave_cost(w, order, g, waves, tile_ic)
    assert bal <= ident
    if K >= 4 * g * waves // 2 and K % (g * waves) == 0:
        assert bal <= 0.92 * ident                      # a clear gain on skewed channels
        assert by_block.max() <= 1.1 * by_block.mean()  # and no straggler workgroup
    assert np.array_equal(order, T.oc_order_balanced(w, tile))  # deterministic


def test_balanced_order_on_a_shipped_pruned_layer():
    hdr, w, _ = golden_weights("vgg_64x128")  # 64 -> 128 channels, 3x3, 85 % pruned: 7 .. 165 non-zeros per channel
    for g, waves, tile_ic in [(4, 16, 16), (8, 8, 32)]:
        order = T.oc_order_balanced(w, T.Tile(14, 2, g, waves, tile_ic))
        ident, _ = _busiest_wave_cost(w, np.arange(128), g, waves, tile_ic)
        bal, _ = _busiest_wave_cost(w, order, g, waves, tile_ic)
        assert bal <= 0.88 * ident


def test_balanced_order_rejects_bad_arguments():
    w = np.ones((8, 8, 1, 1), np.float32)
    with pytest.raises(T.TetrisError):
        T.oc_order_balanced(w, T.Tile(7, 2, 0, 8, 8))


@pytest.mark.parametrize("masks,count", [("masks_vgg19_92.npz", 8), ("masks_mobilenet_86.npz", 13),
                                         ("masks_resnet50_90.npz", 44), ("masks_resnet50_98.npz", 44),
                                         ("masks_yolov3_89.npz", 55)])
def test_pruned_suites_load_and_balance(masks, count):
    from tetris_amd import workloads as W

    layers = W.pruned_suite(os.path.join(GOLDEN, masks))
    assert len(layers) == count
    gains = []
    for L in layers:
        assert L.mask.shape == (L.K, L.C, L.ks, L.ks) and ("IC_%d_OC_%d_KS_%d" % (L.C, L.K, L.ks)) in L.name
        assert abs((1.0 - L.sparsity) * L.mask.size - W.nnz_of(L)) < 0.5
        if L.C < 16:
            continue
        w = W.make_weights(L)
        assert np.array_equal(w != 0, L.mask)
        tile = T.tile_select(16, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
        order = T.oc_order_balanced(w, tile)
        ident, _ = _busiest_wave_cost(w, np.arange(L.K), tile.oc_per_wave, tile.waves, tile.tile_ic)
        bal, _ = _busiest_wave_cost(w, order, tile.oc_per_wave, tile.waves, tile.tile_ic)
        gains.append(bal / ident)
    assert max(gains) <= 1.0 and np.mean(gains) <= 0.93, gains


def test_host_packer_on_negative_zeros_and_denormals(oracle):
    # `value != 0.f` (Tetris/spconv2d_utils.h:47, :87): -0.0 is dropped, a denormal is kept -- in all four flag sets
    rng = np.random.default_rng(17)
    w = sparse_filter(rng, 40, 24, 3, 0.7, neg_zero=True)
    flat = w.reshape(-1)
    nz = np.flatnonzero(flat)
    flat[nz[::4]] = np.float32(1e-40)
    flat[nz[1::4]] = np.float32(-1.4e-45)
    assert np.signbit(flat[flat == 0]).any()
    for flags in (0, 1, 2, 3):
        sf = T.SparseFilter(w, 24, 40, 3, 16, True, True, flags)
        ref = oracle.SpfPack(w, 16, True, True, bool(flags & 1), bool(flags & 2))
        assert sf.values_.tobytes() == ref.values.tobytes() and np.array_equal(sf.position_, ref.position)
        assert int((sf.values_ != 0).sum()) == int((w != 0).sum())            # every denormal packed, no zero packed
        assert not (sf.values_.view(np.uint32) == 0x80000000).any()           # -0.0 never stored
        sf.close()
    sf = T.SparseFilter(w, 24, 40, 3, 16, False, True, 0)
    assert sf.nnz_ == int((w != 0).sum())
    sf.close()


def test_offsets_check_of_the_raw_launchers(oracle):
    # What the raw launchers verify on a host copy of offsets_ before any kernel reads the arrays
    # (Tetris/spconv2d_utils.h:45-47, 209-216: starts at 0, never decreases, steps of the vector width)
    rng = np.random.default_rng(5)
    w = sparse_filter(rng, 70, 40, 3, 0.8)
    for vec, args in [(4, (True, True, True, True)), (1, (True, False, True, True)), (0, (False,))]:
        p = oracle.SpfPack(w, 16, *args)
        off, n_ent = p.offsets, len(p.values)
        T.spf_check_offsets(off, vec, n_ent)
        T.spf_check_offsets(off, vec, 0)  # capacity not known
        for bad, cap in [(off, n_ent - 1), (off[::-1], n_ent), (off + 1, n_ent), (-off, n_ent)]:
            with pytest.raises(T.TetrisError) as e:
                T.spf_check_offsets(bad, vec, cap)
            assert e.value.code == T.EINVAL
    p = oracle.SpfPack(w, 16, True, True, True, True)
    odd = p.offsets.copy()
    odd[1:] += 2
    with pytest.raises(T.TetrisError):
        T.spf_check_offsets(odd, 4, 0)
    T.spf_check_offsets(odd - np.where(np.arange(len(odd)) > 0, 2, 0), 4, 0)
    with pytest.raises(T.TetrisError):
        T.spf_check_offsets(p.offsets, 3, 0)  # no such vector width


def test_tile_table_loaded_at_run_time_wins_over_the_built_in_one(tmp_path):
    shape = (3, 37, 41, 24, 40, 3, 1, 1)  # in no built-in table
    model = T.tile_select(*shape)
    want = (5, 1, 8, 2, 8)
    assert (model.lanes_w, model.quads, model.oc_per_wave, model.waves, model.tile_ic) != want
    table = tmp_path / "tiles.inc"
    table.write_text("// Generated elsewhere\n"
                     "    {3, 37, 41, 24, 40, 3, 1, 1, {5, 1, 8, 2, 8}},  // mine: 12.3 us\n"
                     "    {3, 38, 41, 24, 40, 3, 1, 1, {62, 4, 32, 16, 4096}},  // a tile the kernel refuses\n"
                     "not a row\n")
    assert T.tile_table_load(str(table)) == 2
    t = T.tile_select(*shape)
    assert (t.lanes_w, t.quads, t.oc_per_wave, t.waves, t.tile_ic) == want
    bad = T.tile_select(3, 38, 41, 24, 40, 3, 1, 1)  # refused row: falls through to the model
    assert (bad.lanes_w, bad.quads, bad.oc_per_wave, bad.waves, bad.tile_ic) != (62, 4, 32, 16, 4096)
    with pytest.raises(T.TetrisError) as e:
        T.tile_table_load(str(tmp_path / "missing"))
    assert e.value.code == T.EIO


def test_tile_select_borrows_from_the_nearest_measured_layer():
    # a VGG19 layer shape at a batch size the table does not hold gets a measured neighbour's tile, not the cycle model's
    t6 = T.tile_select(6, 56, 56, 256, 256, 3, 1, 1)
    near = [T.tile_select(n, 56, 56, 256, 256, 3, 1, 1) for n in (4, 8)]
    as_tuple = lambda t: (t.lanes_w, t.quads, t.oc_per_wave, t.waves, t.tile_ic)
    assert as_tuple(t6) in [as_tuple(t) for t in near]
    # the neighbour's lane count is refitted to the image width: a 52-wide layer is not given 14 lanes (two units per row)
    t52 = T.tile_select(16, 52, 52, 256, 256, 3, 1, 1)
    t50 = T.tile_select(16, 50, 50, 256, 256, 3, 1, 1)
    assert -(-50 // (4 * t50.lanes_w)) == -(-52 // (4 * t52.lanes_w)) and 4 * t50.lanes_w - 50 < 4
    # a kernel size no measured layer has falls through to the model and still gets a launchable tile
    t5 = T.tile_select(2, 20, 20, 32, 32, 5, 1, 2)
    assert t5.lanes_w >= 1 and t5.waves in (1, 2, 4, 8, 16)
