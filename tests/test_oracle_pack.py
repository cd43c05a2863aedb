"""Pins the oracle's restatement of the reference SparseFilter constructor (spconv2d_utils.h:25-246,
:275-420) and of its two host decoders (:422-493)."""
import json
import os
from collections import Counter

import numpy as np
import pytest

from conftest import GOLDEN, REFERENCE, golden_weights
from helpers import relu_like, sparse_filter

KAT = json.load(open(os.path.join(GOLDEN, "spf_known_answers.json")))["rows"]
BIG = {
    "yolo_1024": "yolov3/yolov3-89-acc-62.4/module74_0_module5_0_conv2d_0_H_20_W_20_IC_1024_OC_512_KS_1_Pad_0_S_1_G_1",
    "vgg_256": "vgg19/vgg19-92-acc-71.7/module8_0_module2_0_conv2d_3_H_56_W_56_IC_256_OC_256_KS_3_Pad_1_S_1_G_1",
}
_cache = {}


def layer(oracle, name):
    if name not in _cache:
        if name in BIG:
            path = os.path.join(REFERENCE, "evalution", "conv_weight_data", BIG[name])
            if not os.path.exists(path):
                pytest.skip("large layer only in the reference checkout")
            _cache[name] = oracle.read_weight_file(path)[1]
        else:
            _cache[name] = golden_weights(name)[1]
    return _cache[name]


@pytest.mark.parametrize("row", KAT, ids=lambda r: "%s-%s-%d" % (r["flags"], r["layer"], r["tile_ic"]))
def test_known_answers_from_compiled_reference(oracle, row):
    w = layer(oracle, row["layer"])
    br = row["flags"] == "BR"
    p = oracle.SpfPack(w, row["tile_ic"], True, True, bank_optimize=br, reorder_out_channel=br)
    assert p.bank_oob == 0
    assert (len(p.offsets), len(p.stage_len), len(p.position), int(p.offsets[-1])) == (
        row["n_offsets"], row["n_stage_len"], row["n_entries"], row["offsets_back"])
    assert int((w != 0).sum()) == row["nnz"]
    assert "%016x" % oracle.fnv1a(p.perm) == row["fnv_perm"]
    assert "%016x" % oracle.fnv1a(p.position) == row["fnv_position"]
    assert "%016x" % oracle.fnv1a(*p.arrays()) == row["fnv_all"]


def decode_spf(p, vec):
    """-> Counter of (k, c, r, s, value-bits) over non-pad entries, reading the arrays the way the reference
    kernel indexes them (spconv2d_kernel.cu:91-105)."""
    out = Counter()
    S, T = p.stages, p.tile_ic
    for slot in range(p.K):
        g, lane = divmod(slot, 32)
        for st in range(S):
            start = int(p.offsets[g * S + st])
            n = int(p.offsets[g * S + st + 1]) - start
            for e in range(n):
                at = 32 * start + (e // vec) * 32 * vec + lane * vec + e % vec
                v = p.values[at]
                if v == 0:
                    continue
                pos = int(p.position[at])
                out[(int(p.perm[slot]), (pos >> 6) + st * T, (pos >> 3) & 7, pos & 7, v.tobytes())] += 1
    return out


def filter_nonzeros(w):
    out = Counter()
    for k, c, r, s in zip(*np.nonzero(w)):
        out[(int(k), int(c), int(r), int(s), w[k, c, r, s].tobytes())] += 1
    return out


CASES = [  # K, C, ks, tile_ic, sparsity
    (40, 20, 3, 8, 0.8), (64, 48, 1, 32, 0.7), (33, 7, 3, 32, 0.5), (70, 70, 1, 32, 0.9), (16, 3, 7, 32, 0.85),
    (96, 40, 3, 16, 0.95), (8, 64, 3, 64, 0.9),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("bank,reoc,vec", [(0, 0, 1), (0, 0, 4), (1, 0, 4), (0, 1, 4), (1, 1, 4), (1, 1, 1)])
def test_spf_invariants(oracle, case, bank, reoc, vec):
    K, C, ks, T, sp = case
    rng = np.random.default_rng(K * 1000 + C + ks)
    w = sparse_filter(rng, K, C, ks, sp)
    p = oracle.SpfPack(w, T, True, vec == 4, bool(bank), bool(reoc))
    S, G = p.stages, (K + 31) // 32
    assert p.bank_oob == 0
    assert S == (C - 1) // T + 1
    assert len(p.offsets) == G * S + 1 and p.offsets[0] == 0
    d = np.diff(p.offsets)
    assert (d >= 0).all() and (d % vec == 0).all()
    assert len(p.values) == len(p.position) == 32 * p.offsets[-1]
    assert sorted(p.perm.tolist()) == list(range(K))
    if not reoc:
        assert p.perm.tolist() == list(range(K))
    # Bank-SR pads carry a bank number (< 32) in the channel field (spconv2d_utils.h:174-175)
    limit = max(T, 32) if bank else T
    assert (p.position >= 0).all() and (p.position < (limit << 6)).all()
    assert ((p.position & 7) < ks).all() and (((p.position >> 3) & 7) < ks).all()
    # stage_len_[g*32*S + st*32 + lane]; offsets = running max of the rounded-up lane lengths
    sl = p.stage_len.reshape(G, S, 32)
    assert np.array_equal(-(-sl.max(axis=2) // vec) * vec, d.reshape(G, S))
    if not bank:
        assert int(sl.sum()) == int((w != 0).sum())  # Bank-SR adds zero-valued entries to the lane lists
    assert decode_spf(p, vec) == filter_nonzeros(w)
    if not bank:  # plain step 1 keeps the (channel, row, column) scan order inside every lane list
        for slot in range(K):
            g, lane = divmod(slot, 32)
            for st in range(S):
                start = int(p.offsets[g * S + st])
                n = int(sl[g, st, lane])
                at = [32 * start + (e // vec) * 32 * vec + lane * vec + e % vec for e in range(n)]
                pos = p.position[at]
                key = ((pos >> 6) << 6) | (((pos >> 3) & 7) << 3) | (pos & 7)
                assert (np.diff(key) > 0).all()


def test_plain_rows_format(oracle):
    # apply_reorder=false (spconv2d_utils.h:38-61): per (oc, stage) runs in scan order, offsets of size K*S+1
    rng = np.random.default_rng(3)
    K, C, ks, T = 10, 20, 3, 8
    w = sparse_filter(rng, K, C, ks, 0.7)
    p = oracle.SpfPack(w, T, False)
    S = p.stages
    assert len(p.offsets) == K * S + 1 and len(p.stage_len) == 0
    assert p.nnz_counted == int((w != 0).sum()) == len(p.values) == p.offsets[-1]
    got = []
    for o in range(K):
        for st in range(S):
            for e in range(p.offsets[o * S + st], p.offsets[o * S + st + 1]):
                pos = int(p.position[e])
                got.append((o, (pos >> 6) + st * T, (pos >> 3) & 7, pos & 7, p.values[e]))
    expect = [(int(k), int(c), int(r), int(s), w[k, c, r, s]) for k, c, r, s in zip(*np.nonzero(w))]
    assert got == expect


@pytest.mark.parametrize("shape", [(2, 20, 9, 11, 40, 3, 1, 1, 8), (1, 48, 8, 8, 64, 1, 1, 0, 32),
                                   (1, 7, 13, 13, 33, 3, 2, 1, 32), (2, 3, 17, 17, 16, 7, 2, 3, 32),
                                   (1, 70, 6, 6, 70, 1, 2, 0, 32)])
def test_host_decoders_reproduce_dense_conv(oracle, shape):
    n, c, h, w_, k, ks, stride, pad, T = shape
    rng = np.random.default_rng(sum(shape))
    w = sparse_filter(rng, k, c, ks, 0.8)
    x = relu_like(rng, (n, c, h, w_))
    dense = oracle.host_conv2d(x, w, stride, pad)
    # keep-as-is format: same (ic, r, s) summation order as the dense loop minus exact-zero terms
    rows = oracle.SpfPack(w, T, False).conv(x, stride, pad)
    np.testing.assert_allclose(rows, dense, rtol=1e-6, atol=1e-6)
    for bank, reoc, vec in [(0, 0, 1), (0, 0, 4), (1, 1, 4), (1, 0, 1), (0, 1, 4)]:
        got = oracle.SpfPack(w, T, True, vec == 4, bool(bank), bool(reoc)).conv(x, stride, pad)
        np.testing.assert_allclose(got, dense, rtol=1e-5, atol=1e-5)
        assert oracle.tensor_first_mismatch(got, dense) == -1  # the reference's own tolerance predicate


@pytest.mark.parametrize("shape", [(2, 20, 9, 11, 40, 3, 1, 1, 8, 8), (1, 48, 8, 8, 64, 1, 1, 0, 32, 16),
                                   (1, 7, 13, 13, 33, 3, 2, 1, 4, 32), (2, 3, 17, 17, 16, 7, 2, 3, 3, 4),
                                   (1, 70, 6, 6, 130, 1, 2, 0, 16, 8)])
def test_gfx950_stream_layout(oracle, shape):
    """The layout the HIP kernel consumes, as the oracle defines it: structure, content and convolution."""
    n, c, h, w_, k, ks, stride, pad, T, G = shape
    rng = np.random.default_rng(sum(shape))
    w = sparse_filter(rng, k, c, ks, 0.8)
    x = relu_like(rng, (n, c, h, w_))
    order = rng.permutation(k).astype(np.int32)
    for perm in (None, order):
        p = oracle.G950Pack(w, T, G, perm)
        S = (c - 1) // T + 1
        assert p.slots == -(-k // 128) * 128 and p.stages == S
        groups = p.slots // G
        assert len(p.grp_off) == groups * S + 1 and p.grp_off[0] == 0
        d = np.diff(p.grp_off)
        assert (d % 8 == 0).all() and np.array_equal(-(-p.grp_nnz // 8) * 8, d)
        assert int(p.grp_nnz.sum()) == int((w != 0).sum())
        exp_order = np.full(p.slots, -1, np.int32)
        exp_order[:k] = np.arange(k) if perm is None else perm
        assert np.array_equal(p.order, exp_order)
        got = Counter()
        for grp in range(groups):
            for st in range(S):
                b, nn = int(p.grp_off[grp * S + st]), int(p.grp_nnz[grp * S + st])
                pos, val = p.position[b:b + nn], p.values[b:b + nn]
                key = (pos & 0xFFFFFF).astype(np.int64) * 256 + (pos >> 24)
                assert (np.diff(key) > 0).all()  # position-major, slots ascending inside a position
                assert (p.position[b + nn:p.grp_off[grp * S + st + 1]] == 0).all()
                assert (p.values[b + nn:p.grp_off[grp * S + st + 1]] == 0).all()
                for q, v in zip(pos, val):
                    q = int(q)
                    oc = int(exp_order[grp * G + (q >> 24)])
                    got[(oc, ((q >> 6) & 0x3FFFF) + st * T, (q >> 3) & 7, q & 7, v.tobytes())] += 1
        assert got == filter_nonzeros(w)
        np.testing.assert_allclose(p.conv(x, stride, pad, threads=2), oracle.host_conv2d(x, w, stride, pad), rtol=1e-5,
                                   atol=1e-5)
