"""Pins the oracle's dense convolution, tolerance predicate, transposes and weight-file reader."""
import os

import numpy as np
import pytest
import torch

from conftest import REFERENCE, golden_weights
from helpers import relu_like, sparse_filter

SHAPES = [  # N, C, H, W, K, ks, stride, pad
    (1, 3, 9, 11, 5, 3, 1, 1),
    (2, 4, 8, 8, 6, 1, 1, 0),
    (1, 5, 13, 9, 4, 3, 2, 1),
    (2, 3, 15, 15, 4, 7, 2, 3),
    (1, 6, 7, 7, 3, 1, 2, 0),
    (1, 2, 6, 10, 3, 3, 1, 0),
    (1, 2, 8, 8, 2, 5, 3, 2),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_host_conv2d_matches_torch(oracle, shape):
    n, c, h, w, k, ks, stride, pad = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    f = rng.standard_normal((k, c, ks, ks)).astype(np.float32)
    got = oracle.host_conv2d(x, f, stride, pad)
    ref = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(f).double(), stride=stride,
                                     padding=pad).numpy()
    assert got.shape == ref.shape
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", SHAPES)
def test_host_conv2d_all_ones_counts_taps(oracle, shape):
    # the reference's DEBUG mode (tensor_utils.cc:10-12, :74-76): every output = C x (in-bounds taps)
    n, c, h, w, k, ks, stride, pad = shape
    got = oracle.host_conv2d(np.ones((n, c, h, w), np.float32), np.ones((k, c, ks, ks), np.float32), stride, pad)
    oh, ow = got.shape[2:]
    rows = np.array([sum(pad <= i * stride + r < h + pad for r in range(ks)) for i in range(oh)])
    cols = np.array([sum(pad <= j * stride + s < w + pad for s in range(ks)) for j in range(ow)])
    expect = (c * rows[:, None] * cols[None, :]).astype(np.float32)
    assert np.array_equal(got, np.broadcast_to(expect, got.shape))


def test_host_conv2d_one_hot_filter_is_a_shifted_strided_copy(oracle):
    rng = np.random.default_rng(5)
    n, c, h, w, ks, stride, pad = 2, 3, 10, 12, 3, 2, 1
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    for (ic, r, s) in [(0, 0, 0), (1, 2, 1), (2, 1, 2)]:
        f = np.zeros((1, c, ks, ks), np.float32)
        f[0, ic, r, s] = 1.0
        got = oracle.host_conv2d(x, f, stride, pad)
        xp = np.pad(x, ((0, 0), (0, 0), (pad, pad), (pad, pad)))
        oh, ow = got.shape[2:]
        expect = xp[:, ic, r:r + stride * oh:stride, s:s + stride * ow:stride]
        assert np.array_equal(got[:, 0], expect)  # r is the row tap, s the column tap (cross-correlation)


def test_host_conv2d_threads_do_not_change_bits(oracle):
    rng = np.random.default_rng(9)
    x = relu_like(rng, (2, 8, 12, 12))
    f = sparse_filter(rng, 16, 8, 3, 0.8)
    assert np.array_equal(oracle.host_conv2d(x, f, 1, 1, threads=1), oracle.host_conv2d(x, f, 1, 1, threads=4))


def test_host_conv2d_equals_compiled_reference(oracle):
    if not oracle.ref_available():
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    for shape in SHAPES:
        n, c, h, w, k, ks, stride, pad = shape
        rng = np.random.default_rng(100 + sum(shape))
        x = rng.standard_normal((n, c, h, w)).astype(np.float32)
        f = sparse_filter(rng, k, c, ks, 0.5)
        assert np.array_equal(oracle.host_conv2d(x, f, stride, pad), oracle.ref_host_conv2d(x, f, stride, pad))


def test_float_equal_predicate(oracle):
    # tensor_utils.cc:17-19: |x-y| <= 1e-5*(|x|+|y|) + 1e-5
    cases = [(0.0, 0.0), (0.0, 1e-5), (0.0, 1.01e-5), (1.0, 1.00003), (1.0, 1.00002), (-3.0, -3.0001), (1e6, 1e6 + 15),
             (1e6, 1e6 + 25), (1.0, -1.0)]
    for a, b in cases:
        a32, b32 = float(np.float32(a)), float(np.float32(b))
        expect = abs(a32 - b32) <= 1e-5 * (abs(a32) + abs(b32)) + 1e-5
        assert oracle.float_equal(a, b) == expect, (a, b)
        if oracle.ref_available():
            assert oracle.ref_float_equal(a, b) == oracle.float_equal(a, b)
    x = np.arange(10, dtype=np.float32)
    y = x.copy()
    assert oracle.tensor_first_mismatch(x, y) == -1
    y[7] += 1
    assert oracle.tensor_first_mismatch(x, y) == 7


def test_layout_transposes(oracle):
    # tensor_utils.cc:85-134 (NCHW2NHWC / NHWC2NCHW): against numpy.transpose, as a round trip, on ragged extents and
    # on an empty tensor, and against the reference's own in-place routines compiled as they lie
    rng = np.random.default_rng(31)
    for shape in [(1, 1, 1, 1), (2, 3, 5, 7), (3, 8, 4, 4), (1, 17, 2, 9), (2, 1, 6, 1), (0, 4, 3, 3)]:
        x = rng.standard_normal(shape).astype(np.float32)
        nhwc = oracle.nchw_to_nhwc(x)
        assert nhwc.shape == (shape[0], shape[2], shape[3], shape[1])
        assert np.array_equal(nhwc, np.transpose(x, (0, 2, 3, 1)))
        back = oracle.nhwc_to_nchw(nhwc)
        assert np.array_equal(back, x) and np.array_equal(back, np.transpose(nhwc, (0, 3, 1, 2)))
        if oracle.ref_available() and x.size:
            assert np.array_equal(oracle.ref_nchw_to_nhwc(x), nhwc)
            assert np.array_equal(oracle.ref_nhwc_to_nchw(nhwc), x)
    # a tensor whose value IS its NCHW index makes a swapped pair of axes visible element by element
    x = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    nhwc = oracle.nchw_to_nhwc(x)
    assert nhwc[1, 2, 3, 1] == x[1, 1, 2, 3] == 1 * 60 + 1 * 20 + 2 * 5 + 3


def test_weight_reader_on_a_written_file(oracle, tmp_path):
    # header order H W IC OC KS PAD STRIDE GROUPS (tensor_utils.cc:66), then OC*IC*KS*KS floats, OIHW
    vals = np.array([0.0, -0.0, 1.5, -2.25e-3, 7, 1e-8, 0.0, 3.25], np.float32)
    p = tmp_path / "w.txt"
    p.write_text("5 6 2 4 1 0 1 1\n" + " ".join(repr(float(v)) for v in vals[:4]) + "\n" +
                 " ".join(repr(float(v)) for v in vals[4:]) + "\n")
    hdr, w, nnz = oracle.read_weight_file(str(p))
    assert hdr == dict(H=5, W=6, IC=2, OC=4, KS=1, PAD=0, STRIDE=1, GROUPS=1)
    assert w.shape == (4, 2, 1, 1) and np.array_equal(w.ravel(), vals)
    assert nnz == 5  # -0.0 compares equal to zero
    with pytest.raises(FileNotFoundError):
        oracle.read_weight_file(str(tmp_path / "missing"))


def test_weight_reader_equals_reference_reader(oracle):
    if not (oracle.ref_available() and os.path.isdir(REFERENCE)):
        pytest.skip("reference checkout absent")
    for name in ("rn98_1x1", "rn90_stem", "yolo_255"):
        hdr_g, w_g, rel = golden_weights(name)
        path = os.path.join(REFERENCE, "evalution", "conv_weight_data", rel)
        hdr, w, nnz = oracle.read_weight_file(path)
        hdr_r, w_r = oracle.ref_read_weight_file(path)
        assert hdr == hdr_r == hdr_g
        assert w.tobytes() == w_r.tobytes() == w_g.tobytes()
        assert nnz == int((w_g != 0).sum())
