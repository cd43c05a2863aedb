"""Parity of every layer of the four benchmark suites at the batch sizes the benchmark times.

The tile the library picks depends on the batch (images side by side, split channel reduction, 16-wave
variants), so each (suite, batch) the benchmark reports is run here layer by layer -- every layer, not one
per distinct shape, because layers of one shape differ in sparsity and in their seeded masks -- with the
library-chosen tile and the balanced output-channel order the benchmark packs with, on the whole batch,
against the CPU oracle's packed-format convolution of the same seeded tensors.

test_error_against_float64 shows what the floor in that measure hides: on the layer with the longest sums of each
suite the device's fp32 result and the oracle's fp32 result are both compared with a float64 convolution under a
denominator with (almost) no floor.

Bar: max |got-ref| / max(|ref|, eps) <= 1e-4, eps = max(1e-3, 1 % of the largest |ref|) (helpers.max_rel_err).
Counterpart of the reference's per-run check, Tetris/spconv2d.cc:430-441.
"""
import numpy as np
import pytest

from helpers import max_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4

# every (suite, batch) the library's table of measured tiles has rows for: batch 1, 2, 4, 8 and 16 of the four suites
CONFIGS = [(suite, batch) for suite in ("vgg19", "resnet50", "mobilenet", "yolov3") for batch in (1, 2, 4, 8, 16)] + \
          [("single", 1)]


@pytest.fixture(scope="module")
def env(oracle):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import tetris_amd as T

    return T, torch, oracle


@pytest.mark.parametrize("suite,batch", CONFIGS, ids=["%s-b%d" % c for c in CONFIGS])
def test_every_layer_at_the_benchmark_batch(env, suite, batch):
    T, torch, O = env
    from tetris_amd import workloads as W

    threads = min(16, O.max_threads())
    layers = W.SUITES[suite]()
    worst = (0.0, None)
    for L in layers:
        w, x = W.make_weights(L), W.make_activations(L, batch)
        tile = T.tile_select(batch, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
        pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
        oh, ow = W.out_hw(L)
        dx = torch.from_numpy(x).cuda()
        dy = torch.full((batch, L.K, oh, ow), float("nan"), device="cuda")
        pk.launch(dx.data_ptr(), dy.data_ptr(), batch, L.H, L.W, L.stride, L.pad, tile)
        torch.cuda.synchronize()
        got = dy.cpu().numpy()
        pk.close()
        del dx, dy
        ref = O.G950Pack(w, 32, 8).conv(x, L.stride, L.pad, threads=threads)
        assert not np.isnan(got).any(), (L.name, tile)
        err = max_rel_err(got, ref)
        assert err <= TOL, (suite, batch, L.name, tile, err)
        if err > worst[0]:
            worst = (err, L.name)
    print("%s batch %d: %d layers, worst max_rel_err %.3g (%s)" % (suite, batch, len(layers), worst[0], worst[1]))


def _conv_f64(torch, x, w, stride, pad):
    import torch.nn.functional as F

    return F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), None, stride, pad).numpy()


@pytest.mark.parametrize("suite", ["vgg19", "resnet50", "mobilenet", "yolov3"])
def test_error_against_float64(env, suite):
    """Two fp32 summation orders of one convolution differ; how far is each from the exact sum?  On the layer of the
    suite whose outputs sum the most non-zero products, at batch 2 with the library's tile: the device result and the
    oracle's fp32 result against a float64 convolution (torch on the CPU), relative to max(|ref|, 1e-6 * max|ref|) --
    a denominator that lets outputs near zero count in full.  The device must be no further from float64 than twice
    the oracle's own distance; the test also prints the smallest floor (as a fraction of max|ref|) under which the
    device meets 1e-4, which is the floor the parity bar needs."""
    T, torch, O = env
    from tetris_amd import workloads as W

    L = max(W.SUITES[suite](), key=lambda l: W.nnz_of(l) / l.K)
    batch = 2
    w, x = W.make_weights(L), W.make_activations(L, batch)
    tile = T.tile_select(batch, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    oh, ow = W.out_hw(L)
    dx = torch.from_numpy(x).cuda()
    dy = torch.full((batch, L.K, oh, ow), float("nan"), device="cuda")
    pk.launch(dx.data_ptr(), dy.data_ptr(), batch, L.H, L.W, L.stride, L.pad, tile)
    torch.cuda.synchronize()
    got = dy.cpu().numpy().astype(np.float64)
    pk.close()
    ref32 = O.G950Pack(w, 32, 8).conv(x, L.stride, L.pad, threads=min(16, O.max_threads())).astype(np.float64)
    dense32 = O.host_conv2d(x, w, L.stride, L.pad, threads=min(16, O.max_threads())).astype(np.float64)
    ref64 = _conv_f64(torch, x, w, L.stride, L.pad)
    big = float(np.max(np.abs(ref64)))
    den = np.maximum(np.abs(ref64), 1e-6 * big)
    e_dev = float(np.max(np.abs(got - ref64) / den))
    e_orc = float(np.max(np.abs(ref32 - ref64) / den))
    e_dense = float(np.max(np.abs(dense32 - ref64) / den))
    a_dev, a_orc = float(np.max(np.abs(got - ref64))) / big, float(np.max(np.abs(ref32 - ref64))) / big
    diff = np.abs(got - ref64)
    over = diff > 1e-4 * np.abs(ref64)
    eps_min = float(np.max(diff[over])) / (1e-4 * big) if over.any() else 0.0
    print("%s %s (%d products per output at most): strict relative error device %.3g, oracle packed %.3g, oracle "
          "dense %.3g; largest absolute error / max|ref| device %.3g, oracle %.3g; 1e-4 holds for the device with a floor "
          "of %.3g * max|ref| or more" % (suite, L.name, int((w != 0).reshape(L.K, -1).sum(1).max()), e_dev, e_orc,
                                          e_dense, a_dev, a_orc, eps_min))
    assert e_dev <= 2.0 * max(e_orc, e_dense), (suite, L.name, tile, e_dev, e_orc, e_dense)
    assert a_dev <= 2.0 * a_orc, (suite, L.name, a_dev, a_orc)
    assert eps_min <= 1e-2  # the floor of helpers.max_rel_err is 1 % of max|ref|
