"""Parity of every layer of the four benchmark suites at the batch sizes the benchmark times.

The tile the library picks depends on the batch (images side by side, split channel reduction, 16-wave
variants), so each (suite, batch) the benchmark reports is run here layer by layer -- every layer, not one
per distinct shape, because layers of one shape differ in sparsity and in their seeded masks -- with the
library-chosen tile and the balanced output-channel order the benchmark packs with, on the whole batch,
against the CPU oracle's packed-format convolution of the same seeded tensors.

Bar: max |got-ref| / max(|ref|, eps) <= 1e-4, eps = max(1e-3, 1 % of the largest |ref|) (helpers.max_rel_err).
Counterpart of the reference's per-run check, Tetris/spconv2d.cc:430-441.
"""
import numpy as np
import pytest

from helpers import max_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-4

CONFIGS = [("vgg19", 1), ("vgg19", 4), ("vgg19", 8), ("vgg19", 16), ("resnet50", 1), ("resnet50", 8), ("resnet50", 16),
           ("mobilenet", 1), ("mobilenet", 8), ("mobilenet", 16), ("yolov3", 16), ("single", 1)]


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
