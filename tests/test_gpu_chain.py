"""Layers run as a network: ReLU / 2x2 max-pooling glue (tetris_relu_maxpool) and a chain of sparse convolutions
whose inputs are the activations of the layer before, against numpy and the CPU oracle's dense convolution."""
import numpy as np
import pytest

from helpers import max_rel_err, sparse_filter

pytestmark = pytest.mark.gpu


def _np_relu_pool(x, pool):
    y = np.maximum(x, 0.0)
    if pool == 2:
        n, c, h, w = y.shape
        y = y[:, :, : h // 2 * 2, : w // 2 * 2].reshape(n, c, h // 2, 2, w // 2, 2).max(axis=(3, 5))
    return y


@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (1, 5, 7, 9), (3, 4, 14, 14), (2, 2, 13, 16), (1, 1, 2, 2), (2, 7, 30, 20)])
@pytest.mark.parametrize("pool", [1, 2])
@pytest.mark.parametrize("misalign", [0, 1])
def test_relu_maxpool_matches_numpy(shape, pool, misalign):
    import torch
    import tetris_amd as T

    rng = np.random.default_rng(hash((shape, pool)) % 2**32)
    x = rng.normal(size=shape).astype(np.float32)
    n, c, h, w = shape
    want = _np_relu_pool(x, pool)
    # misalign: tensors that start 4 bytes into an allocation (the 16-byte paths must not be taken)
    dx_all = torch.zeros(x.size + 4, device="cuda")
    dy_all = torch.full((want.size + 4,), float("nan"), device="cuda")
    dx = dx_all[misalign: misalign + x.size]
    dy = dy_all[misalign: misalign + want.size]
    dx.copy_(torch.from_numpy(x.reshape(-1)))
    T.relu_maxpool(dx.data_ptr(), dy.data_ptr(), n, c, h, w, pool)
    torch.cuda.synchronize()
    got = dy.cpu().numpy().reshape(want.shape)
    assert np.array_equal(got, want)
    assert np.isnan(dy_all[misalign + want.size:].cpu().numpy()).all()  # nothing written past the end
    if pool == 1:  # in place
        T.relu_maxpool(dx.data_ptr(), dx.data_ptr(), n, c, h, w, 1)
        torch.cuda.synchronize()
        assert np.array_equal(dx.cpu().numpy().reshape(shape), want)


def test_relu_maxpool_rejects_bad_arguments():
    import torch
    import tetris_amd as T

    d = torch.zeros(16, device="cuda")
    with pytest.raises(T.TetrisError):
        T.relu_maxpool(d.data_ptr(), d.data_ptr(), 1, 1, 4, 4, 3)
    with pytest.raises(T.TetrisError):
        T.relu_maxpool(0, d.data_ptr(), 1, 1, 4, 4, 1)
    with pytest.raises(T.TetrisError):
        T.relu_maxpool(d.data_ptr(), d.data_ptr(), 1, 1, 1, 4, 2)


def test_chain_of_layers_matches_the_oracle(oracle):
    """conv -> ReLU -> conv -> ReLU + pool -> conv -> ReLU -> conv (1x1) on the device, every conv through the C ABI with
    the library's tile and balanced channel order; the CPU chain uses the oracle's dense convolution."""
    import torch
    import tetris_amd as T

    rng = np.random.default_rng(4242)
    N, hw = 3, 28
    specs = [(3, 24, 3, 1, 1, 0.5, 1), (24, 40, 3, 1, 1, 0.85, 2), (40, 64, 3, 1, 1, 0.9, 1), (64, 32, 1, 1, 0, 0.8, 0)]
    x = rng.random((N, 3, hw, hw), dtype=np.float32)
    ref = x
    dev = torch.from_numpy(x).cuda()
    h = hw
    for (c, k, ks, stride, pad, sp, pool) in specs:
        w = sparse_filter(rng, k, c, ks, sp)
        tile = T.tile_select(N, h, h, c, k, ks, stride, pad)
        pk = T.G950Filter.for_tile(w, tile, oc_order=T.oc_order_balanced(w, tile))
        oh = (h + 2 * pad - ks) // stride + 1
        y = torch.full((N, k, oh, oh), float("nan"), device="cuda")
        pk.launch(dev.data_ptr(), y.data_ptr(), N, h, h, stride, pad, tile)
        ref = oracle.host_conv2d(np.ascontiguousarray(ref), w, stride, pad)
        if pool:
            z = torch.full((N, k, oh // pool, oh // pool), float("nan"), device="cuda")
            T.relu_maxpool(y.data_ptr(), z.data_ptr(), N, k, oh, oh, pool)
            ref = _np_relu_pool(ref, pool)
            dev, h = z, oh // pool
        else:
            dev, h = y, oh
        torch.cuda.synchronize()
        pk.close()
        assert max_rel_err(dev.cpu().numpy(), ref) <= 1e-4  # north-star tolerance, layer after layer


def test_cold_timing_option(oracle):
    """TETRIS_OPT_COLD_TIMING: single launches timed after a cache-evicting pass.  A launch from cold caches is not
    faster than back-to-back ones, the tuner still returns a tile that launches and computes the right thing, and the
    option is switched off again afterwards."""
    import torch
    import tetris_amd as T

    rng = np.random.default_rng(99)
    N, C, H, K, ks = 8, 64, 28, 128, 1
    w = sparse_filter(rng, K, C, ks, 0.8)
    x = rng.random((N, C, H, H), dtype=np.float32)
    dx = torch.from_numpy(x).cuda()
    dy = torch.full((N, K, H, H), float("nan"), device="cuda")
    tile = T.tile_select(N, H, H, C, K, ks, 1, 0)
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    warm = min(pk.time(dx.data_ptr(), dy.data_ptr(), N, H, H, 1, 0, tile, warm=5, repeat=30) for _ in range(3))
    before = T.options_get()
    try:
        T.options_set(before | T.OPT_COLD_TIMING)
        cold = min(pk.time(dx.data_ptr(), dy.data_ptr(), N, H, H, 1, 0, tile, warm=1, repeat=10) for _ in range(3))
        tuned, ms = T.tile_autotune(w, N, H, H, 1, 0, 8)
    finally:
        T.options_set(before)
    assert T.options_get() == before
    assert cold >= 0.9 * warm and ms > 0, (cold, warm, ms)
    pk2 = T.G950Filter.for_tile(w, tuned, oc_order="balanced")
    pk2.launch(dx.data_ptr(), dy.data_ptr(), N, H, H, 1, 0, tuned)
    torch.cuda.synchronize()
    assert max_rel_err(dy.cpu().numpy(), oracle.host_conv2d(x, w, 1, 0)) <= 1e-4
    pk.close()
    pk2.close()


# (tile, N, C, K, H, W, ks, stride, pad, pooling expected to be possible)
_FUSED_CASES = [
    ((14, 2, 8, 16, 16), 4, 32, 128, 56, 56, 3, 1, 1, True),    # sixteen waves, three LDS buffers
    ((14, 2, 8, 8, 8), 3, 16, 64, 56, 56, 3, 1, 1, True),       # eight waves
    ((14, 1, 8, 8, 16), 3, 32, 64, 56, 56, 3, 1, 1, True),
    ((28, 4, 8, 4, 3), 2, 3, 64, 56, 56, 3, 1, 1, True),        # single LDS tile, register staging
    ((7, 2, 2, 16, 16), 2, 16, 32, 28, 28, 3, 1, 1, False),     # odd number of lanes per row
    ((14, 2, 8, 16, 16), 5, 16, 128, 14, 14, 3, 1, 1, True),    # four images side by side, one stage: not split
    ((14, 2, 8, 16, 16), 3, 16, 128, 28, 28, 3, 1, 1, True),    # two images side by side
    ((14, 2, 8, 16, 16), 2, 256, 128, 14, 14, 3, 1, 1, True),   # split layer: the adding kernel pools (scalar path)
    ((14, 2, 8, 16, 16), 1, 256, 128, 28, 28, 3, 1, 1, True),   # split layer, 16-byte path of the adding kernel
    ((16, 1, 4, 8, 8), 2, 8, 24, 15, 15, 3, 1, 1, True),        # odd output: last row and column dropped
    ((14, 1, 8, 16, 8), 2, 16, 64, 56, 56, 3, 2, 1, True),      # stride 2
    ((13, 2, 8, 16, 8), 2, 16, 64, 52, 52, 3, 1, 1, False),
    ((64, 1, 4, 16, 64), 2, 64, 64, 28, 28, 1, 1, 0, None),     # flat tile: pools only where the layer is split
    ((64, 1, 4, 16, 64), 2, 512, 64, 7, 7, 1, 1, 0, None),
]


@pytest.mark.parametrize("case", _FUSED_CASES, ids=lambda c: "t%s_n%d_c%d_k%d_%dx%d_ks%d_s%d" % (("-".join(map(str, c[0])),) + c[1:8]))
def test_activation_fused_into_the_launch(case, oracle):
    """tetris_spconv2d_launch_act: ReLU, and ReLU + 2x2 max-pooling, written by the conv (or the adding) kernel itself
    are bit-identical to the plain launch followed by tetris_relu_maxpool; the ReLU result also matches the oracle.
    Where a tile cannot pool, the launch is refused with TETRIS_EUNSUPPORTED and writes nothing."""
    import torch
    import tetris_amd as T

    tl, N, Cc, K, H, W, ks, stride, pad, can_pool = case
    rng = np.random.default_rng(hash(case[:9]) % (1 << 32))
    tile = T.Tile(*tl)
    w = sparse_filter(rng, K, Cc, ks, 0.8)
    x = (rng.random((N, Cc, H, W), dtype=np.float32) - 0.5)
    OH, OW = (H + 2 * pad - ks) // stride + 1, (W + 2 * pad - ks) // stride + 1
    pk = T.G950Filter.for_tile(w, tile, oc_order=T.oc_order_balanced(w, tile))
    dx = torch.from_numpy(x).cuda()
    y = torch.full((N, K, OH, OW), float("nan"), device="cuda")
    pk.launch(dx.data_ptr(), y.data_ptr(), N, H, W, stride, pad, tile)
    for act in (T.ACT_RELU, T.ACT_RELU_POOL2):
        shape = (N, K, OH, OW) if act == T.ACT_RELU else (N, K, OH // 2, OW // 2)
        two = torch.full(shape, float("nan"), device="cuda")
        T.relu_maxpool(y.data_ptr(), two.data_ptr(), N, K, OH, OW, act)
        one = torch.full(shape, float("nan"), device="cuda")
        ok = pk.act_supported(N, H, W, stride, pad, tile, act)
        if act == T.ACT_RELU:
            assert ok
        elif can_pool is not None:
            assert ok == can_pool
        if not ok:
            with pytest.raises(T.TetrisError) as e:
                pk.launch_act(dx.data_ptr(), one.data_ptr(), N, H, W, stride, pad, tile, act)
            assert e.value.code == 3  # TETRIS_EUNSUPPORTED
            torch.cuda.synchronize()
            assert bool(torch.isnan(one).all())
            continue
        pk.launch_act(dx.data_ptr(), one.data_ptr(), N, H, W, stride, pad, tile, act)
        torch.cuda.synchronize()
        assert not bool(torch.isnan(one).any())
        assert torch.equal(one, two)
        if act == T.ACT_RELU:
            ref = np.maximum(oracle.host_conv2d(x, w, stride, pad), 0.0)
            assert max_rel_err(one.cpu().numpy(), ref) <= 1e-4
    with pytest.raises(T.TetrisError):
        pk.launch_act(dx.data_ptr(), y.data_ptr(), N, H, W, stride, pad, tile, 3)
    pk.close()


def test_chain_with_fused_activations_in_a_hip_graph(oracle):
    """conv+ReLU -> conv+ReLU+pool -> conv+ReLU (split layer) captured once and replayed on new inputs: each replay
    equals the eager two-pass chain bit for bit and the CPU chain within tolerance."""
    import torch
    import tetris_amd as T

    rng = np.random.default_rng(77)
    N, H = 4, 28
    specs = [(8, 32, 3, 1, T.ACT_RELU), (32, 64, 3, 1, T.ACT_RELU_POOL2), (64, 256, 3, 1, T.ACT_RELU)]  # C, K, ks, pad, act
    x0 = torch.zeros((N, 8, H, H), device="cuda")
    layers, cur, h = [], x0, H
    for C, K, ks, pad, act in specs:
        w = sparse_filter(rng, K, C, ks, 0.8)
        tile = T.tile_select(N, h, h, C, K, ks, 1, pad)
        pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
        if not pk.act_supported(N, h, h, 1, pad, tile, act):  # the table's tile for this shape cannot pool
            tile = T.Tile(14, 2, tile.oc_per_wave, 16, tile.tile_ic)
            assert pk.act_supported(N, h, h, 1, pad, tile, act)
        oh = h // 2 if act == T.ACT_RELU_POOL2 else h
        y = torch.empty((N, K, oh, oh), device="cuda")
        raw = torch.empty((N, K, h, h), device="cuda")
        layers.append((w, pk, tile, cur, y, raw, h, pad, act))
        cur, h = y, oh

    side = torch.cuda.Stream()
    for _, pk, tile, xin, y, raw, hh, pad, act in layers:
        pk.prepare(N, hh, hh, 1, pad, tile, stream=side.cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _, pk, tile, xin, y, raw, hh, pad, act in layers:
            pk.launch_act(xin.data_ptr(), y.data_ptr(), N, hh, hh, 1, pad, tile, act, stream=side.cuda_stream)
    for rep in range(3):
        x = rng.random((N, 8, H, H), dtype=np.float32) - 0.3
        x0.copy_(torch.from_numpy(x))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [l[4].clone() for l in layers]
        ref = x
        for (w, pk, tile, xin, y, raw, hh, pad, act), g in zip(layers, got):  # eager, two passes, same buffers
            pk.launch(xin.data_ptr(), raw.data_ptr(), N, hh, hh, 1, pad, tile)
            T.relu_maxpool(raw.data_ptr(), y.data_ptr(), N, raw.shape[1], hh, hh, act)
            torch.cuda.synchronize()
            assert torch.equal(y, g), rep
            ref = _np_relu_pool(oracle.host_conv2d(np.ascontiguousarray(ref), w, 1, pad), act)
            assert max_rel_err(g.cpu().numpy(), ref) <= 1e-4, rep
            ref = g.cpu().numpy()
    for l in layers:
        l[1].close()
