"""Parity of the HIP path (through the C ABI) with the CPU oracle, on a real MI355X.

Bars: packed index arrays bit-exact; fp32 outputs within max relative error 1e-4, measured as
max |got-ref| / max(|ref|, eps), eps = max(1e-3, 1% of the largest |ref|) (see helpers.max_rel_err).
"""
import os

import numpy as np
import pytest

from conftest import REFERENCE, golden_weights
from helpers import max_rel_err, relu_like, sparse_filter

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def env(oracle):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import tetris_amd as T

    return T, torch, oracle


def run_conv(T, torch, pk, x, K, ks, stride, pad, tile=None):
    n, c, h, w = x.shape
    dx = torch.from_numpy(x).cuda()
    dy = torch.full((n, K, T.out_extent(h, pad, ks, stride), T.out_extent(w, pad, ks, stride)), float("nan"),
                    device="cuda")
    pk.launch(dx.data_ptr(), dy.data_ptr(), n, h, w, stride, pad, tile)
    torch.cuda.synchronize()
    return dy.cpu().numpy()


SHAPES = [  # N, C, H, W, K, ks, stride, pad, sparsity  -- the reference's kernel-size/stride families, ragged edges
    (1, 8, 12, 12, 16, 3, 1, 1, 0.7),
    (2, 20, 9, 11, 40, 3, 1, 1, 0.8),
    (1, 48, 8, 8, 64, 1, 1, 0, 0.7),
    (1, 7, 13, 13, 33, 3, 2, 1, 0.5),
    (2, 3, 17, 17, 16, 7, 2, 3, 0.85),
    (1, 70, 6, 6, 70, 1, 2, 0, 0.9),
    (3, 16, 14, 14, 32, 3, 1, 1, 0.9),
    (5, 32, 7, 7, 64, 1, 1, 0, 0.8),
    (1, 130, 5, 9, 129, 3, 1, 0, 0.9),
    (2, 4, 30, 61, 8, 5, 1, 2, 0.6),
    (1, 16, 10, 10, 24, 3, 1, 1, 1.0),   # all-zero filter
    (1, 16, 10, 10, 24, 3, 1, 1, 0.0),   # dense filter
    (17, 5, 3, 3, 260, 1, 1, 0, 0.5),    # more images than a tile folds, K over two slot paddings
    (2, 160, 7, 7, 48, 3, 1, 1, 0.8),    # few pixels, many channels: workgroups split the channel reduction
    (1, 300, 5, 5, 20, 1, 1, 0, 0.7),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_conv_matches_oracle(env, shape):
    T, torch, O = env
    N, C, H, W, K, ks, stride, pad, sp = shape
    rng = np.random.default_rng(sum(shape[:8]))
    w = sparse_filter(rng, K, C, ks, sp)
    x = relu_like(rng, (N, C, H, W))
    tile = T.tile_select(N, H, W, C, K, ks, stride, pad)
    pk = T.G950Filter.for_tile(w, tile)
    a, o = pk.host_arrays(), O.G950Pack(w, tile.tile_ic, tile.oc_per_wave)
    assert np.array_equal(a["grp_offsets"], o.grp_off) and np.array_equal(a["grp_nnz"], o.grp_nnz)
    assert np.array_equal(a["position"], o.position) and a["values"].tobytes() == o.values.tobytes()
    assert np.array_equal(a["oc_order"], o.order) and a["nnz"] == int((w != 0).sum())
    y = run_conv(T, torch, pk, x, K, ks, stride, pad, tile)
    assert not np.isnan(y).any()
    ref = O.host_conv2d(x, w, stride, pad, threads=4)
    assert max_rel_err(y, ref) <= TOL
    # same arrays decoded on the CPU in the same accumulation order
    assert max_rel_err(y, o.conv(x, stride, pad, threads=4)) <= TOL
    assert T.TensorEqual(y, ref)  # the reference's own predicate (tensor_utils.cc:17-34)


def _odd_weights(rng, K, C, ks):
    """A filter whose zeros are +0.0 and -0.0 alike and whose non-zeros include fp32 denormals of both signs."""
    w = sparse_filter(rng, K, C, ks, 0.7, neg_zero=True)
    flat = w.reshape(-1)
    nz = np.flatnonzero(flat)
    tiny = np.array([1e-40, -1e-40, 1.4e-45, -1.4e-45, 1.1754942e-38], np.float32)  # denormals: bits != 0, value != 0
    flat[nz[::5]] = tiny[np.arange(len(nz[::5])) % len(tiny)]
    assert (flat[nz[::5]] != 0).all() and np.signbit(flat).any()
    return w


@pytest.mark.parametrize("conv", [(3, 1, 1), (1, 1, 0)])
def test_negative_zeros_and_denormal_weights(env, conv):
    # The walk leaves its last batch at the first entry whose weight BITS are zero: that is sound only while every
    # packed entry has non-zero bits and every +-0.0 weight is dropped (Tetris/spconv2d_utils.h:87 drops `!= 0.f`).
    # Denormal weights are non-zero: they must be packed, by the host packer and by the device pass alike, and -0.0
    # must not be (its bits are not zero, its value is).
    T, torch, O = env
    ks, stride, pad = conv
    rng = np.random.default_rng(91 + ks)
    N, C, H, W, K = 2, 40, 14, 14, 72
    w = _odd_weights(rng, K, C, ks)
    x = relu_like(rng, (N, C, H, W)) * np.float32(1e3)
    tile = T.tile_select(N, H, W, C, K, ks, stride, pad)
    pk = T.G950Filter.for_tile(w, tile)
    a, o = pk.host_arrays(), O.G950Pack(w, tile.tile_ic, tile.oc_per_wave)
    assert a["nnz"] == int((w != 0).sum()) == int(o.grp_nnz.sum())
    assert np.array_equal(a["grp_offsets"], o.grp_off) and np.array_equal(a["position"], o.position)
    assert a["values"].tobytes() == o.values.tobytes()
    vals = a["values"].view(np.uint32)
    pads = np.ones(len(vals), bool)
    for beg, n in zip(o.grp_off[:-1], o.grp_nnz):
        pads[beg:beg + n] = False
    assert (vals[~pads] != 0).all() and (vals[pads] == 0).all()   # real entries: non-zero bits; pads: +0.0
    assert (vals[~pads] != 0x80000000).all()                      # no -0.0 among them
    y = run_conv(T, torch, pk, x, K, ks, stride, pad, tile)
    pk.close()
    # denormal products may be flushed by either side: compare on the scale of the normal terms
    assert max_rel_err(y, O.host_conv2d(x, w, stride, pad, threads=4)) <= TOL
    sf = T.SparseFilter(w, C, K, ks, 32, True, True, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL)
    ref = O.SpfPack(w, 32, True, True, True, True)
    assert sf.values_.tobytes() == ref.values.tobytes() and np.array_equal(sf.position_, ref.position)
    sf.close()


TILES = [  # lanes_w, quads, oc_per_wave, waves
    (16, 4, 8, 8), (16, 2, 16, 8), (16, 1, 32, 8), (8, 2, 16, 8), (4, 4, 8, 8), (2, 2, 8, 8), (14, 2, 16, 8),
    (7, 4, 4, 8), (13, 1, 16, 8), (16, 2, 8, 4), (8, 1, 32, 4), (16, 1, 8, 2), (1, 2, 16, 8), (5, 4, 8, 8),
    (16, 1, 16, 1), (3, 1, 32, 8),
    (16, 2, 8, 16), (14, 2, 8, 16), (7, 1, 16, 16), (4, 1, 8, 16), (8, 2, 4, 16), (2, 1, 16, 16),  # four waves per SIMD
    (14, 2, 8, 8), (7, 2, 4, 8), (8, 1, 16, 8), (3, 1, 8, 8), (16, 1, 4, 8)]  # ... as two 8-wave workgroups per CU


@pytest.mark.parametrize("tile", TILES)
@pytest.mark.parametrize("conv", [(3, 1, 1), (1, 1, 0), (3, 2, 1), (7, 2, 3), (1, 2, 0), (5, 1, 2)])
def test_every_tile_shape(env, tile, conv):
    T, torch, O = env
    ks, stride, pad = conv
    lw, nq, g, waves = tile
    N, C, H, W, K = 3, 12, 23, 29, 37
    rng = np.random.default_rng(lw * 100 + nq * 10 + g + ks + stride)
    w = sparse_filter(rng, K, C, ks, 0.7)
    x = relu_like(rng, (N, C, H, W))
    ref = O.host_conv2d(x, w, stride, pad, threads=4)
    ran = 0
    for tile_ic in (1, 2, 5, 16):
        t = T.Tile(lw, nq, g, waves, tile_ic)
        pk = T.G950Filter(w, tile_ic, g)
        try:
            y = run_conv(T, torch, pk, x, K, ks, stride, pad, t)
        except T.TetrisError as e:  # the shape cannot stage that many channels with that many threads
            assert e.code == T.EINVAL and any(m in str(e) for m in ("LDS", "thread", "slot padding", "accumulators")), str(e)
            continue
        ran += 1
        assert max_rel_err(y, ref) <= TOL, (tile, conv, tile_ic)
    if waves >= 8 and waves * g <= 128 and nq <= 2 and ks <= 3:  # the big shapes cannot stage every conv
        assert ran >= 1, (tile, conv)


FLAT_TILES = [  # quads, oc_per_wave, waves: the flat (lanes_w = 64) tiles of pointwise layers
    (1, 8, 16), (1, 2, 16), (1, 1, 16), (2, 8, 16), (2, 4, 16), (2, 1, 16), (2, 16, 8), (4, 8, 8), (1, 8, 8),
    (2, 8, 8), (1, 16, 8), (1, 4, 8), (2, 2, 8)]


@pytest.mark.parametrize("tile", FLAT_TILES)
@pytest.mark.parametrize("shape", [(3, 12, 23, 29, 37), (5, 70, 7, 7, 130), (2, 33, 13, 13, 16), (1, 8, 20, 12, 260),
                                   (17, 5, 3, 3, 40), (2, 300, 14, 14, 24)])
def test_flat_tiles_of_pointwise_layers(env, tile, shape):
    # 1x1, stride 1, no padding: a lane owns four consecutive pixels of an image.  Shapes with H*W not a multiple of
    # four (short last quad, unaligned 16-byte loads, dword stores), ragged channel counts, more images than a unit
    # holds, and enough input channels for the reduction to be split over workgroups.
    T, torch, O = env
    nq, g, waves = tile
    N, C, H, W, K = shape
    rng = np.random.default_rng(nq * 100 + g * 10 + waves + C)
    w = sparse_filter(rng, K, C, 1, 0.7)
    x = relu_like(rng, (N, C, H, W)) + 0.25
    ref = O.host_conv2d(x.astype(np.float32), w, 1, 0, threads=4)
    ran = 0
    for tile_ic in (1, 5, 16, 64):
        t = T.Tile(64, nq, g, waves, tile_ic)
        pk = T.G950Filter(w, tile_ic, g)
        try:
            y = run_conv(T, torch, pk, x.astype(np.float32), K, 1, 1, 0, t)
        except T.TetrisError as e:
            assert e.code == T.EINVAL and "LDS" in str(e), str(e)
            continue
        ran += 1
        assert max_rel_err(y, ref) <= TOL, (tile, shape, tile_ic)
    assert ran >= 3
    # flat tiles are for pointwise layers only
    with pytest.raises(T.TetrisError) as e:
        run_conv(T, torch, T.G950Filter(sparse_filter(rng, K, C, 3, 0.7), 8, g), x.astype(np.float32), K, 3, 1, 1,
                 T.Tile(64, nq, g, waves, 8))
    assert e.value.code == T.EINVAL


@pytest.mark.parametrize("tile", [(1, 8, 16), (2, 4, 16), (1, 2, 16), (2, 16, 8), (4, 8, 8), (1, 4, 8)])
@pytest.mark.parametrize("shape", [(3, 12, 23, 29, 37, 2), (5, 70, 14, 14, 130, 2), (2, 33, 13, 13, 16, 2),
                                   (4, 300, 28, 28, 24, 2), (2, 9, 20, 31, 40, 3), (9, 40, 7, 7, 64, 2)])
def test_flat_tiles_of_strided_pointwise_layers(env, tile, shape):
    # 1x1 layers of stride 2 or 3 (projection shortcuts): the flat tile runs on the sub-grid the layer reads; a quad is
    # four sub-grid pixels, staged as four dwords, and may straddle two rows of the image.  Odd sizes (the sub-grid's
    # last row and column are the image's last), quads cut short at the end of an image, split channel reduction.
    T, torch, O = env
    nq, g, waves = tile
    N, C, H, W, K, stride = shape
    rng = np.random.default_rng(nq * 1000 + g * 10 + waves + C + stride)
    w = sparse_filter(rng, K, C, 1, 0.7)
    x = (relu_like(rng, (N, C, H, W)) + 0.25).astype(np.float32)
    ref = O.host_conv2d(x, w, stride, 0, threads=4)
    ran = 0
    for tile_ic in (3, 16, 64):
        t = T.Tile(64, nq, g, waves, tile_ic)
        pk = T.G950Filter(w, tile_ic, g)
        try:
            y = run_conv(T, torch, pk, x, K, 1, stride, 0, t)
        except T.TetrisError as e:
            assert e.code == T.EINVAL and "LDS" in str(e), str(e)
            continue
        ran += 1
        assert max_rel_err(y, ref) <= TOL, (tile, shape, tile_ic)
    assert ran >= 2


@pytest.mark.parametrize("opts", [1, 2, 3])
def test_ablation_switches_keep_the_results(env, opts):
    # TETRIS_OPT_PAIRS (streams rearranged into pairs sharing an LDS read + singles) and TETRIS_OPT_NO_BANK_RULE (LDS
    # rows packed densely, bank conflicts allowed) change how the kernels run, never what they compute.  Channel
    # orders: file order, the reference's ReorderOutChannel permutation, the balanced order.
    T, torch, O = env
    rng = np.random.default_rng(40 + opts)
    cases = [(3, 40, 23, 29, 64, 3, 1, 1, (14, 2, 8, 16, 8)), (2, 24, 30, 30, 48, 3, 2, 1, (8, 1, 8, 4, 4)),
             (2, 3, 33, 33, 16, 7, 2, 3, (9, 1, 16, 4, 3)), (4, 96, 14, 14, 128, 1, 1, 0, (14, 1, 8, 4, 32)),
             (2, 64, 28, 28, 64, 3, 1, 1, (14, 2, 16, 8, 8)), (2, 32, 20, 20, 32, 5, 1, 2, (5, 1, 4, 8, 2))]
    assert T.options_get() == 0
    try:
        T.options_set(opts)
        assert T.options_get() == opts
        for N, C, H, W, K, ks, stride, pad, tile in cases:
            w = sparse_filter(rng, K, C, ks, 0.6)  # dense enough for many entries to share a position
            x = relu_like(rng, (N, C, H, W))
            ref = O.host_conv2d(x, w, stride, pad, threads=4)
            tile = T.Tile(*tile)
            ref_order = T.SparseFilter(w, C, K, ks, 32, True, True, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL).oc_permutation_
            for order in (None, ref_order, "balanced"):
                pk = T.G950Filter.for_tile(w, tile, oc_order=order)
                y = run_conv(T, torch, pk, x, K, ks, stride, pad, tile)
                assert max_rel_err(y, ref) <= TOL, (opts, tile, order is None)
                pk.close()
        with pytest.raises(T.TetrisError):
            T.options_set(0x100)
    finally:
        T.options_set(0)


def test_channel_order_is_honoured(env):
    T, torch, O = env
    N, C, H, W, K, ks = 2, 16, 11, 11, 72, 3
    rng = np.random.default_rng(77)
    w = sparse_filter(rng, K, C, ks, 0.8)
    x = relu_like(rng, (N, C, H, W))
    sf = T.SparseFilter(w, C, K, ks, 32, True, True, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL)
    order = sf.oc_permutation_
    assert sorted(order.tolist()) == list(range(K)) and order.tolist() != list(range(K))
    tile = T.tile_select(N, H, W, C, K, ks, 1, 1)
    pk = T.G950Filter.for_tile(w, tile, oc_order=order)
    a, o = pk.host_arrays(), O.G950Pack(w, tile.tile_ic, tile.oc_per_wave, order)
    assert np.array_equal(a["position"], o.position) and np.array_equal(a["oc_order"], o.order)
    y = run_conv(T, torch, pk, x, K, ks, 1, 1, tile)
    assert max_rel_err(y, O.host_conv2d(x, w, 1, 1, threads=4)) <= TOL
    with pytest.raises(T.TetrisError):
        T.G950Filter(w, 8, 8, oc_order=np.zeros(K, np.int32))
    with pytest.raises(T.TetrisError) as e:  # a tile the pack was not made for
        pk.launch(0x1000, 0x1000, N, H, W, 1, 1, T.Tile(tile.lanes_w, tile.quads, tile.oc_per_wave, tile.waves,
                                                         tile.tile_ic + 1))
    assert e.value.code == T.EINVAL


def test_reference_shaped_entry_points(env):
    T, torch, O = env
    N, C, H, W, K, ks, stride, pad = 2, 24, 20, 20, 48, 3, 1, 1
    rng = np.random.default_rng(11)
    w = sparse_filter(rng, K, C, ks, 0.85)
    x = relu_like(rng, (N, C, H, W))
    ref = O.host_conv2d(x, w, stride, pad, threads=4)
    for fn in (T.CudaSparseConv2d, T.SparseConv2d_SPF):
        for reorder in (True, False):
            y, ms = fn(x, w, N, H, W, C, K, ks, stride, pad, 0, "NHWC", reorder)
            assert ms > 0 and max_rel_err(y, ref) <= TOL
    # raw launcher with a SparseFilter's device arrays, as the reference's mains call it
    sf = T.SparseFilter(w, C, K, ks, 128, True, True, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL)
    dx = torch.from_numpy(x).cuda()
    dy = torch.zeros((N, K, H, W), device="cuda")
    T.SparseConv2d(dx.data_ptr(), sf.GetDeviceOffsets(), sf.GetDeviceStageLen(), sf.GetDeviceOCPermutation(),
                   sf.GetDevicePosition(), sf.GetDeviceValues(), dy.data_ptr(), N, H, W, C, K, ks, stride, pad)
    torch.cuda.synchronize()
    assert max_rel_err(dy.cpu().numpy(), ref) <= TOL
    # the device copies hold the same bytes as the host vectors
    dev_vals = torch.empty(len(sf.values_), device="cuda")
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy(ctypes.c_void_p(dev_vals.data_ptr()), ctypes.c_void_p(sf.GetDeviceValues()),
                  ctypes.c_size_t(4 * len(sf.values_)), 3)
    assert dev_vals.cpu().numpy().tobytes() == sf.values_.tobytes()
    with pytest.raises(T.TetrisError) as e:
        T.SparseConv2d(dx.data_ptr(), 0, 0, 0, 0, dx.data_ptr(), dy.data_ptr(), N, H, W, C, K, ks, stride, pad)
    assert e.value.code == T.ENOTFOUND


def test_raw_launcher_computes_from_the_arrays_it_is_given(env):
    # SparseConv2d<...> of the reference convolves whatever its five device arrays hold
    # (Tetris/spconv2d_kernel.cuh:14-21, spconv2d_kernel.cu:91-156).  Arrays made by the ORACLE's packer (no library
    # handle owns them) in every layout the constructor can produce -- plain / Bank-SR / Filter-GR / both, vector width
    # 4 and 1, and the keep-as-is rows of apply_reorder = false -- must give the dense convolution; rewriting the values
    # in place on the device must change the result of the next launch.
    T, torch, O = env
    N, C, H, W, K, ks, stride, pad = 2, 40, 17, 19, 70, 3, 1, 1
    rng = np.random.default_rng(61)
    w = sparse_filter(rng, K, C, ks, 0.8)
    x = relu_like(rng, (N, C, H, W))
    ref = O.host_conv2d(x, w, stride, pad, threads=4)
    dx = torch.from_numpy(x).cuda()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731

    def launch(arrs, tile_ic, vec):
        dy = torch.full((N, K, H, W), float("nan"), device="cuda")
        T.SparseConv2d(dx.data_ptr(), arrs[0].data_ptr(), arrs[1].data_ptr() if arrs[1].numel() else 0, arrs[4].data_ptr(),
                       arrs[2].data_ptr(), arrs[3].data_ptr(), dy.data_ptr(), N, H, W, C, K, ks, stride, pad, TILE_IC=tile_ic,
                       vec_width=vec)
        torch.cuda.synchronize()
        return dy.cpu().numpy()

    for tile_ic in (16, 128):
        for bank, reoc, vec in [(0, 0, 4), (1, 0, 4), (0, 1, 4), (1, 1, 4), (1, 1, 1)]:
            p = O.SpfPack(w, tile_ic, True, vec == 4, bool(bank), bool(reoc))
            arrs = [dev(a) for a in p.arrays()]
            assert max_rel_err(launch(arrs, tile_ic, vec), ref) <= TOL, (tile_ic, bank, reoc, vec)
        p = O.SpfPack(w, tile_ic, False)  # keep-as-is rows: offsets per (channel, stage), no stage_len
        arrs = [dev(a) for a in p.arrays()]
        assert max_rel_err(launch(arrs, tile_ic, 0), ref) <= TOL
    # in-place rewrite of the values on the device: same addresses, new content
    p = O.SpfPack(w, 32, True, True, True, True)
    arrs = [dev(a) for a in p.arrays()]
    assert max_rel_err(launch(arrs, 32, 4), ref) <= TOL
    arrs[3].mul_(-2.0)
    torch.cuda.synchronize()
    assert max_rel_err(launch(arrs, 32, 4), -2.0 * ref) <= TOL
    # a permutation that is none is refused, and so are nonsense offsets
    bad = [a.clone() for a in arrs]
    bad[4].zero_()
    with pytest.raises(T.TetrisError) as e:
        launch(bad, 32, 4)
    assert e.value.code == T.EINVAL


def test_raw_launcher_refuses_arrays_that_do_not_fit_the_shape(env):
    # A wrong out_channel, tile_ic or vector width makes the launcher read offsets that are not there: the offsets are
    # checked on the host before any kernel reads the arrays, and the call fails with EINVAL instead of reading (or
    # hashing) beyond them.  Nothing is launched in these cases.
    T, torch, O = env
    N, C, H, W, K, ks = 1, 40, 9, 9, 70, 3
    rng = np.random.default_rng(66)
    w = sparse_filter(rng, K, C, ks, 0.8)
    p = O.SpfPack(w, 16, True, True, True, True)
    offsets, stage_len, position, values, perm = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in p.arrays()]
    dx = torch.zeros((N, C, H, W), device="cuda")
    dy = torch.zeros((N, K, H, W), device="cuda")
    n_ent = values.numel()

    def call(off=offsets, k=K, tile_ic=16, vec=4, n_entries=n_ent):
        T.SparseConv2d(dx.data_ptr(), off.data_ptr(), stage_len.data_ptr(), perm.data_ptr(), position.data_ptr(),
                       values.data_ptr(), dy.data_ptr(), N, H, W, C, k, ks, 1, 1, TILE_IC=tile_ic, vec_width=vec,
                       n_entries=n_entries)
        torch.cuda.synchronize()

    call()  # the right shape runs
    for kwargs in [dict(n_entries=n_ent - 32),              # the arrays are shorter than the offsets say
                   dict(off=offsets.flip(0).contiguous()),  # offsets that decrease
                   dict(off=offsets + 1),                   # offsets that do not start at 0
                   dict(off=-offsets)]:                     # negative offsets
        with pytest.raises(T.TetrisError) as e:
            call(**kwargs)
        assert e.value.code == T.EINVAL, kwargs
    odd = offsets.clone()
    odd[1:] += 2  # every stream but the first shifted by half a vector step
    with pytest.raises(T.TetrisError) as e:
        call(off=odd)
    assert e.value.code == T.EINVAL


def test_raw_launcher_trusting_arrays_it_has_seen(env):
    # TETRIS_OPT_TRUST_SPF_ARRAYS: a set of arrays decoded once is launched again without a read-back (so an in-place
    # rewrite goes unseen) until tetris_spf_invalidate says the arrays have changed.
    T, torch, O = env
    N, C, H, W, K, ks = 2, 24, 12, 12, 40, 3
    rng = np.random.default_rng(67)
    w = sparse_filter(rng, K, C, ks, 0.85)
    x = relu_like(rng, (N, C, H, W))
    ref = O.host_conv2d(x, w, 1, 1, threads=4)
    p = O.SpfPack(w, 32, True, True, True, True)
    arrs = [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in p.arrays()]
    dx = torch.from_numpy(x).cuda()
    dy = torch.zeros((N, K, H, W), device="cuda")

    def launch():
        dy.fill_(float("nan"))
        T.SparseConv2d(dx.data_ptr(), arrs[0].data_ptr(), arrs[1].data_ptr(), arrs[4].data_ptr(), arrs[2].data_ptr(),
                       arrs[3].data_ptr(), dy.data_ptr(), N, H, W, C, K, ks, 1, 1, TILE_IC=32, vec_width=4,
                       n_entries=arrs[3].numel())
        torch.cuda.synchronize()
        return dy.cpu().numpy()

    before = T.options_get()
    try:
        T.options_set(before | T.OPT_TRUST_SPF_ARRAYS)
        assert max_rel_err(launch(), ref) <= TOL      # first sight: decoded
        arrs[3].mul_(-2.0)
        torch.cuda.synchronize()
        assert max_rel_err(launch(), ref) <= TOL      # trusted: the rewrite is not seen
        T.spf_invalidate(arrs[3].data_ptr())
        assert max_rel_err(launch(), -2.0 * ref) <= TOL
        T.options_set(before)
        arrs[3].mul_(-0.5)
        torch.cuda.synchronize()
        assert max_rel_err(launch(), ref) <= TOL      # without the option every call looks
    finally:
        T.options_set(before)
        T.spf_invalidate(arrs[3].data_ptr())


def test_live_sparse_filter_arrays_rewritten_in_place(env):
    # The reference-shaped call (no TILE_IC argument) on a live SparseFilter's device arrays: the handle only
    # supplies TILE_IC; the weights are read from the device arrays at every launch.
    T, torch, O = env
    import ctypes
    N, C, H, W, K, ks = 2, 24, 12, 12, 40, 3
    rng = np.random.default_rng(62)
    w = sparse_filter(rng, K, C, ks, 0.85)
    x = relu_like(rng, (N, C, H, W))
    ref = O.host_conv2d(x, w, 1, 1, threads=4)
    sf = T.SparseFilter(w, C, K, ks, 64, True, True, T.BANK_OPTIMIZE | T.REORDER_OUT_CHANNEL)
    dx = torch.from_numpy(x).cuda()
    dy = torch.zeros((N, K, H, W), device="cuda")
    args = (dx.data_ptr(), sf.GetDeviceOffsets(), sf.GetDeviceStageLen(), sf.GetDeviceOCPermutation(), sf.GetDevicePosition(),
            sf.GetDeviceValues(), dy.data_ptr(), N, H, W, C, K, ks, 1, 1)
    T.SparseConv2d(*args)
    torch.cuda.synchronize()
    assert max_rel_err(dy.cpu().numpy(), ref) <= TOL
    hip = ctypes.CDLL("libamdhip64.so")
    tripled = np.ascontiguousarray(3.0 * sf.values_)
    assert hip.hipMemcpy(ctypes.c_void_p(sf.GetDeviceValues()), tripled.ctypes.data_as(ctypes.c_void_p),
                         ctypes.c_size_t(tripled.nbytes), 1) == 0
    T.SparseConv2d(*args)
    torch.cuda.synchronize()
    assert max_rel_err(dy.cpu().numpy(), 3.0 * ref) <= TOL
    sf.close()


@pytest.mark.parametrize("flags", [0, 1, 2, 3])
def test_spf_entry_point_runs_the_fixed_configuration(env, flags):
    # SparseConv2d_SPF: SparseFilter(TILE_IC = 128, always reordered) built with the given macros, its device arrays
    # fed to the launcher, one fixed tile (Tetris/spf.cc:43-60)
    T, torch, O = env
    rng = np.random.default_rng(63 + flags)
    for N, C, H, W, K, ks, stride, pad in [(2, 24, 20, 20, 48, 3, 1, 1), (1, 200, 9, 9, 36, 3, 1, 1), (3, 16, 14, 14, 32, 1, 1, 0)]:
        w = sparse_filter(rng, K, C, ks, 0.85)
        x = relu_like(rng, (N, C, H, W))
        y, ms = T.SparseConv2d_SPF(x, w, N, H, W, C, K, ks, stride, pad, 0, "NHWC", False, flags)
        assert ms > 0 and max_rel_err(y, O.host_conv2d(x, w, stride, pad, threads=4)) <= TOL


@pytest.mark.parametrize("name", ["rn90_3x3", "rn90_stem", "rn98_1x1", "vgg_64x128", "yolo_255"])
def test_shipped_pruned_layers(env, name):
    # real magnitude-pruned weights: very uneven rows, channels with no weights at all, K = 255
    T, torch, O = env
    hdr, w, _ = golden_weights(name)
    N = 2
    H = min(hdr["H"], 40)
    rng = np.random.default_rng(5)
    x = relu_like(rng, (N, hdr["IC"], H, H))
    y, _ = T.CudaSparseConv2d(x, w, N, H, H, hdr["IC"], hdr["OC"], hdr["KS"], hdr["STRIDE"], hdr["PAD"])
    ref = O.host_conv2d(x, w, hdr["STRIDE"], hdr["PAD"], threads=8)
    assert max_rel_err(y, ref) <= TOL


def test_config1_full_size(env):
    # BASELINE config 1: N=1, C=64, 56x56, K=128, 3x3/s1/p1, 90 % sparse
    T, torch, O = env
    from tetris_amd import workloads as W

    L = W.single_layer()[0]
    w, x = W.make_weights(L), W.make_activations(L, 1)
    assert int((w != 0).sum()) == 7373
    tile = T.tile_select(1, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
    pk = T.G950Filter.for_tile(w, tile)
    y = run_conv(T, torch, pk, x, L.K, L.ks, L.stride, L.pad, tile)
    ref = O.host_conv2d(x, w, L.stride, L.pad, threads=8)
    assert max_rel_err(y, ref) <= TOL
    if O.ref_available():
        assert max_rel_err(y, O.ref_host_conv2d(x, w, L.stride, L.pad)) <= TOL


def test_full_size_properties(env):
    # At sizes the CPU cannot check densely: linearity in the filter, and a slice checked against the oracle.
    T, torch, O = env
    from tetris_amd import workloads as W

    L = W.vgg19()[5]  # 256 -> 256 at 56x56
    N = 16
    w, x = W.make_weights(L), W.make_activations(L, N)
    tile = T.tile_select(N, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
    rng = np.random.default_rng(1)
    mask = rng.random(w.shape) < 0.5
    wa, wb = np.where(mask, w, 0).astype(np.float32), np.where(mask, 0, w).astype(np.float32)
    ys = []
    dx = torch.from_numpy(x).cuda()
    for part in (w, wa, wb):
        pk = T.G950Filter.for_tile(part, tile)
        dy = torch.empty((N, L.K, 56, 56), device="cuda")
        pk.launch(dx.data_ptr(), dy.data_ptr(), N, L.H, L.W, L.stride, L.pad, tile)
        torch.cuda.synchronize()
        ys.append(dy)
    err = (ys[0] - (ys[1] + ys[2])).abs() / ys[0].abs().clamp_min(max(1e-3, 1e-2 * float(ys[0].abs().max())))
    assert float(err.max()) <= TOL
    # one image, a few output channels, against the dense oracle
    sel = [0, 1, 127, 255]
    ref = O.host_conv2d(x[3:4], w[sel], L.stride, L.pad, threads=8)
    assert max_rel_err(ys[0][3:4, sel].cpu().numpy(), ref) <= TOL


@pytest.mark.parametrize("suite", ["vgg19", "resnet50", "mobilenet", "yolov3"])
def test_every_layer_shape_of_the_suites(env, suite):
    # Every distinct layer shape of the benchmark suites at batch 1 and full resolution, tile chosen by the library,
    # against the oracle's packed-format conv (itself pinned to the dense one in test_oracle_pack.py).
    T, torch, O = env
    from tetris_amd import workloads as W

    seen, worst = set(), 0.0
    for L in W.SUITES[suite]():
        key = (L.C, L.H, L.W, L.K, L.ks, L.stride, L.pad)
        if key in seen:
            continue
        seen.add(key)
        w, x = W.make_weights(L), W.make_activations(L, 1)
        tile = T.tile_select(1, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
        pk = T.G950Filter.for_tile(w, tile)
        y = run_conv(T, torch, pk, x, L.K, L.ks, L.stride, L.pad, tile)
        ref = O.G950Pack(w, 32, 8).conv(x, L.stride, L.pad, threads=min(16, O.max_threads()))
        err = max_rel_err(y, ref)
        assert err <= TOL, (L.name, tile, err)
        worst = max(worst, err)
        pk.close()
    assert len(seen) >= 4


def test_random_shapes_with_library_tiles(env):
    # Seeded random layer shapes (all kernel-size/stride families, ragged channel counts, tiny and wide images), the
    # tile left to the library: exercises every kernel variant the selector can reach, the channel-split path included.
    T, torch, O = env
    rng = np.random.default_rng(2024)
    variants = set()
    for case in range(60):
        ks, stride = [(1, 1), (3, 1), (3, 2), (1, 2), (5, 1), (7, 2)][int(rng.integers(6))]
        pad = int(rng.integers(0, ks // 2 + 1)) if ks > 1 else 0
        N = int(rng.integers(1, 6))
        C = int(rng.choice([3, 8, 17, 32, 96, 130, 256, 520]))
        K = int(rng.choice([4, 16, 33, 64, 128, 200, 384]))
        H = int(rng.choice([5, 7, 13, 14, 28, 31, 56, 75]))
        W = int(rng.choice([5, 7, 13, 14, 28, 33, 56, 90]))
        if H + 2 * pad < ks or W + 2 * pad < ks or N * C * H * W > 6e6 or N * K * H * W * C * ks * ks > 3e10:
            continue
        sp = float(rng.choice([0.5, 0.8, 0.9, 0.97]))
        w = sparse_filter(rng, K, C, ks, sp)
        x = relu_like(rng, (N, C, H, W))
        tile = T.tile_select(N, H, W, C, K, ks, stride, pad)
        pk = T.G950Filter.for_tile(w, tile, oc_order="balanced" if case % 2 else None)
        y = run_conv(T, torch, pk, x, K, ks, stride, pad, tile)
        ref = O.G950Pack(w, 32, 8).conv(x, stride, pad, threads=min(16, O.max_threads()))
        err = max_rel_err(y, ref)
        assert err <= TOL, (case, (N, C, H, W, K, ks, stride, pad, sp), tile, err)
        variants.add((tile.waves, tile.quads))
        pk.close()
    assert len(variants) >= 3, variants


@pytest.mark.parametrize("masks", ["masks_vgg19_92.npz", "masks_mobilenet_86.npz", "masks_resnet50_90.npz",
                                   "masks_resnet50_98.npz", "masks_yolov3_89.npz"])
def test_pruned_networks_in_balanced_channel_order(env, masks):
    # The zero patterns of the shipped pruned networks the reference's timing loop walks (evalution/conv2d_timing.py:
    # 136-176): channels of very different density, many of them empty at 98 %, K = 255, C = 384 / 768 and 80 / 40 /
    # 20-pixel maps in YOLOv3.  Every layer at full resolution and batch 2, packed in the output-channel order that
    # balances the waves, with the tile the library picks.
    T, torch, O = env
    from conftest import GOLDEN
    from tetris_amd import workloads as W

    layers = W.pruned_suite(os.path.join(GOLDEN, masks))
    assert len(layers) >= 8
    for L in layers:
        w, x = W.make_weights(L), W.make_activations(L, 2)
        assert int((w != 0).sum()) == W.nnz_of(L)
        tile = T.tile_select(2, L.H, L.W, L.C, L.K, L.ks, L.stride, L.pad)
        order = T.oc_order_balanced(w, tile)
        pk = T.G950Filter.for_tile(w, tile, oc_order=order)
        assert np.array_equal(pk.host_arrays()["oc_order"][:L.K], order)
        y = run_conv(T, torch, pk, x, L.K, L.ks, L.stride, L.pad, tile)
        ref = O.G950Pack(w, 32, 8).conv(x, L.stride, L.pad, threads=min(16, O.max_threads()))
        err = max_rel_err(y, ref)
        assert err <= TOL, (L.name, tile, err)
        pk.close()


@pytest.mark.parametrize("order", ["file", "reference", "balanced"])
def test_channel_order_switch(env, order):
    # The three output-channel orders a pack can be built with: as in the filter, the reference's
    # ReorderOutChannel order (must equal the oracle's restatement of that pass), and the wave-balancing one.
    T, torch, O = env
    rng = np.random.default_rng(77)
    N, C, H, W, K, ks = 2, 48, 19, 23, 72, 3
    w = rng.standard_normal((K, C, ks, ks)).astype(np.float32)
    w *= rng.random(w.shape) < rng.uniform(0.02, 0.5, (K, 1, 1, 1))
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    tile = T.tile_select(N, H, W, C, K, ks, 1, 1)
    pk = T.G950Filter.for_tile(w, tile, oc_order=order)
    got_order = np.array(pk.host_arrays()["oc_order"][:K])
    assert sorted(got_order.tolist()) == list(range(K))
    if order == "file":
        assert np.array_equal(got_order, np.arange(K))
    if order == "reference":
        ref_perm = O.SpfPack(w, tile.tile_ic, apply_reorder=True, reorder_out_channel=True).perm
        assert np.array_equal(got_order, ref_perm)
    y = run_conv(T, torch, pk, x, K, ks, 1, 1, tile)
    pk.close()
    assert max_rel_err(y, O.host_conv2d(x, w, 1, 1, threads=4)) <= TOL
    with pytest.raises(ValueError):
        T.G950Filter.for_tile(w, tile, oc_order="densest-first")


def test_tile_from_a_table_loaded_at_run_time(env, tmp_path):
    T, torch, O = env
    N, C, H, W, K, ks = 3, 24, 37, 41, 40, 3
    table = tmp_path / "tiles.inc"
    table.write_text("    {3, 37, 41, 24, 40, 3, 1, 1, {5, 1, 8, 2, 8}},\n")
    assert T.tile_table_load(str(table)) == 1
    tile = T.tile_select(N, H, W, C, K, ks, 1, 1)
    assert (tile.lanes_w, tile.quads, tile.oc_per_wave, tile.waves, tile.tile_ic) == (5, 1, 8, 2, 8)
    rng = np.random.default_rng(5)
    w, x = sparse_filter(rng, K, C, ks, 0.85), relu_like(rng, (N, C, H, W))
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    y = run_conv(T, torch, pk, x, K, ks, 1, 1, None)  # NULL tile: the library chooses, from the loaded row
    assert max_rel_err(y, O.host_conv2d(x, w, 1, 1, threads=4)) <= TOL


def test_smoke_entry_point(env):
    import importlib
    import sys

    from conftest import ROOT
    sys.path.insert(0, ROOT)
    importlib.import_module("__graft_entry__").smoke()


def test_split_layers_are_bit_reproducible(env):
    # A 14x14 layer whose channel reduction is split over workgroups: the partial sums are added in a fixed order,
    # so two launches give the same bits, and a pack reused for a second shape regrows its scratch correctly.
    T, torch, O = env
    rng = np.random.default_rng(11)
    C, K, ks = 512, 256, 1
    w = sparse_filter(rng, K, C, ks, 0.85)
    tile = T.tile_select(16, 14, 14, C, K, ks, 1, 0)  # one pack (tile) for all three launches
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    for N in (4, 16, 4):
        x = relu_like(rng, (N, C, 14, 14))
        a = run_conv(T, torch, pk, x, K, ks, 1, 0, tile)
        b = run_conv(T, torch, pk, x, K, ks, 1, 0, tile)
        assert a.tobytes() == b.tobytes()
        assert max_rel_err(a, O.host_conv2d(x, w, 1, 0, threads=8)) <= TOL
    pk.close()


@pytest.mark.parametrize("case", [
    # C, K, H, ks, pad, (lanes_w, quads, oc_per_wave, waves, tile_ic)
    (256, 64, 14, 3, 1, (7, 2, 2, 16, 16)),    # triple-buffered kernel, 16 waves
    (256, 64, 14, 3, 1, (14, 1, 8, 8, 8)),     # ... 8 waves
    (128, 32, 7, 3, 1, (7, 1, 8, 4, 8)),       # single-tile kernel
    (512, 96, 14, 1, 0, (64, 1, 2, 16, 32)),   # flat kernel, 16 waves
    (512, 96, 7, 1, 0, (64, 2, 4, 8, 16)),     # flat kernel, 8 waves
])
def test_slices_of_the_channel_reduction_chosen_by_the_tile(env, case):
    # tetris_tile.csplit: 1 = none, 2..8 workgroups share an output tile.  Every legal value gives the convolution and
    # the same bits on a second launch (the slices are added in a fixed order); ReLU on the way out equals ReLU of the
    # plain result bit for bit; a value that leaves a slice fewer than two stages, or is out of range, is refused.
    T, torch, O = env
    C, K, H, ks, pad, t5 = case
    rng = np.random.default_rng(C + K + H)
    w = sparse_filter(rng, K, C, ks, 0.85)
    x = relu_like(rng, (3, C, H, H))
    ref = O.host_conv2d(x, w, 1, pad, threads=8)
    stages = -(-C // t5[4])
    seen = set()
    for cs in (1, 2, 3, 4, 5, 8):
        tile = T.Tile(*t5, cs)
        pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
        if stages < 2 * cs:
            with pytest.raises(T.TetrisError) as e:
                run_conv(T, torch, pk, x, K, ks, 1, pad, tile)
            assert e.value.code == T.EINVAL
            pk.close()
            continue
        a = run_conv(T, torch, pk, x, K, ks, 1, pad, tile)
        b = run_conv(T, torch, pk, x, K, ks, 1, pad, tile)
        assert not np.isnan(a).any() and a.tobytes() == b.tobytes(), (case, cs)
        assert max_rel_err(a, ref) <= TOL, (case, cs)
        # the slices added by the conv kernel's last waves instead of by a second kernel: the same sums in the same order
        before = T.options_get()
        try:
            T.options_set(before | T.OPT_ADD_IN_KERNEL)
            assert T.split_layers_add_in_kernel()  # MI355X keeps workgroup ids that are equal modulo 8 on one XCD
            c = run_conv(T, torch, pk, x, K, ks, 1, pad, tile)
            c2 = run_conv(T, torch, pk, x, K, ks, 1, pad, tile)  # the tickets were left at zero
        finally:
            T.options_set(before)
        assert c2.tobytes() == a.tobytes(), (case, cs)
        assert c.tobytes() == a.tobytes(), (case, cs)
        for opts in (before, before | T.OPT_ADD_IN_KERNEL):  # ReLU on the way out, by either adder
            try:
                T.options_set(opts)
                dx = torch.from_numpy(x).cuda()
                dy = torch.full(ref.shape, float("nan"), device="cuda")
                pk.launch_act(dx.data_ptr(), dy.data_ptr(), 3, H, H, 1, pad, tile, T.ACT_RELU)
                torch.cuda.synchronize()
            finally:
                T.options_set(before)
            assert dy.cpu().numpy().tobytes() == np.maximum(a, 0).tobytes(), (case, cs, opts)
        seen.add(cs)
        pk.close()
    assert {1, 2} <= seen
    assert not T.split_layers_add_in_kernel()  # the switch is off by default
    pk = T.G950Filter.for_tile(w, T.Tile(*t5), oc_order="balanced")
    for bad in (9, -1):
        with pytest.raises(T.TetrisError) as e:
            run_conv(T, torch, pk, x, K, ks, 1, pad, T.Tile(*t5, bad))
        assert e.value.code == T.EINVAL
    pk.close()


def test_launch_shape_query(env):
    # tetris_launch_shape_of: what the launcher derives from (shape, tile) without launching
    T, torch, O = env
    w = sparse_filter(np.random.default_rng(5), 96, 256, 3, 0.9)
    N, H = 4, 14
    for t5, cs in [((7, 2, 2, 16, 16), 0), ((7, 2, 2, 16, 16), 1), ((7, 2, 2, 16, 16), 4), ((14, 1, 8, 4, 8), 2)]:
        tile = T.Tile(*t5, cs)
        pk = T.G950Filter.for_tile(w, tile)
        sh = pk.launch_shape(N, H, H, 1, 1, tile)
        assert sh.stages == -(-256 // t5[4]) and sh.channel_blocks == -(-96 // (t5[2] * t5[3]))
        assert sh.workgroups == sh.unit_groups * sh.channel_blocks * sh.csplit and 1 <= sh.lanes_used <= 64
        assert sh.kernel == (3 if t5[3] >= 8 else 2)
        if cs:
            assert sh.csplit == cs
        assert sh.scratch_bytes == (0 if sh.csplit == 1 else 65536 + 4 * sh.csplit * N * 96 * H * H)
        pk.close()
    w1 = sparse_filter(np.random.default_rng(6), 64, 128, 1, 0.8)
    tile = T.Tile(64, 2, 4, 8, 16)
    pk = T.G950Filter.for_tile(w1, tile)
    sh = pk.launch_shape(3, 13, 13, 1, 0, tile)
    assert sh.kernel == 4 and sh.lanes_used == 64 and sh.unit_groups == -(-(-(-(3 * ((169 + 3) // 4)) // 64)) // 2)
    with pytest.raises(T.TetrisError):
        pk.launch_shape(3, 13, 13, 1, 0, T.Tile(64, 2, 4, 8, 16, 9))
    pk.close()


def test_raw_launcher_from_several_threads(env):
    # The raw launchers keep the packs they decode in a small cache that other calls may evict; a call holds the
    # cache's lock until its launch is issued.  Four threads, each with its own arrays (more sets than the cache
    # would need to start evicting at 16 is not the point here: concurrent decode + launch is), all results right.
    T, torch, O = env
    import threading
    N, C, H, W, K, ks = 2, 24, 12, 12, 40, 3
    x = relu_like(np.random.default_rng(70), (N, C, H, W))
    dx = torch.from_numpy(x).cuda()
    jobs = []
    for i in range(20):  # twenty sets of arrays: the cache holds sixteen
        w = sparse_filter(np.random.default_rng(100 + i), K, C, ks, 0.8)
        p = O.SpfPack(w, 32, True, True, True, True)
        jobs.append((w, [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in p.arrays()],
                     torch.full((N, K, H, W), float("nan"), device="cuda")))
    torch.cuda.synchronize()
    errors = []

    def work(lo):
        try:
            for rep in range(3):
                for w, a, dy in jobs[lo::4]:
                    T.SparseConv2d(dx.data_ptr(), a[0].data_ptr(), a[1].data_ptr(), a[4].data_ptr(), a[2].data_ptr(),
                                   a[3].data_ptr(), dy.data_ptr(), N, H, W, C, K, ks, 1, 1, TILE_IC=32, vec_width=4,
                                   n_entries=a[3].numel())
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for w, a, dy in jobs:
        assert max_rel_err(dy.cpu().numpy(), O.host_conv2d(x, w, 1, 1, threads=4)) <= TOL
        T.spf_invalidate(a[3].data_ptr())


def test_launches_can_be_captured_in_a_hip_graph(env):
    # After one eager launch per shape (which makes the launch plan and, for a split layer, its scratch buffer) a
    # launch is nothing but kernel launches on the caller's stream, so a chain of layers can be captured once and
    # replayed.  Checked on three layers, one of them split over workgroups, over several replays with new inputs.
    T, torch, O = env
    rng = np.random.default_rng(21)
    N = 4
    specs = [(16, 28, 32, 3, 1, 1), (32, 28, 512, 1, 2, 0), (512, 14, 64, 1, 1, 0)]  # C, H, K, ks, stride, pad
    ws, packs, tiles, bufs = [], [], [], []
    x0 = torch.zeros((N, 16, 28, 28), device="cuda")
    cur = x0
    for C, H, K, ks, stride, pad in specs:
        w = sparse_filter(rng, K, C, ks, 0.8)
        tile = T.tile_select(N, H, H, C, K, ks, stride, pad)
        pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
        oh = T.out_extent(H, pad, ks, stride)
        y = torch.empty((N, K, oh, oh), device="cuda")
        ws.append(w); packs.append(pk); tiles.append(tile); bufs.append((cur, y, H, stride, pad))
        cur = y

    def run(stream):
        for pk, tile, (xin, y, H, stride, pad) in zip(packs, tiles, bufs):
            pk.launch(xin.data_ptr(), y.data_ptr(), N, H, H, stride, pad, tile, stream=stream)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run(side.cuda_stream)  # eager warm-up: plans, scratch
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run(side.cuda_stream)
    for rep in range(3):
        x = relu_like(rng, (N, 16, 28, 28))
        x0.copy_(torch.from_numpy(x))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref = x
        for w, (C, H, K, ks, stride, pad) in zip(ws, specs):
            ref = O.host_conv2d(ref, w, stride, pad, threads=8)
        got = bufs[-1][1].cpu().numpy()
        assert max_rel_err(got, ref) <= 3 * TOL, rep  # three chained layers: errors of the first two feed the third
    for pk in packs:
        pk.close()


def test_prepare_then_capture_without_an_eager_launch(env):
    # tetris_g950_prepare makes the plan and a split layer's scratch, so the very first launch can be a captured one;
    # an unprepared launch under capture is refused instead of allocating (which would break the capture).
    T, torch, O = env
    rng = np.random.default_rng(22)
    N, C, H, K = 4, 512, 14, 64
    w = sparse_filter(rng, K, C, 1, 0.8)
    tile = T.Tile(14, 1, 8, 4, 32)  # split over workgroups on this shape
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    other = T.G950Filter.for_tile(w, tile)
    x = torch.zeros((N, C, H, H), device="cuda")
    y = torch.empty((N, K, H, H), device="cuda")
    side = torch.cuda.Stream()
    pk.prepare(N, H, H, 1, 0, tile, stream=side.cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        pk.launch(x.data_ptr(), y.data_ptr(), N, H, H, 1, 0, tile, stream=side.cuda_stream)
        with pytest.raises(T.TetrisError) as e:
            other.launch(x.data_ptr(), y.data_ptr(), N, H, H, 1, 0, tile, stream=side.cuda_stream)
        assert e.value.code == T.EINVAL and "prepare" in str(e.value)
    for rep in range(3):
        xn = relu_like(rng, (N, C, H, H))
        x.copy_(torch.from_numpy(xn))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert max_rel_err(y.cpu().numpy(), O.host_conv2d(xn, w, 1, 0, threads=8)) <= TOL, rep
    pk.close()
    other.close()


def test_autotune_and_timing_entry_points(env):
    # tetris_tile_autotune (GetTetrisSparseConv2dTime, Tetris/spconv2d.cc:72-329) and tetris_spconv2d_time
    # (TimingTetrisSparseConv2d, :29-69): the measured tile launches and computes the right thing, and so does the tile
    # of the exhaustive mode (every legal tile, the reference's table walk :285-329); the timing loop agrees with events
    # recorded around the same launches.  Times are compared with wide bounds only (a factor of two: a wrong unit or a
    # broken search shows, a noisy box does not); the ratios are printed.
    T, torch, O = env
    rng = np.random.default_rng(71)
    N, C, H, W, K, ks, stride, pad = 4, 48, 28, 28, 96, 3, 1, 1
    w = sparse_filter(rng, K, C, ks, 0.85)
    x = relu_like(rng, (N, C, H, W))
    ref = O.host_conv2d(x, w, stride, pad, threads=8)
    dx = torch.from_numpy(x).cuda()
    dy = torch.empty((N, K, H, W), device="cuda")

    def timed(tile):
        pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
        y = run_conv(T, torch, pk, x, K, ks, stride, pad, tile)
        assert max_rel_err(y, ref) <= TOL, tile
        ms = min(pk.time(dx.data_ptr(), dy.data_ptr(), N, H, W, stride, pad, tile, warm=10, repeat=50) for _ in range(3))
        return pk, ms

    tuned, ms_tuned = T.tile_autotune(w, N, H, W, stride, pad, 16)
    assert ms_tuned > 0 and tuned.lanes_w >= 1
    pk_t, t_tuned = timed(tuned)
    pk_s, t_sel = timed(T.tile_select(N, H, W, C, K, ks, stride, pad))
    assert t_tuned <= 2.0 * t_sel, (t_tuned, t_sel)
    full, ms_full = T.tile_autotune(w, N, H, W, stride, pad, -1)  # exhaustive
    pk_f, t_full = timed(full)
    assert ms_full > 0 and t_full <= 2.0 * t_tuned, (t_full, t_tuned)
    print("autotuned / selected %.3f, exhaustive / autotuned %.3f" % (t_tuned / t_sel, t_full / t_tuned))
    # the timing loop against events of our own around the same number of launches
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(10):
        pk_t.launch(dx.data_ptr(), dy.data_ptr(), N, H, W, stride, pad, tuned)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(50):
        pk_t.launch(dx.data_ptr(), dy.data_ptr(), N, H, W, stride, pad, tuned)
    e1.record()
    torch.cuda.synchronize()
    assert 0.5 * t_tuned <= e0.elapsed_time(e1) / 50 <= 2.0 * t_tuned
    with pytest.raises(T.TetrisError) as e:
        pk_t.time(dx.data_ptr(), dy.data_ptr(), N, H, W, stride, pad, tuned, warm=1, repeat=0)
    assert e.value.code == T.EINVAL
    with pytest.raises(T.TetrisError):
        T.tile_autotune(w, 0, H, W, stride, pad, 4)
    for pk in (pk_t, pk_s, pk_f):
        pk.close()


def test_measured_ceilings_are_plausible(env):
    T, torch, O = env
    copy_gbs, fma_tflops = T.measure_peaks()
    assert 2000 < copy_gbs < 8000   # nominal HBM peak 8000 GB/s
    assert 40 < fma_tflops < 157.3  # nominal 157.3 TFLOP/s needs packed fp32; non-packed code can reach half of it


@pytest.mark.parametrize("case", [
    # N, C, H, W, K, ks, stride, pad, (lanes_w, quads, oc_per_wave, waves, tile_ic)
    (5, 24, 14, 14, 40, 3, 1, 1, (7, 1, 8, 4, 8)),     # two images side by side, odd batch: the last pair is half empty
    (5, 24, 14, 14, 40, 3, 1, 1, (14, 2, 8, 16, 8)),   # four side by side, 16 waves
    (3, 16, 28, 28, 32, 3, 1, 1, (14, 2, 8, 8, 8)),    # the 28x28 case of the VGG19 stack
    (6, 32, 13, 13, 64, 3, 2, 1, (7, 1, 4, 4, 4)),     # stride 2: parity planes, four side by side (OW = 7)
    (7, 40, 7, 7, 72, 1, 1, 0, (7, 1, 8, 4, 16)),      # 7x7, 1x1: four side by side, rows of several images folded too
    (4, 8, 10, 6, 16, 5, 1, 2, (3, 1, 4, 2, 4)),       # 5x5 kernel: a two-column halo at every seam
])
def test_images_side_by_side(env, case):
    # Tiles at least twice as wide as the output give the quads of a lane to different images; the seams between the
    # images must behave like image borders (zero padding), which a kernel wider than one column probes.
    T, torch, O = env
    N, C, H, W, K, ks, stride, pad, tile = case
    tile = T.Tile(*tile)
    ow = T.out_extent(W, pad, ks, stride)
    assert 2 * tile.lanes_w >= ow  # the tile folds
    rng = np.random.default_rng(N * 100 + W)
    w = sparse_filter(rng, K, C, ks, 0.6)
    x = relu_like(rng, (N, C, H, W)) + 0.25  # no zeros near the borders: a wrong seam would show
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    y = run_conv(T, torch, pk, x.astype(np.float32), K, ks, stride, pad, tile)
    assert max_rel_err(y, O.host_conv2d(x.astype(np.float32), w, stride, pad, threads=4)) <= TOL
    pk.close()
