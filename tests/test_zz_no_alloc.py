"""The entry point that allocates nothing (tetris_spconv2d_launch_noalloc) against tetris_spconv2d_launch.

Callers that cannot call hipMalloc (code under graph capture, serving loops) launch through it: the partial sums of
layers whose channel reduction is split over workgroups go to a static device array instead of a buffer the pack
allocates.  Checked through the C ABI: same bits as the existing entry point, on two calls in a row, the second with
a smaller input (the array keeps the first call's contents), plus the error paths (no plan prepared, layer too
large for the array).
"""
import numpy as np
import pytest

from helpers import max_rel_err, relu_like, sparse_filter

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env(oracle):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import tetris_amd as T

    return T, torch, oracle


def conv(T, torch, pk, x, K, tile, noalloc):
    n, c, h, w = x.shape
    dx = torch.from_numpy(x).cuda()
    dy = torch.full((n, K, h, w), float("nan"), device="cuda")
    fn = pk.launch_noalloc if noalloc else pk.launch
    fn(dx.data_ptr(), dy.data_ptr(), n, h, w, 1, 0, tile)
    torch.cuda.synchronize()
    return dy.cpu().numpy()


def test_noalloc_matches_launch_on_two_calls_in_a_row(env):
    T, torch, O = env
    rng = np.random.default_rng(31)
    C, K, ks = 512, 256, 1
    w = sparse_filter(rng, K, C, ks, 0.85)
    tile = T.Tile(14, 1, 8, 4, 32, 4)  # csplit = 4: four workgroups share every output tile, so the static array is in use
    pk = T.G950Filter.for_tile(w, tile, oc_order="balanced")
    for N in (16, 4):  # the second call is smaller: the array still holds the first call's partial sums
        x = relu_like(rng, (N, C, 14, 14))
        with pytest.raises(T.TetrisError) as e:  # nothing prepared for this shape yet, and the call must not allocate
            conv(T, torch, pk, x, K, tile, True)
        assert e.value.code == T.ENOTFOUND
        pk.prepare(N, 14, 14, 1, 0, tile)
        got = conv(T, torch, pk, x, K, tile, True)
        want = conv(T, torch, pk, x, K, tile, False)
        assert not np.isnan(got).any()
        assert got.tobytes() == want.tobytes()
        assert max_rel_err(got, O.host_conv2d(x, w, 1, 0, threads=8)) <= 1e-4
        again = conv(T, torch, pk, x, K, tile, True)
        assert again.tobytes() == got.tobytes()
    pk.close()


def test_noalloc_covers_a_split_layer_and_refuses_what_does_not_fit(env):
    T, torch, O = env
    assert T.noalloc_scratch_bytes() == 64 << 20
    rng = np.random.default_rng(32)
    # 7x7 maps, many channels: the reduction is split over eight workgroups per tile (the tile says so)
    C, K = 1024, 128
    w = sparse_filter(rng, K, C, 1, 0.9)
    tile = T.Tile(7, 1, 8, 4, 32, 8)  # csplit = 8
    pk = T.G950Filter.for_tile(w, tile)
    x = relu_like(rng, (2, C, 7, 7))
    pk.prepare(2, 7, 7, 1, 0, tile)
    got = conv(T, torch, pk, x, K, tile, True)
    assert got.tobytes() == conv(T, torch, pk, x, K, tile, False).tobytes()
    assert max_rel_err(got, O.host_conv2d(x, w, 1, 0, threads=8)) <= 1e-4
    # partial sums here: eight copies of 2 x 128 x 7 x 7 floats; a limit below one copy must refuse the layer, and so
    # must a limit of seven copies
    try:
        assert T.noalloc_scratch_limit(2 * 128 * 49 * 4) == 2 * 128 * 49 * 4
        with pytest.raises(T.TetrisError) as e:
            conv(T, torch, pk, x, K, tile, True)
        assert e.value.code == T.EINVAL and "static scratch" in str(e.value)
        T.noalloc_scratch_limit(7 * 2 * 128 * 49 * 4)
        with pytest.raises(T.TetrisError) as e:
            conv(T, torch, pk, x, K, tile, True)
        assert e.value.code == T.EINVAL
        T.noalloc_scratch_limit(8 * 2 * 128 * 49 * 4 + (1 << 16))
        assert conv(T, torch, pk, x, K, tile, True).tobytes() == got.tobytes()
    finally:
        assert T.noalloc_scratch_limit(0) == 64 << 20
    assert conv(T, torch, pk, x, K, tile, True).tobytes() == got.tobytes()
    pk.close()
