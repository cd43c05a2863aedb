"""Seeded synthetic layers for the four benchmark suites (VGG19, ResNet-50, MobileNetV1 pointwise,
YOLOv3/Darknet-53 at 416) plus the single-layer case.

Bit-reproducible anywhere numpy runs: every value comes from a counter-based splitmix64 stream, turned
into floats with explicit integer arithmetic (no library distribution objects).
  weights      OIHW fp32, N(0, 0.05^2) by Box-Muller, then exactly round(sparsity * size) entries zeroed:
               the ones with the smallest 64-bit keys of a second stream (a seeded random subset)
  activations  NCHW fp32, uniform [0, 1) with each element zeroed with probability 1/2 (ReLU-like)
The reference draws its inputs from rand() seeded with time(0) (Tetris/spconv2d.cc:377,
Tetris/tensor_utils.cc:9-14), which cannot be reproduced, and reads pruned weights from text files.

pruned_suite() makes layers whose zero pattern is that of such a pruned network (a file of bit-packed masks), with
seeded values: the time of a launch depends on where the non-zeros are, not on what they are.
"""
import os
import zlib
from collections import namedtuple

import numpy as np

Layer = namedtuple("Layer", "suite index name C H W K ks stride pad sparsity mask", defaults=(None,))

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)
BASE_SEED = 0x7E7A15


def _splitmix64(seed, n, start=0):
    """Outputs start .. start+n-1 of splitmix64 started at `seed` (vectorised: output i hashes seed + (i+1)*gamma)."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (np.arange(start + 1, start + n + 1, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15))
        z ^= z >> np.uint64(30)
        z *= np.uint64(0xBF58476D1CE4E5B9)
        z ^= z >> np.uint64(27)
        z *= np.uint64(0x94D049BB133111EB)
        z ^= z >> np.uint64(31)
        return z


def tensor_seed(suite, index, kind, base_seed=BASE_SEED):
    return (base_seed ^ zlib.crc32(("%s/%d/%s" % (suite, index, kind)).encode())) & 0xFFFFFFFF


def _uniform01(bits):
    return ((bits >> np.uint64(40)).astype(np.float64) + 0.5) * (1.0 / (1 << 24))  # (0, 1), 24 bits


def make_weights(layer, base_seed=BASE_SEED):
    n = layer.K * layer.C * layer.ks * layer.ks
    seed = tensor_seed(layer.suite, layer.index, "w", base_seed)
    u1 = _uniform01(_splitmix64(seed, n))
    u2 = _uniform01(_splitmix64(seed ^ 0xA5A5A5A5, n))
    w = (0.05 * np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)
    w[w == 0] = np.float32(1e-6)  # keep the non-zero count exact
    if layer.mask is not None:
        return np.where(layer.mask, w.reshape(layer.mask.shape), np.float32(0))
    nzero = int(round(layer.sparsity * n))
    keys = _splitmix64(seed ^ 0x3C3C3C3C, n)
    w[np.argsort(keys, kind="stable")[:nzero]] = 0.0
    return w.reshape(layer.K, layer.C, layer.ks, layer.ks)


def make_activations(layer, batch, base_seed=BASE_SEED):
    n = batch * layer.C * layer.H * layer.W
    seed = tensor_seed(layer.suite, layer.index, "x", base_seed)
    x = np.empty(n, np.float32)
    chunk = 1 << 18  # cache-sized pieces: the same values several times faster than one pass over the whole tensor
    for lo in range(0, n, chunk):
        bits = _splitmix64(seed, min(chunk, n - lo), lo)
        v = (bits >> np.uint64(40)).astype(np.float32)
        v *= np.float32(1.0 / (1 << 24))
        v[(bits & np.uint64(1)) == 0] = 0.0
        x[lo:lo + len(v)] = v
    return x.reshape(batch, layer.C, layer.H, layer.W)


def out_hw(layer):
    oh = (layer.H + 2 * layer.pad - layer.ks) // layer.stride + 1
    ow = (layer.W + 2 * layer.pad - layer.ks) // layer.stride + 1
    return oh, ow


def nnz_of(layer):
    if layer.mask is not None:
        return int(layer.mask.sum())
    n = layer.K * layer.C * layer.ks * layer.ks
    return n - int(round(layer.sparsity * n))


def work(layer, batch):
    """Algorithmic work of one launch: HBM bytes (input once, output once, 8 bytes per non-zero), sparse
    and dense-equivalent flops, and which nominal MI355X roof (8 TB/s, 157.3 TFLOP/s vector fp32) binds."""
    oh, ow = out_hw(layer)
    nnz = nnz_of(layer)
    bytes_ = 4 * batch * (layer.C * layer.H * layer.W + layer.K * oh * ow) + 8 * nnz
    fl_sparse = 2 * batch * nnz * oh * ow
    fl_dense = 2 * batch * layer.K * layer.C * layer.ks * layer.ks * oh * ow
    t_hbm = bytes_ / 8e12
    t_fp32 = fl_sparse / 157.3e12
    return dict(bytes=bytes_, flops_sparse=fl_sparse, flops_dense=fl_dense, t_hbm=t_hbm, t_fp32=t_fp32,
                t_roof=max(t_hbm, t_fp32), bound="hbm" if t_hbm >= t_fp32 else "fp32")


def _cycle(values, i):
    return values[i % len(values)]


def single_layer():
    return [Layer("single", 0, "conv_64x128_56_k3", 64, 56, 56, 128, 3, 1, 1, 0.90)]


def vgg19():
    cfg = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56),
           (256, 256, 56), (256, 256, 56), (256, 512, 28), (512, 512, 28), (512, 512, 28), (512, 512, 28),
           (512, 512, 14), (512, 512, 14), (512, 512, 14), (512, 512, 14)]
    out = []
    for i, (c, k, hw) in enumerate(cfg):
        sp = 0.5 if i == 0 else _cycle((0.85, 0.90, 0.95), i - 1)
        out.append(Layer("vgg19", i, "conv%d_%dx%d_%d" % (i, c, k, hw), c, hw, hw, k, 3, 1, 1, sp))
    return out


def resnet50():
    out = []
    sps = (0.80, 0.85, 0.90)

    def add(name, c, hw, k, ks, stride, pad):
        i = len(out)
        out.append(Layer("resnet50", i, name, c, hw, hw, k, ks, stride, pad, _cycle(sps, i)))

    add("stem_7x7", 3, 224, 64, 7, 2, 3)
    cin, hw = 64, 56
    for stage, (width, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3))):
        for b in range(blocks):
            stride = 2 if (b == 0 and stage > 0) else 1
            tag = "s%db%d" % (stage + 1, b)
            add(tag + "_reduce", cin, hw, width, 1, 1, 0)
            add(tag + "_3x3", width, hw, width, 3, stride, 1)
            hw_out = hw // stride
            add(tag + "_expand", width, hw_out, 4 * width, 1, 1, 0)
            if b == 0:
                add(tag + "_proj", cin, hw, 4 * width, 1, stride, 0)
            cin, hw = 4 * width, hw_out
    return out


def mobilenet_v1():
    cfg = [(32, 64, 112), (64, 128, 56), (128, 128, 56), (128, 256, 28), (256, 256, 28), (256, 512, 14)] + \
          [(512, 512, 14)] * 5 + [(512, 1024, 7), (1024, 1024, 7)]
    sps = (0.7, 0.7, 0.7, 0.8, 0.8, 0.8, 0.85, 0.85, 0.9, 0.9, 0.9, 0.9, 0.9)
    return [Layer("mobilenet", i, "pw%d_%dx%d_%d" % (i, c, k, hw), c, hw, hw, k, 1, 1, 0, sps[i])
            for i, (c, k, hw) in enumerate(cfg)]


def yolov3():
    out = []
    sps = (0.80, 0.85, 0.90)

    def add(name, c, hw, k, ks, stride):
        i = len(out)
        out.append(Layer("yolov3", i, name, c, hw, hw, k, ks, stride, ks // 2, _cycle(sps, i)))

    add("conv0", 3, 416, 32, 3, 1)
    c, hw = 32, 416
    for stage, reps in enumerate((1, 2, 8, 8, 4)):
        add("down%d" % stage, c, hw, 2 * c, 3, 2)
        c, hw = 2 * c, hw // 2
        for r in range(reps):
            add("res%d_%d_1x1" % (stage, r), c, hw, c // 2, 1, 1)
            add("res%d_%d_3x3" % (stage, r), c // 2, hw, c, 3, 1)

    def head(tag, cin, mid, hw):
        add(tag + "_a", cin, hw, mid, 1, 1)
        add(tag + "_b", mid, hw, 2 * mid, 3, 1)
        add(tag + "_c", 2 * mid, hw, mid, 1, 1)
        add(tag + "_d", mid, hw, 2 * mid, 3, 1)
        add(tag + "_e", 2 * mid, hw, mid, 1, 1)
        add(tag + "_f", mid, hw, 2 * mid, 3, 1)
        add(tag + "_det", 2 * mid, hw, 255, 1, 1)

    head("head13", 1024, 512, 13)
    add("route13", 512, 13, 256, 1, 1)
    head("head26", 768, 256, 26)
    add("route26", 256, 26, 128, 1, 1)
    head("head52", 384, 128, 52)
    return out


def pruned_suite(npz_path):
    """The layers of a pruned network as recorded in a mask file: `names` (the weight files' names), and per layer
    i `hdr_%02d` (the eight header ints H W IC OC KS PAD STRIDE GROUPS of Tetris/tensor_utils.cc:66) and `bits_%02d`
    (numpy.packbits of `weight != 0` in OIHW order)."""
    z = np.load(npz_path)
    suite = os.path.splitext(os.path.basename(npz_path))[0]
    out = []
    for i, name in enumerate(z["names"]):
        H, Wd, C, K, ks, pad, stride, _ = (int(v) for v in z["hdr_%02d" % i])
        n = K * C * ks * ks
        mask = np.unpackbits(z["bits_%02d" % i])[:n].reshape(K, C, ks, ks).astype(bool)
        out.append(Layer(suite, i, str(name), C, H, Wd, K, ks, stride, pad, 1.0 - float(mask.sum()) / n, mask))
    return out


SUITES = {"single": single_layer, "vgg19": vgg19, "resnet50": resnet50, "mobilenet": mobilenet_v1, "yolov3": yolov3}
