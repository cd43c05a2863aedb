"""Per-layer vendor baselines on this machine, one process per layer like the reference's cudnn_test.o and
cusparse_test.o (Tetris/cudnn_test.cc, Tetris/cuda_utils.cc:6-132; Tetris/cusparse_test.cc:49-246):

    python -m tetris_amd.vendor_test dense <weight_file> [batch]     # the vendor's dense convolution (MIOpen via torch)
    python -m tetris_amd.vendor_test csr   <weight_file> [batch]     # im2col + CSR x dense (rocSPARSE via torch)

Reads a weight file in the reference's text format, makes a seeded input, times the operation with the reference's
protocol (warm-up launches, then timed launches between two events; Tetris/tensor_utils.h:10-11: 30 + 100 -- the CSR
path runs 3 + 10, it is two orders of magnitude slower) and prints the lines the reference's harness reads
(evalution/conv2d_timing.py:51-79): `[Config] ...`, `Time of <vendor> :<ms>ms`, `FLOPS of <vendor> :<x>T` (dense-
equivalent operations / 1024^4, as Tetris/cuda_utils.cc:116).  The zeros of the filter stay in for the dense path; the
CSR path multiplies the K x (C*ks*ks) CSR filter with the unfolded input, image by image (cusparse_test.cc:147-173 does
the same with cusparseSpMM).  These are context figures, not part of the library: PyTorch is what reaches the vendor
libraries here.
"""
import sys


def main(argv=None):
    argv = list(sys.argv[1:] if argv is None else argv)
    print("args : %d %s\n" % (len(argv) + 1, " ".join(["vendor_test"] + argv)))
    check = "--check" in argv
    argv = [a for a in argv if a != "--check"]
    if len(argv) < 2 or argv[0] not in ("dense", "csr"):
        sys.stderr.write("usage: python -m tetris_amd.vendor_test dense|csr <weight_file> [batch] [--check]\n")
        return 2
    kind, weight_file = argv[0], argv[1]
    batch = int(argv[2]) if len(argv) > 2 else 4
    import numpy as np
    import torch
    import torch.nn.functional as F
    import tetris_amd as T

    try:
        h, w, nnz = T.ReadConfigAndDataFromFile(weight_file)
    except T.TetrisError:
        print("Open file error.")
        return 1
    H, Wd, C, K, ks, pad, stride = h["H"], h["W"], h["IC"], h["OC"], h["KS"], h["PAD"], h["STRIDE"]
    print("[Config] sparsity = %g, nnz = %d, batch_size = %d, img_h = %d, img_w = %d, in_channel = %d, out_channel = %d, "
          "kernel_size = %d, padding = %d, stride = %d\n" % (1.0 - nnz / float(K * C * ks * ks), nnz, batch, H, Wd, C, K, ks,
                                                           pad, stride), flush=True)
    if not torch.cuda.is_available():
        sys.stderr.write("vendor_test needs a GPU\n")
        return 1
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(1)
    x = torch.from_numpy(rng.random((batch, C, H, Wd), dtype=np.float32) * 2 - 1).to(dev)
    wt = torch.from_numpy(w).to(dev)
    oh, ow = (H + 2 * pad - ks) // stride + 1, (Wd + 2 * pad - ks) // stride + 1
    if kind == "dense":
        name, warm, repeat = "MIOpen", 30, 100

        def run():
            return F.conv2d(x, wt, None, stride, pad)
    else:
        name, warm, repeat = "Rocsparse", 3, 10
        a = wt.reshape(K, -1).to_sparse_csr()

        def run():
            y = None
            for n in range(batch):  # one image at a time keeps the unfolded matrix small (C*ks*ks x OH*OW)
                y = torch.sparse.mm(a, F.unfold(x[n:n + 1], ks, padding=pad, stride=stride)[0])
            return y
    for _ in range(warm):
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(repeat):
        y = run()
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / repeat
    print("Time of %s :%gms" % (name, ms))
    print("FLOPS of %s :%gT" % (name, oh * ow * batch * K * C * ks * ks * 2 * 1000 / ms / 1024 ** 4))
    if check:  # the dense result against the last image of the CSR product, or itself: a sanity line
        ref = F.conv2d(x[-1:], wt, None, stride, pad)[0].reshape(K, -1)
        got = y[-1].reshape(K, -1) if kind == "dense" else y
        err = float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-6))
        print("Sparse Pass." if err <= 1e-3 else "Sparse Error.")
        return 0 if err <= 1e-3 else 3
    return 0


if __name__ == "__main__":
    sys.exit(main())
