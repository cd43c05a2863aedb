"""Writes the committed fixtures under tests/golden/ from the reference checkout (run in the build container).

* weights_*.npz   five shipped pruned layers, parsed by the reference's own ReadConfigAndDataFromFile
                  (tensor_utils.cc:55-82, compiled unmodified into oracle/_ref) -- data files, stored as float32
                  arrays plus the eight header ints.
* masks_*.npz     the zero patterns of every shipped layer of five pruned networks (VGG19 at 92 %, MobileNetV1 at
                  86 %, ResNet-50 at 90 % and at 98 %, YOLOv3 at 89 %, the loop of evalution/conv2d_timing.py:136-176):
                  per layer the eight header ints and numpy.packbits(weight != 0), plus the file names.
                  tetris_amd.workloads.pruned_suite() turns them into benchmark layers with seeded values.
* spf_known_answers.json is NOT produced here: it is the table of FNV-1a-64 hashes and array sizes that was
  recorded from the compiled reference SparseFilter (spconv2d_utils.h) for these layers; the reference's CUDA
  headers are absent from this image so that class cannot be rebuilt here.

usage: python tests/golden/make_golden.py [/root/reference]
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import oracle_py as O  # noqa: E402

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
D = os.path.join(REF, "evalution", "conv_weight_data")
FILES = {
    "rn90_3x3": "resnet50/ResNet50-magnitude-90-acc-73.91/module8_0_module3_1_conv2d_0_H_56_W_56_IC_64_OC_64_KS_3_Pad_1_S_1_G_1",
    "rn90_stem": "resnet50/ResNet50-magnitude-90-acc-73.91/conv2d_0_H_224_W_224_IC_3_OC_64_KS_7_Pad_3_S_2_G_1",
    "rn98_1x1": "resnet50/ResNet50-magnitude-98-acc-57.90/module8_0_module3_0_conv2d_0_H_56_W_56_IC_64_OC_64_KS_1_Pad_0_S_1_G_1",
    "vgg_64x128": "vgg19/vgg19-92-acc-71.7/module3_0_conv2d_0_H_112_W_112_IC_64_OC_128_KS_3_Pad_1_S_1_G_1",
    "yolo_255": "yolov3/yolov3-89-acc-62.4/module61_0_conv2d_0_H_80_W_80_IC_256_OC_255_KS_1_Pad_0_S_1_G_1",
}
# present only in the reference checkout (3 MB of text each): used by tests when /root/reference exists
BIG_FILES = {
    "yolo_1024": "yolov3/yolov3-89-acc-62.4/module74_0_module5_0_conv2d_0_H_20_W_20_IC_1024_OC_512_KS_1_Pad_0_S_1_G_1",
    "vgg_256": "vgg19/vgg19-92-acc-71.7/module8_0_module2_0_conv2d_3_H_56_W_56_IC_256_OC_256_KS_3_Pad_1_S_1_G_1",
}

MASK_DIRS = {"vgg19_92": "vgg19/vgg19-92-acc-71.7", "mobilenet_86": "mobilenet/mobilenet-86-acc-70.1",
             "resnet50_90": "resnet50/ResNet50-magnitude-90-acc-73.91", "resnet50_98": "resnet50/ResNet50-magnitude-98-acc-57.90",
             "yolov3_89": "yolov3/yolov3-89-acc-62.4"}


def write_masks(tag, rel):
    names = sorted(os.listdir(os.path.join(D, rel)))
    arrays = {}
    for i, fn in enumerate(names):
        hdr, w = O.ref_read_weight_file(os.path.join(D, rel, fn))
        arrays["hdr_%02d" % i] = np.array([hdr[k] for k in ("H", "W", "IC", "OC", "KS", "PAD", "STRIDE", "GROUPS")], np.int32)
        arrays["bits_%02d" % i] = np.packbits((w != 0).reshape(-1))
    out = os.path.join(HERE, "masks_%s.npz" % tag)
    np.savez_compressed(out, names=np.array(names), source=np.array(rel), **arrays)
    print(tag, len(names), "layers", os.path.getsize(out))


if __name__ == "__main__":
    assert O.ref_available(), "build oracle/_ref first: make -C oracle"
    for tag, rel in MASK_DIRS.items():
        write_masks(tag, rel)
    for name, rel in FILES.items():
        hdr, w = O.ref_read_weight_file(os.path.join(D, rel))
        header = np.array([hdr[k] for k in ("H", "W", "IC", "OC", "KS", "PAD", "STRIDE", "GROUPS")], np.int32)
        out = os.path.join(HERE, "weights_%s.npz" % name)
        np.savez_compressed(out, header=header, filter=w, source=np.array(rel))
        print(name, w.shape, int((w != 0).sum()), os.path.getsize(out))
