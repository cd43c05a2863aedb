// TEST INFRASTRUCTURE ONLY -- C entry points around the reference's own tensor_utils.cc, which is
// compiled unmodified from the reference checkout into oracle/_ref/ (see oracle/Makefile).  It gives
// tests and the benchmark's cpu_baseline leg the reference's HostConv2d, FloatEqual and weight-file
// reader as they are, to check the restatement in tetris_oracle.cpp against.
#include <cstdint>
#include <cstdlib>
#include <string>

#include "tensor_utils.h"  // from the reference checkout (-I<reference>/Tetris)

extern "C" {

void ref_host_conv2d(float* input, float* filter, float* output, int N, int H, int W, int C, int K, int ks,
                     int stride, int pad) {
  HostConv2d(input, filter, output, N, H, W, C, K, ks, stride, pad);
}

int ref_float_equal(float x, float y) { return FloatEqual(x, y) ? 1 : 0; }

// hdr: H W IC OC KS PAD STRIDE GROUPS.  The reference prints its "[Config] ..." line to stdout.
float* ref_read_weight_file(const char* path, int batch, int32_t* hdr) {
  int h, w, ic, oc, ks, stride, pad, groups;
  float* f = ReadConfigAndDataFromFile(std::string(path), batch, std::string("NHWC"), h, w, ic, oc, ks, stride, pad,
                                       groups);
  hdr[0] = h; hdr[1] = w; hdr[2] = ic; hdr[3] = oc; hdr[4] = ks; hdr[5] = pad; hdr[6] = stride; hdr[7] = groups;
  return f;
}

void ref_free(void* p) { free(p); }

void ref_nchw2nhwc(float* t, int N, int C, int H, int W) { NCHW2NHWC(t, N, C, H, W); }
void ref_nhwc2nchw(float* t, int N, int C, int H, int W) { NHWC2NCHW(t, N, C, H, W); }
}
