// spconv2d_test <weight_file> [batch] [--seed S] [--dump FILE] [--check]
//
// One source, built once per binary of the reference (its names without the ".o"):
//   spconv2d_test, para_test   Tetris/spconv2d.cc:369-450 with -DBANK_OPTIMIZE -DREORDER_OUT_CHANNEL
//                              (evalution/script/build_all.sh:14, build_ablation.sh:16): the library's path, tile
//                              from its table; prints "Time of Spconv2d :<ms>ms" / "FLOPS of Spconv2d :<x>T"
//   spf_test, bank_sr_test, filter_gr_test, wo_bank_sr_test, wi_bank_sr_test   (-DTETRIS_CLI_SPF)
//                              Tetris/spf.cc:95-176 with no switch, -DBANK_OPTIMIZE, both, -DREORDER_OUT_CHANNEL
//                              alone, both (build_ablation.sh:13-18): the fixed configuration on the SparseFilter's
//                              device arrays; prints "Time of Ablation :<ms>ms"
//   baseline_test              (-DTETRIS_CLI_BASELINE) Tetris/baseline.cc:95-176: the same on the keep-as-is,
//                              CSR-like arrays; prints "Time of Baseline :<ms>ms" / "FLOPS of Baseline :<x>T"
// BANK_OPTIMIZE makes the SparseFilter run Bank-SR, as in the reference.  That pass orders entries for the banks of
// the reference's kernel; what keeps this library's kernel free of LDS bank conflicts is the pitch rule of its LDS
// tiles, so the binaries of the fixed configuration built WITHOUT BANK_OPTIMIZE also switch that rule off
// (TETRIS_OPT_NO_BANK_RULE): the rung "Bank-SR" of the ladder then measures conflict avoidance here as it does there.
//
// Each reads one pruned layer in the reference's text format, makes a random input, runs the host-to-host entry
// point (upload, pack, 30 warm-up + 100 timed launches, download) and prints the reference's lines, so a loop over
// weight files that parses the reference's stdout (evalution/conv2d_timing.py:51-79, ablation_timing.py:15-57) can
// drive it unchanged.
//
// The reference seeds rand() with time(0) (Tetris/spconv2d.cc:377); here the input comes from a
// seeded generator so that a run can be repeated, and --dump writes input and output tensors (raw
// fp32: N*C*H*W inputs, then N*K*OH*OW outputs, both NCHW) for an external checker.  Like the
// reference's shipped builds (BENCHMARK is defined in Tetris/tensor_utils.h:8) no CPU convolution is
// run by default; --check does what the reference's other build does (Tetris/spconv2d.cc:430-440): a dense
// convolution on the host, "HostConv2d begin" / "HostConv2d end", then "Sparse Pass." or "Sparse Error.".
#include <hip/hip_runtime_api.h>

#include <cassert>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>

#include "tetris_spconv2d.hpp"  // BANK_OPTIMIZE / REORDER_OUT_CHANNEL come from the build line, as in the reference

namespace {

struct SplitMix64 {
  uint64_t s;
  uint64_t next() {
    uint64_t z = (s += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
  }
};

// uniform in [-1, 1), the range of the reference's RandFloat (Tetris/tensor_utils.cc:9-14)
void GenRandTensor(float* t, size_t len, uint64_t seed) {
  SplitMix64 g{seed};
  for (size_t i = 0; i < len; ++i) t[i] = static_cast<float>(g.next() >> 40) * (2.0f / 16777216.0f) - 1.0f;
}

#define CLI_HIP(call)                                                                              \
  do {                                                                                             \
    hipError_t e_ = (call);                                                                        \
    if (e_ != hipSuccess) {                                                                        \
      std::fprintf(stderr, "HIP error at %s %d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
      std::exit(EXIT_FAILURE);                                                                     \
    }                                                                                              \
  } while (0)

}  // namespace

int main(int argc, char* argv[]) {
  std::cout << "args : " << argc;
  for (int i = 0; i < argc; ++i) std::cout << " " << argv[i];
  std::cout << "\n\n";

  std::string weight_file, dump;
  bool check = false;
  int batch_size = 4;
  uint64_t seed = 1;
  int positional = 0;
  for (int i = 1; i < argc; ++i) {
    if (!std::strcmp(argv[i], "--seed") && i + 1 < argc) {
      seed = std::strtoull(argv[++i], nullptr, 10);
    } else if (!std::strcmp(argv[i], "--dump") && i + 1 < argc) {
      dump = argv[++i];
    } else if (!std::strcmp(argv[i], "--check")) {
      check = true;
    } else if (positional == 0) {
      weight_file = argv[i];
      ++positional;
    } else if (positional == 1) {
      batch_size = std::atoi(argv[i]);
      ++positional;
    } else {
      std::fprintf(stderr, "usage: %s <weight_file> [batch] [--seed S] [--dump FILE] [--check]\n", argv[0]);
      return 2;
    }
  }
  if (weight_file.empty() || batch_size <= 0) {
    std::fprintf(stderr, "usage: %s <weight_file> [batch] [--seed S] [--dump FILE] [--check]\n", argv[0]);
    return 2;
  }

  const int dev_id = 0;
  hipDeviceProp_t prop;
  CLI_HIP(hipSetDevice(dev_id));
  CLI_HIP(hipGetDeviceProperties(&prop, dev_id));
  std::printf("GPU Device %d: \"%s\" (%s, %d compute units)\n\n", dev_id, prop.name, prop.gcnArchName,
              prop.multiProcessorCount);
  std::fflush(stdout);

  const std::string layout = "NHWC";  // what the reference's mains pass; host tensors stay NCHW
  const bool apply_reorder = true;
  int in_channel, img_h, img_w, kernel_size, out_channel, stride, padding, groups;
  float* h_filter = ReadConfigAndDataFromFile(weight_file, batch_size, layout, img_h, img_w, in_channel, out_channel,
                                              kernel_size, stride, padding, groups);

  const int out_h = (img_h + padding * 2 - kernel_size) / stride + 1;
  const int out_w = (img_w + padding * 2 - kernel_size) / stride + 1;
  const size_t n_in = (size_t)batch_size * in_channel * img_h * img_w;
  const size_t n_out = (size_t)batch_size * out_h * out_w * out_channel;
  float* h_input = static_cast<float*>(std::malloc(n_in * sizeof(float)));
  float* h_sparse = static_cast<float*>(std::malloc(n_out * sizeof(float)));
  if (!h_input || !h_sparse) {
    std::fprintf(stderr, "out of host memory\n");
    return 1;
  }
  GenRandTensor(h_input, n_in, seed);

  hipStream_t stream;
  CLI_HIP(hipStreamCreate(&stream));
#if (defined(TETRIS_CLI_SPF) || defined(TETRIS_CLI_BASELINE)) && !defined(BANK_OPTIMIZE)
  if (tetris_options_set(tetris_options_get() | TETRIS_OPT_NO_BANK_RULE) != TETRIS_OK) {
    std::fprintf(stderr, "%s\n", tetris_last_error());
    return 1;
  }
#endif
#if defined(TETRIS_CLI_BASELINE)
  SparseConv2d_Baseline<float, int, int>(h_input, h_filter, h_sparse, batch_size, img_h, img_w, in_channel, out_channel,
                                         kernel_size, stride, padding, stream, layout, false);
#elif defined(TETRIS_CLI_SPF)
  SparseConv2d_SPF<float, int, int>(h_input, h_filter, h_sparse, batch_size, img_h, img_w, in_channel, out_channel,
                                    kernel_size, stride, padding, stream, layout, apply_reorder);
#else
  CudaSparseConv2d<float, int, int>(h_input, h_filter, h_sparse, batch_size, img_h, img_w, in_channel, out_channel,
                                    kernel_size, stride, padding, stream, layout, apply_reorder);
#endif
  CLI_HIP(hipStreamDestroy(stream));

  int exit_code = 0;
  if (check) {  // what the reference's mains do when not built with -DBENCHMARK (Tetris/spconv2d.cc:430-440)
    float* h_check = static_cast<float*>(std::malloc(n_out * sizeof(float)));
    if (!h_check) {
      std::fprintf(stderr, "out of host memory\n");
      return 1;
    }
    std::cout << "HostConv2d begin\n";
    HostConv2d(h_input, h_filter, h_check, batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride,
               padding);
    std::cout << "HostConv2d end\n";
    const bool same = TensorEqual(h_sparse, h_check, n_out);
    std::cout << (same ? "Sparse Pass.\n" : "Sparse Error.\n");
    std::free(h_check);
    if (!same) exit_code = 3;  // the reference only prints the verdict; a script gets it from the exit status here
  }

  if (!dump.empty()) {
    FILE* fp = std::fopen(dump.c_str(), "wb");
    if (!fp || std::fwrite(h_input, sizeof(float), n_in, fp) != n_in ||
        std::fwrite(h_sparse, sizeof(float), n_out, fp) != n_out) {
      std::fprintf(stderr, "cannot write %s\n", dump.c_str());
      return 1;
    }
    std::fclose(fp);
  }
  std::free(h_input);
  std::free(h_filter);
  std::free(h_sparse);
  return exit_code;
}
