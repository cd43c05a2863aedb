// Header-only C++ face of libtetris_spconv2d.so with the reference's own names, so that a main written
// against Tetris/spconv2d_kernel.cuh and Tetris/spconv2d_utils.h compiles after swapping the include
// and spelling the stream type hipStream_t.
//
//   SparseFilter<V,O,P>      Tetris/spconv2d_utils.h:23-515   (constructor, getters, public vectors)
//   SparseConv2d<V,O,P,...>  Tetris/spconv2d_kernel.cuh:14-21 (launcher on the filter's device arrays)
//   CudaSparseConv2d<V,O,P>  Tetris/spconv2d_kernel.cuh:7-12, Tetris/spconv2d.cc:332-367
//   SparseConv2d_SPF<V,O,P>  Tetris/spf.cc:22-93
//   SparseConv2d_Baseline<V,O,P>  Tetris/baseline.cc:22-93
//   ReadConfigAndDataFromFile, PrintConv2dConfig, FloatEqual, TensorEqual   Tetris/tensor_utils.cc:17-82
//
// Only <float, int, int> exists, as in the reference (Tetris/spconv2d.cc:427, spconv2d_kernel.cu:197-200).
// Error behaviour follows the reference: a failing call prints the library's message and exits
// (Tetris/cuda_utils.h:9-16); "Open file error." + exit(1) for an unreadable weight file
// (Tetris/tensor_utils.cc:61-64).
//
// Differences a caller can see: device tensors are NCHW (the reference keeps NHWC on the device; the
// host entry points take and return NCHW in both); the TILE_H/TILE_W template arguments of
// SparseConv2d are accepted and ignored (tile shapes are chosen by the library); the preprocessor
// switches BANK_OPTIMIZE and REORDER_OUT_CHANNEL select the same variants as in the reference.
#ifndef TETRIS_SPCONV2D_HPP_
#define TETRIS_SPCONV2D_HPP_

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <type_traits>
#include <vector>

#include "tetris_spconv2d.h"

namespace tetris_detail {
inline void check(int rc, const char* file, int line) {
  if (rc != TETRIS_OK) {
    std::fprintf(stderr, "tetris error at %s %d: %s\n", file, line, tetris_last_error());
    std::exit(EXIT_FAILURE);
  }
}
inline unsigned build_flags() {
  unsigned f = 0;
#ifdef BANK_OPTIMIZE
  f |= TETRIS_BANK_OPTIMIZE;
#endif
#ifdef REORDER_OUT_CHANNEL
  f |= TETRIS_REORDER_OUT_CHANNEL;
#endif
  return f;
}
}  // namespace tetris_detail
#define TETRIS_CHECK(call) ::tetris_detail::check((call), __FILE__, __LINE__)

template <typename ValueType, typename OffsetType, typename PositionType>
struct SparseFilter {
  static_assert(std::is_same<ValueType, float>::value && sizeof(OffsetType) == 4 && sizeof(PositionType) == 4,
                "only SparseFilter<float, int, int> exists");

  SparseFilter(float* filter, int in_channel, int out_channel, int kernel_size, int TILE_IC = 32,
               bool apply_reorder = false, bool apply_vectorize = true)
      : in_channel_(in_channel), out_channel_(out_channel), kernel_size_(kernel_size), TILE_IC_(TILE_IC) {
    TETRIS_CHECK(tetris_spf_create(filter, in_channel, out_channel, kernel_size, TILE_IC, apply_reorder,
                                   apply_vectorize, tetris_detail::build_flags(), &handle_));
    tetris_spf_arrays h{};
    TETRIS_CHECK(tetris_spf_host_arrays(handle_, &h));
    nnz_ = static_cast<int>(h.nnz);
    offsets_.assign(h.offsets, h.offsets + h.n_offsets);
    stage_len_.assign(h.stage_len, h.stage_len + h.n_stage_len);
    position_.assign(h.position, h.position + h.n_position);
    values_.assign(h.values, h.values + h.n_values);
    oc_permutation_.assign(h.oc_permutation, h.oc_permutation + h.n_oc_permutation);
    tetris_spf_arrays d{};
    TETRIS_CHECK(tetris_spf_device_arrays(handle_, &d));  // the reference uploads in the constructor
    d_offsets_ = const_cast<OffsetType*>(reinterpret_cast<const OffsetType*>(d.offsets));
    d_stage_len_ = const_cast<OffsetType*>(reinterpret_cast<const OffsetType*>(d.stage_len));
    d_position_ = const_cast<PositionType*>(reinterpret_cast<const PositionType*>(d.position));
    d_oc_permutation_ = const_cast<PositionType*>(reinterpret_cast<const PositionType*>(d.oc_permutation));
    d_values_ = const_cast<ValueType*>(d.values);
  }
  ~SparseFilter() { tetris_spf_destroy(handle_); }
  SparseFilter(const SparseFilter&) = delete;
  SparseFilter& operator=(const SparseFilter&) = delete;

  OffsetType* GetDeviceOffsets() { return d_offsets_; }
  OffsetType* GetDeviceStageLen() { return d_stage_len_; }
  ValueType* GetDeviceValues() { return d_values_; }
  PositionType* GetDevicePosition() { return d_position_; }
  PositionType* GetDeviceOCPermutation() { return d_oc_permutation_; }
  int GetTileIC() { return TILE_IC_; }

  int in_channel_, out_channel_, kernel_size_;
  int nnz_ = 0;
  int TILE_IC_;
  std::vector<OffsetType> oc_permutation_;
  std::vector<OffsetType> stage_len_;
  std::vector<OffsetType> offsets_;
  std::vector<PositionType> position_;
  std::vector<ValueType> values_;
  OffsetType* d_offsets_ = nullptr;
  OffsetType* d_stage_len_ = nullptr;
  PositionType* d_position_ = nullptr;
  PositionType* d_oc_permutation_ = nullptr;
  ValueType* d_values_ = nullptr;

 private:
  tetris_spf* handle_ = nullptr;
};

// Computes from the device arrays passed (offsets, positions, values, permutation), as the reference launcher does.
// With TILE_IC given (the reference's callers always give the SparseFilter's own, Tetris/spf.cc:59-60) any arrays in
// the SparseFilter layout work; without it they must belong to a live SparseFilter, whose TILE_IC is then looked up
// through `values`.  TILE_H / TILE_W are accepted and ignored: the library picks its tile.  `input` and `output`
// are NCHW device tensors.  The call hashes the arrays on the device and synchronises `stream` (a caller may have
// rewritten them in place); the kernels run asynchronously.
template <typename ValueType, typename OffsetType, typename PositionType, int KERNEL_SIZE = 0, int STRIDE = 0,
          int TILE_IC = 0, int TILE_H = 0, int TILE_W = 0, typename Stream = void*>
void SparseConv2d(ValueType* input, OffsetType* offsets, OffsetType* stage_len, PositionType* oc_permutation,
                  PositionType* position, ValueType* values, ValueType* output, int batch_size, int img_h, int img_w,
                  int in_channel, int out_channel, int kernel_size, int stride, int padding, Stream stream) {
  if (TILE_IC > 0)
    TETRIS_CHECK(tetris_spconv2d_launch_spf_arrays(
        input, reinterpret_cast<const int32_t*>(offsets), reinterpret_cast<const int32_t*>(stage_len),
        reinterpret_cast<const int32_t*>(oc_permutation), reinterpret_cast<const int32_t*>(position), values, output,
        batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride, padding, TILE_IC, 4, /*n_entries unknown*/ 0, nullptr,
        reinterpret_cast<void*>(stream)));
  else
    TETRIS_CHECK(tetris_spconv2d_launch_spf(input, reinterpret_cast<const int32_t*>(offsets),
                                            reinterpret_cast<const int32_t*>(stage_len),
                                            reinterpret_cast<const int32_t*>(oc_permutation),
                                            reinterpret_cast<const int32_t*>(position), values, output, batch_size,
                                            img_h, img_w, in_channel, out_channel, kernel_size, stride, padding,
                                            reinterpret_cast<void*>(stream)));
}

// Prints the two result lines of the reference (Tetris/spconv2d.cc:357-358): milliseconds per launch and the
// dense-equivalent rate divided by 1024^4.
template <typename ValueType, typename OffsetType, typename PositionType, typename Stream = void*>
void CudaSparseConv2d(float* h_input, float* h_filter, float* h_output, int batch_size, int img_h, int img_w,
                      int in_channel, int out_channel, int kernel_size, int stride, int padding, Stream stream,
                      std::string layout, bool apply_reorder) {
  float ms = 0.f;
  TETRIS_CHECK(tetris_spconv2d_host(h_input, h_filter, h_output, batch_size, img_h, img_w, in_channel, out_channel,
                                    kernel_size, stride, padding, reinterpret_cast<void*>(stream), layout.c_str(),
                                    apply_reorder, &ms));
  const int out_h = (img_h + padding * 2 - kernel_size) / stride + 1;
  const int out_w = (img_w + padding * 2 - kernel_size) / stride + 1;
  std::cout << "Time of Spconv2d :" << ms << "ms"
            << "\n";
  std::cout << "FLOPS of Spconv2d :"
            << (long long)out_h * out_w * batch_size * out_channel * in_channel * kernel_size * kernel_size * 2 * 1000 /
                   (ms) / 1024 / 1024 / 1024 / 1024
            << "T\n";
}

// Prints "Time of Ablation :<ms>ms" and "FLOPS of Ablation :<x>T" like Tetris/spf.cc:83-84.
template <typename ValueType, typename OffsetType, typename PositionType, typename Stream = void*>
void SparseConv2d_SPF(float* h_input, float* h_filter, float* h_output, int batch_size, int img_h, int img_w,
                      int in_channel, int out_channel, int kernel_size, int stride, int padding, Stream stream,
                      std::string layout, bool apply_reorder) {
  float ms = 0.f;
  TETRIS_CHECK(tetris_spconv2d_spf_host(h_input, h_filter, h_output, batch_size, img_h, img_w, in_channel,
                                        out_channel, kernel_size, stride, padding, reinterpret_cast<void*>(stream),
                                        layout.c_str(), apply_reorder, tetris_detail::build_flags(), &ms));
  const int out_h = (img_h + padding * 2 - kernel_size) / stride + 1;
  const int out_w = (img_w + padding * 2 - kernel_size) / stride + 1;
  std::cout << "Time of Ablation :" << ms << "ms"
            << "\n";
  std::cout << "FLOPS of Ablation :"
            << (long long)out_h * out_w * batch_size * out_channel * in_channel * kernel_size * kernel_size * 2 * 1000 /
                   (ms) / 1024 / 1024 / 1024 / 1024
            << "T\n";
}

// Prints "Time of Baseline :<ms>ms" and "FLOPS of Baseline :<x>T" like Tetris/baseline.cc:82-83.
template <typename ValueType, typename OffsetType, typename PositionType, typename Stream = void*>
void SparseConv2d_Baseline(float* h_input, float* h_filter, float* h_output, int batch_size, int img_h, int img_w,
                           int in_channel, int out_channel, int kernel_size, int stride, int padding, Stream stream,
                           std::string layout, bool /*apply_reorder*/) {
  float ms = 0.f;
  TETRIS_CHECK(tetris_spconv2d_baseline_host(h_input, h_filter, h_output, batch_size, img_h, img_w, in_channel,
                                             out_channel, kernel_size, stride, padding,
                                             reinterpret_cast<void*>(stream), layout.c_str(), &ms));
  const int out_h = (img_h + padding * 2 - kernel_size) / stride + 1;
  const int out_w = (img_w + padding * 2 - kernel_size) / stride + 1;
  std::cout << "Time of Baseline :" << ms << "ms"
            << "\n";
  std::cout << "FLOPS of Baseline :"
            << (long long)out_h * out_w * batch_size * out_channel * in_channel * kernel_size * kernel_size * 2 * 1000 /
                   (ms) / 1024 / 1024 / 1024 / 1024
            << "T\n";
}

inline void PrintConv2dConfig(int64_t nnz, int batch_size, std::string /*layout*/, int img_h, int img_w, int in_channel,
                              int out_channel, int kernel_size, int stride, int padding, int /*groups*/) {
  std::cout << "[Config] sparsity = "
            << (1.0 - nnz * 1.0 / (int64_t)(out_channel * in_channel * kernel_size * kernel_size)) << ", nnz = " << nnz
            << ", batch_size = " << batch_size << ", img_h = " << img_h << ", img_w = " << img_w
            << ", in_channel = " << in_channel << ", out_channel = " << out_channel
            << ", kernel_size = " << kernel_size << ", padding = " << padding << ", stride = " << stride << "\n\n";
}

// The returned filter is malloc'ed; release it with free(), as the reference's mains do.
inline float* ReadConfigAndDataFromFile(std::string weight_file, int batch_size, std::string layout, int& img_h,
                                        int& img_w, int& in_channel, int& out_channel, int& kernel_size, int& stride,
                                        int& padding, int& groups) {
  int32_t h[8];
  float* filter = nullptr;
  int64_t nnz = 0;
  const int rc = tetris_read_weight_file(weight_file.c_str(), h, &filter, &nnz);
  if (rc == TETRIS_EIO) {
    std::cout << "Open file error.\n";
    std::exit(1);
  }
  TETRIS_CHECK(rc);
  img_h = h[0]; img_w = h[1]; in_channel = h[2]; out_channel = h[3];
  kernel_size = h[4]; padding = h[5]; stride = h[6]; groups = h[7];
  PrintConv2dConfig(nnz, batch_size, layout, img_h, img_w, in_channel, out_channel, kernel_size, stride, padding,
                    groups);
  return filter;
}

inline bool FloatEqual(float x, float y) { return tetris_float_equal(x, y) != 0; }
inline bool TensorEqual(float* tensor_x, float* tensor_y, size_t len) {
  const int64_t at = tetris_tensor_first_mismatch(tensor_x, tensor_y, static_cast<int64_t>(len));
  if (at >= 0) {  // the reference prints the first differing pair (Tetris/tensor_utils.cc:24-26)
    std::cout << "pos = " << at << ", value_x = " << tensor_x[at] << ", value_y = " << tensor_y[at] << "\n";
    return false;
  }
  return true;
}

// Dense direct convolution on the host, for checking a result the way the reference's mains do when they are not
// built for benchmarking (HostConv2d, Tetris/tensor_utils.cc:136-170; used at Tetris/spconv2d.cc:430-440): NCHW
// input, OIHW filter, NCHW output, zero padding, every output summed over (ic, row, column) in that order.  It is a
// checker: nothing in the library calls it.
inline void HostConv2d(const float* input, const float* filter, float* output, int batch_size, int img_h, int img_w,
                       int in_channel, int out_channel, int kernel_size, int stride, int padding) {
  const int out_h = (img_h + 2 * padding - kernel_size) / stride + 1;
  const int out_w = (img_w + 2 * padding - kernel_size) / stride + 1;
  for (int n = 0; n < batch_size; ++n)
    for (int k = 0; k < out_channel; ++k)
      for (int oy = 0; oy < out_h; ++oy)
        for (int ox = 0; ox < out_w; ++ox) {
          float sum = 0.f;
          for (int c = 0; c < in_channel; ++c) {
            const float* plane = input + (static_cast<size_t>(n) * in_channel + c) * img_h * img_w;
            const float* taps = filter + (static_cast<size_t>(k) * in_channel + c) * kernel_size * kernel_size;
            for (int r = 0; r < kernel_size; ++r) {
              const int iy = oy * stride - padding + r;
              if (iy < 0 || iy >= img_h) continue;
              for (int t = 0; t < kernel_size; ++t) {
                const int ix = ox * stride - padding + t;
                if (ix < 0 || ix >= img_w) continue;
                sum += plane[iy * img_w + ix] * taps[r * kernel_size + t];
              }
            }
          }
          output[((static_cast<size_t>(n) * out_channel + k) * out_h + oy) * out_w + ox] = sum;
        }
}

#endif  // TETRIS_SPCONV2D_HPP_
