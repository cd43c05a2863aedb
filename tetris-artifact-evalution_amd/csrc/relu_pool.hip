// ReLU and ReLU + 2x2 max-pooling between two convolution layers, so that a stack of sparse layers runs as a whole
// network (each layer's input is the activation of the one before).  The reference times its layers one by one on
// random inputs (Tetris/spconv2d.cc:369-450) and has no such pass; this is the glue a whole-network run needs.
// One pass over the tensor, bound by HBM: 4 bytes read per input element, 4 written per output element.
#include <algorithm>

#include "common.h"

namespace tetris {
namespace {

// out[i] = max(in[i], 0) over n floats; 16 bytes per lane when the pointers allow it
__global__ __launch_bounds__(256) void relu_kernel(const float* __restrict__ in, float* __restrict__ out, long long n,
                                                   int vec) {
  const long long step = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (vec) {
    const float4* in4 = reinterpret_cast<const float4*>(in);
    float4* out4 = reinterpret_cast<float4*>(out);
    for (long long i = t; i < (n >> 2); i += step) {
      float4 v = in4[i];
      v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f); v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f);
      out4[i] = v;
    }
    for (long long i = (n & ~3ll) + t; i < n; i += step) out[i] = fmaxf(in[i], 0.f);
  } else {
    for (long long i = t; i < n; i += step) out[i] = fmaxf(in[i], 0.f);
  }
}

// out[p][y][x] = max(0, in[p][2y..2y+1][2x..2x+1]) for planes p of H x W floats; OH = H / 2, OW = W / 2 (an odd last
// row or column is dropped).  A thread makes two neighbouring outputs from two 16-byte loads when W is a multiple of
// four and the pointers are aligned (vec), else one output from four scalar loads.
__global__ __launch_bounds__(256) void relu_pool2_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                         long long planes, int H, int W, int vec) {
  const int OH = H >> 1, OW = W >> 1;
  const long long step = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (vec) {
    const int pairs = OW >> 1;  // output pairs per row
    const long long total = planes * OH * pairs;
    for (long long i = t; i < total; i += step) {
      const long long row = i / pairs;  // plane * OH + y
      const int xp = (int)(i - row * pairs);
      const long long p = row / OH;
      const int y = (int)(row - p * OH);
      const float* src = in + (p * H + 2 * y) * W + 4 * xp;
      const float4 a = *reinterpret_cast<const float4*>(src);
      const float4 b = *reinterpret_cast<const float4*>(src + W);
      float2 r;
      r.x = fmaxf(fmaxf(fmaxf(a.x, a.y), fmaxf(b.x, b.y)), 0.f);
      r.y = fmaxf(fmaxf(fmaxf(a.z, a.w), fmaxf(b.z, b.w)), 0.f);
      *reinterpret_cast<float2*>(out + row * OW + 2 * xp) = r;
    }
  } else {
    const long long total = planes * OH * OW;
    for (long long i = t; i < total; i += step) {
      const long long row = i / OW;
      const int x = (int)(i - row * OW);
      const long long p = row / OH;
      const int y = (int)(row - p * OH);
      const float* src = in + (p * H + 2 * y) * W + 2 * x;
      out[i] = fmaxf(fmaxf(fmaxf(src[0], src[1]), fmaxf(src[W], src[W + 1])), 0.f);
    }
  }
}

}  // namespace
}  // namespace tetris

extern "C" int tetris_relu_maxpool(const float* d_input, float* d_output, int batch, int channels, int img_h, int img_w,
                                   int pool, void* stream) {
  using namespace tetris;
  if (!d_input || !d_output) return fail(TETRIS_EINVAL, "null argument");
  if (batch <= 0 || channels <= 0 || img_h <= 0 || img_w <= 0)
    return fail(TETRIS_EINVAL, "bad tensor shape %d x %d x %d x %d", batch, channels, img_h, img_w);
  if (pool != 1 && pool != 2) return fail(TETRIS_EINVAL, "pool must be 1 (ReLU only) or 2 (ReLU + 2x2 max-pooling), got %d", pool);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long long planes = (long long)batch * channels;
  const bool aligned = ((reinterpret_cast<size_t>(d_input) | reinterpret_cast<size_t>(d_output)) & 15) == 0;
  if (pool == 1) {
    const long long n = planes * img_h * img_w;
    const int blocks = (int)std::min<long long>(((n + 3) / 4 + 255) / 256, 8192);
    hipLaunchKernelGGL(relu_kernel, dim3(blocks), dim3(256), 0, s, d_input, d_output, n, aligned ? 1 : 0);
  } else {
    if (img_h < 2 || img_w < 2) return fail(TETRIS_EINVAL, "2x2 pooling needs an image of at least 2 x 2");
    const int vec = aligned && (img_w & 3) == 0;  // rows then start 16-byte aligned and output rows 8-byte aligned
    const long long items = planes * (img_h / 2) * (vec ? img_w / 4 : img_w / 2);
    const int blocks = (int)std::min<long long>((items + 255) / 256, 8192);
    hipLaunchKernelGGL(relu_pool2_kernel, dim3(blocks), dim3(256), 0, s, d_input, d_output, planes, img_h, img_w, vec);
  }
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}
