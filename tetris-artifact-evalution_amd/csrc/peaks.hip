// What this GPU delivers to the two plainest kernels there are, for reading a roofline fraction against a measured
// ceiling as well as the nominal one: a device-to-device copy (HBM bytes per second, read + write) and a loop of
// independent fp32 FMAs (vector FLOP/s; this library is compiled without packed fp32, so the loop issues v_fma_f32).
// No reference counterpart: the reference reports milliseconds and "T" per layer only (Tetris/spconv2d.cc:357-358).
#include "common.h"

namespace tetris {
namespace {

__global__ __launch_bounds__(256) void copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, long long n4) {
  const long long step = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += step) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void fma_kernel(float* out, int iters, float x, float y) {
  float a[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) a[k] = (float)(threadIdx.x + k);
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int k = 0; k < 16; ++k) a[k] = __builtin_fmaf(a[k], x, y);  // sixteen independent chains
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < 16; ++k) s += a[k];
  if (s == 12345.678f) out[0] = s;  // keeps the loop alive, practically never true
}

__global__ __launch_bounds__(256) void sweep_kernel(float4* __restrict__ buf, long long n4) {
  const long long step = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += step) {
    float4 v = buf[i];
    v.x += 1.f;
    buf[i] = v;
  }
}

}  // namespace

// Reads and rewrites a 512 MiB buffer (made on first use, kept until the process ends): more than the caches in front
// of HBM hold, so that whatever runs next on `stream` finds its tensors, its weights and its code in memory, as a
// layer in the middle of a network does.
int sweep_caches(hipStream_t stream) {
  static float4* buf = nullptr;
  static std::mutex mu;
  const long long n4 = 32ll << 20;
  std::lock_guard<std::mutex> lock(mu);
  if (!buf) {
    TETRIS_HIP(hipMalloc(&buf, n4 * sizeof(float4)));
    TETRIS_HIP(hipMemsetAsync(buf, 0, n4 * sizeof(float4), stream));
  }
  hipLaunchKernelGGL(sweep_kernel, dim3(8192), dim3(256), 0, stream, buf, n4);
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}

}  // namespace tetris

using namespace tetris;

extern "C" int tetris_measure_peaks(void* stream_, float* copy_gbs_out, float* fma_tflops_out) {
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const long long n4 = 16ll << 20;  // 256 MiB each way
  float4 *src = nullptr, *dst = nullptr;
  float* sink = nullptr;
  hipEvent_t a = nullptr, b = nullptr;
  auto done = [&](int code) {
    if (src) (void)hipFree(src);
    if (dst) (void)hipFree(dst);
    if (sink) (void)hipFree(sink);
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
    return code;
  };
#define HIPP(call)                                                                                          \
  do {                                                                                                      \
    hipError_t e_ = (call);                                                                                 \
    if (e_ != hipSuccess)                                                                                   \
      return done(fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__, hipGetErrorString(e_))); \
  } while (0)
  HIPP(hipMalloc(&src, n4 * sizeof(float4)));
  HIPP(hipMalloc(&dst, n4 * sizeof(float4)));
  HIPP(hipMalloc(&sink, sizeof(float)));
  HIPP(hipEventCreate(&a));
  HIPP(hipEventCreate(&b));
  hipLaunchKernelGGL(copy_kernel, dim3(4096), dim3(256), 0, stream, dst, src, n4);  // first touch of both buffers
  const int reps = 10;
  for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(copy_kernel, dim3(4096), dim3(256), 0, stream, src, dst, n4);
  HIPP(hipEventRecord(a, stream));
  for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(copy_kernel, dim3(4096), dim3(256), 0, stream, src, dst, n4);
  HIPP(hipEventRecord(b, stream));
  HIPP(hipEventSynchronize(b));
  float ms = 0;
  HIPP(hipEventElapsedTime(&ms, a, b));
  if (copy_gbs_out) *copy_gbs_out = (float)(2.0 * reps * n4 * sizeof(float4) / (ms * 1e-3) / 1e9);

  // The shader clock idles near 2.1 GHz and takes 10-25 ms of unbroken work to reach what it holds under load
  // (about 2.37 GHz): eight launches of 3.7 ms go first, three are timed.
  const int blocks = 256 * 16, iters = 8192, warm = 8, timed = 3;
  for (int i = 0; i < warm; ++i)
    hipLaunchKernelGGL(fma_kernel, dim3(blocks), dim3(256), 0, stream, sink, iters, 1.0001f, 0.5f);
  HIPP(hipEventRecord(a, stream));
  for (int i = 0; i < timed; ++i)
    hipLaunchKernelGGL(fma_kernel, dim3(blocks), dim3(256), 0, stream, sink, iters, 1.0001f, 0.5f);
  HIPP(hipEventRecord(b, stream));
  HIPP(hipEventSynchronize(b));
  HIPP(hipEventElapsedTime(&ms, a, b));
  HIPP(hipGetLastError());
  if (fma_tflops_out)
    *fma_tflops_out = (float)(2.0 * 16 * iters * (double)blocks * 256 * timed / (ms * 1e-3) / 1e12);
#undef HIPP
  return done(TETRIS_OK);
}
