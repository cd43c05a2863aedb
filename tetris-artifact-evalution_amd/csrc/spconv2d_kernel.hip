// Filter-sparse direct conv2d for gfx950 (wave64): lanes own output pixels, weights are wave-uniform.
//
// Replaces the reference's SparseConv2dKernel + LoadImg2SharedMem + SparseConv2d launcher
// (Tetris/spconv2d_kernel.cu:13-188), which maps lanes to output channels and pays one LDS read per FMA
// at a lane-dependent address.  Here a workgroup stages a halo'd NCHW input tile for `tile_ic` channels
// in LDS, every wave walks the packed (LDS offset, value) entries of its own output channels through
// the scalar unit, and each entry costs NQ aligned 16-byte LDS reads and 4*NQ FMAs with the weight as
// an SGPR operand.  Accumulators stay in VGPRs across the input-channel stages; outputs are written
// once, NCHW, contiguous along the row.
#include "common.h"

namespace tetris {
namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

template <int NQ, int G, int WMAX>
__global__ __launch_bounds__(WMAX * 64) void spconv2d_kernel(const float* __restrict__ in, float* __restrict__ out,
                                                             const int2* __restrict__ entries,
                                                             const int32_t* __restrict__ seg_off,
                                                             const int32_t* __restrict__ oc_order, const Geom g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = uniform(tid >> 6);
  const int nwaves = blockDim.x >> 6;

  // Workgroup -> (spatial tile, channel block).  Consecutive workgroup ids go round-robin to the eight
  // XCDs; give each XCD a contiguous range of logical ids so that the channel blocks of one spatial
  // tile (which re-read the same input) share an L2.
  const int total = g.tiles_n * g.tiles_h * g.tiles_w * g.kblocks;
  const int per_xcd = gridDim.x >> 3;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const int kblock = logical % g.kblocks;
  int t = logical / g.kblocks;
  const int tw = t % g.tiles_w;
  t /= g.tiles_w;
  const int th = t % g.tiles_h;
  const int tn = t / g.tiles_h;
  const int n0 = tn * g.nb, oh0 = th * g.thi, ow0 = tw * 4 * g.lw;

  const int tile_dwords = g.nb * g.img_stride;
  i4* fill_src = reinterpret_cast<i4*>(smem + 4 * (size_t)tile_dwords);   // global offsets per slot, -1 = zero
  int* fill_dst = reinterpret_cast<int*>(fill_src + g.fill_slots);        // LDS dword index per slot

  // ---- once per workgroup: where each 16-byte LDS slot of a staged channel comes from --------------
  {
    const int per_row = g.stride * g.ng;
    const int per_img = g.ih * per_row;
    const int chw = g.C * g.H * g.W;
    for (int s = tid; s < g.fill_slots; s += blockDim.x) {
      const int img = s / per_img;
      const int r1 = s - img * per_img;
      const int row = r1 / per_row;
      const int r2 = r1 - row * per_row;
      const int q = r2 / g.ng;
      const int m = r2 - q * g.ng;
      const int ihh = oh0 * g.stride - g.pad + row;
      const int col0 = ow0 * g.stride - g.pad + q + g.stride * m;
      const bool row_ok = (n0 + img) < g.N && ihh >= 0 && ihh < g.H;
      const int base = img * chw + ihh * g.W;
      i4 o;
      int c;
      c = col0;                       o.x = (row_ok && c >= 0 && c < g.W) ? base + c : -1;
      c = col0 + g.stride * g.lw;     o.y = (row_ok && c >= 0 && c < g.W) ? base + c : -1;
      c = col0 + 2 * g.stride * g.lw; o.z = (row_ok && c >= 0 && c < g.W) ? base + c : -1;
      c = col0 + 3 * g.stride * g.lw; o.w = (row_ok && c >= 0 && c < g.W) ? base + c : -1;
      fill_src[s] = o;
      fill_dst[s] = img * g.img_stride + row * g.pitch + q * g.par + m * 4;
    }
  }

  // ---- lane -> pixels ------------------------------------------------------------------------------
  const int lx = lane % g.lw;
  const int ly = lane / g.lw;
  const bool lane_ok = ly < g.lh;
  int base[NQ];  // LDS byte address of the lane's quad for entry offset 0
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int vr = ly + q * g.lh;
    const int img = vr / g.thi;
    const int row = vr - img * g.thi;
    const bool ok = lane_ok && img < g.nb;
    base[q] = ok ? 4 * (img * g.img_stride + row * g.stride * g.pitch + lx * 4) : 0;
  }

  f4 acc[G][NQ];
#pragma unroll
  for (int k = 0; k < G; ++k)
#pragma unroll
    for (int q = 0; q < NQ; ++q) acc[k][q] = (f4)(0.f);

  const int slot0 = kblock * g.kb + wave * G;
  const size_t hw = (size_t)g.H * g.W;

  for (int st = 0; st < g.stages; ++st) {
    __syncthreads();  // previous stage fully consumed (and the fill table written, first time round)
    // ---- stage the input tile: one wave per channel, one lane per 16-byte slot ----------------------
    const int c0 = st * g.tile_ic;
    const int cs = min(g.tile_ic, g.C - c0);
    for (int c = wave; c < cs; c += nwaves) {
      const float* src = in + ((size_t)n0 * g.C + c0 + c) * hw;
      f4* dstc = reinterpret_cast<f4*>(smem) ;
      for (int s = lane; s < g.fill_slots; s += 64) {
        const i4 o = fill_src[s];
        const int d = fill_dst[s] + c * g.plane;
        f4 v;
        v.x = o.x >= 0 ? src[o.x] : 0.f;
        v.y = o.y >= 0 ? src[o.y] : 0.f;
        v.z = o.z >= 0 ? src[o.z] : 0.f;
        v.w = o.w >= 0 ? src[o.w] : 0.f;
        dstc[d >> 2] = v;
      }
    }
    __syncthreads();

    // ---- walk this wave's entries --------------------------------------------------------------------
#pragma unroll
    for (int k = 0; k < G; ++k) {
      const int seg = (slot0 + k) * g.stages + st;
      const int beg = seg_off[seg];
      const int end = seg_off[seg + 1];
      for (int i = beg; i < end; i += 4) {
        const int2 e0 = entries[i], e1 = entries[i + 1], e2 = entries[i + 2], e3 = entries[i + 3];
        f4 x0[NQ], x1[NQ], x2[NQ], x3[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          x0[q] = *reinterpret_cast<const f4*>(smem + base[q] + e0.x);
          x1[q] = *reinterpret_cast<const f4*>(smem + base[q] + e1.x);
          x2[q] = *reinterpret_cast<const f4*>(smem + base[q] + e2.x);
          x3[q] = *reinterpret_cast<const f4*>(smem + base[q] + e3.x);
        }
        const float w0 = __int_as_float(e0.y), w1 = __int_as_float(e1.y);
        const float w2 = __int_as_float(e2.y), w3 = __int_as_float(e3.y);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          acc[k][q] += w0 * x0[q];
          acc[k][q] += w1 * x1[q];
          acc[k][q] += w2 * x2[q];
          acc[k][q] += w3 * x3[q];
        }
      }
    }
  }

  // ---- write the outputs ---------------------------------------------------------------------------
#pragma unroll
  for (int k = 0; k < G; ++k) {
    const int oc = oc_order[slot0 + k];
    if (oc < 0) continue;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      const int vr = ly + q * g.lh;
      const int img = vr / g.thi;
      const int row = vr - img * g.thi;
      const int n = n0 + img, oh = oh0 + row;
      if (!(lane_ok && img < g.nb && n < g.N && oh < g.OH)) continue;
      float* o = out + (((size_t)n * g.K + oc) * g.OH + oh) * g.OW;
      const int ow = ow0 + lx;
      if (ow < g.OW) o[ow] = acc[k][q].x;
      if (ow + g.lw < g.OW) o[ow + g.lw] = acc[k][q].y;
      if (ow + 2 * g.lw < g.OW) o[ow + 2 * g.lw] = acc[k][q].z;
      if (ow + 3 * g.lw < g.OW) o[ow + 3 * g.lw] = acc[k][q].w;
    }
  }
}

template <int NQ, int G, int WMAX>
int launch_one(const Geom& g, int waves, const float* d_in, float* d_out, const int2* entries, const int32_t* seg_off,
               const int32_t* oc_order, hipStream_t stream) {
  auto kern = spconv2d_kernel<NQ, G, WMAX>;
  static int lds_limit_set = 0;  // per instantiation
  if (g.lds_bytes > lds_limit_set) {
    TETRIS_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024));
    lds_limit_set = 160 * 1024;
  }
  const int total = g.tiles_n * g.tiles_h * g.tiles_w * g.kblocks;
  const int grid = (total + 7) / 8 * 8;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(waves * 64), g.lds_bytes, stream, d_in, d_out, entries, seg_off, oc_order,
                     g);
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}

}  // namespace

size_t conv_lds_bytes(const Geom& g) {
  return 4 * (size_t)g.nb * g.img_stride + (size_t)g.fill_slots * (sizeof(i4) + sizeof(int));
}

int launch_conv(const Geom& g, const tetris_tile& t, const float* d_in, float* d_out, const int2* entries,
                const int32_t* seg_off, const int32_t* oc_order, hipStream_t stream) {
#define TETRIS_CASE(NQ, G)                                                                                      \
  if (t.quads == NQ && t.oc_per_wave == G) {                                                                    \
    if (t.waves <= 4) return launch_one<NQ, G, 4>(g, t.waves, d_in, d_out, entries, seg_off, oc_order, stream);  \
    if (t.waves <= 8) return launch_one<NQ, G, 8>(g, t.waves, d_in, d_out, entries, seg_off, oc_order, stream);  \
  }
  TETRIS_CASE(1, 8)
  TETRIS_CASE(1, 16)
  TETRIS_CASE(2, 4)
  TETRIS_CASE(2, 8)
  TETRIS_CASE(2, 16)
  TETRIS_CASE(4, 4)
  TETRIS_CASE(4, 8)
#undef TETRIS_CASE
  return fail(TETRIS_EINVAL, "no kernel for quads=%d oc_per_wave=%d waves=%d", t.quads, t.oc_per_wave, t.waves);
}

}  // namespace tetris
