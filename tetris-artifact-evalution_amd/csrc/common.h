// Internal declarations shared by the translation units of libtetris_spconv2d.so.
#ifndef TETRIS_CSRC_COMMON_H_
#define TETRIS_CSRC_COMMON_H_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "tetris_spconv2d.h"

namespace tetris {

// ---- error reporting -------------------------------------------------------------------------
int fail(int code, const char* fmt, ...);  // records the message for tetris_last_error(), returns code

#define TETRIS_HIP(call)                                                                           \
  do {                                                                                             \
    hipError_t e_ = (call);                                                                        \
    if (e_ != hipSuccess)                                                                          \
      return ::tetris::fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__,      \
                            hipGetErrorString(e_));                                                \
  } while (0)

constexpr int kBatch = 8;        // entries per 64-byte scalar fetch; segments are padded to this
constexpr int kWave = 64;
constexpr int kRefLanes = 32;    // the reference layout's lane count (Tetris/spconv2d_utils.h:15)
constexpr int kMaxKs = 7;        // 3-bit row/column fields of the position word

inline int out_extent(int in, int pad, int ks, int stride) { return (in + 2 * pad - ks) / stride + 1; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// ---- kernel geometry --------------------------------------------------------------------------
// One workgroup computes, for `nb` images, a `thi` x (4*lw) patch of output pixels and
// waves*G output-channel slots.  A lane owns `NQ` quads; quad q of lane (ly, lx) is the four pixels
// (virtual row ly + q*lh, columns lx + j*lw, j = 0..3).  Virtual row v is row v % thi of image v / thi.
//
// LDS holds, per image and staged input channel, `ih` input rows of `pitch` dwords.  A row stores the
// columns regrouped so that the four inputs a quad needs for kernel column s sit in one aligned
// 16-byte slot: with u = stride*lx + s, slot (u % stride, u / stride) holds input columns
// u + stride*lw*j, j = 0..3.  Slots of one parity (u % stride) are contiguous (`par` dwords apart per
// parity), so neighbouring lanes read neighbouring slots for every s and every stride.
struct Geom {
  int N, C, H, W, K, OH, OW, ks, stride, pad;
  int tile_ic, stages;
  int lw, lh, thi, nb;
  int ng;          // 16-byte slots per parity per row
  int pitch;       // dwords per LDS row (>= stride*ng*4)
  int par;         // dwords between parity planes inside a row (= ng*4)
  int ih;          // staged input rows per image
  int plane;       // dwords per (image, channel) = ih*pitch
  int img_stride;  // dwords per image = tile_ic*plane
  int fill_slots;  // nb*ih*stride*ng: 16-byte slots to fill per staged channel
  int tiles_w, tiles_h, tiles_n;
  int kblocks;     // workgroups along the output-channel slots
  int kb;          // slots per workgroup = waves*G
  int slots;       // padded slot count of the pack
  int lds_bytes;   // tile + fill table
};

// Byte offset (inside one image's LDS tile) that the packed entry (ic_local, r, s) adds to a lane's base.
inline int lds_entry_offset(const Geom& g, int ic_local, int r, int s) {
  return 4 * (ic_local * g.plane + r * g.pitch + (s % g.stride) * g.par + (s / g.stride) * 4);
}

// ---- gfx950 pack ------------------------------------------------------------------------------
struct BoundKey {
  int plane, pitch, par, stride;
  bool operator<(const BoundKey& o) const {
    if (plane != o.plane) return plane < o.plane;
    if (pitch != o.pitch) return pitch < o.pitch;
    if (par != o.par) return par < o.par;
    return stride < o.stride;
  }
};

}  // namespace tetris

struct tetris_g950 {
  int C = 0, K = 0, ks = 0, tile_ic = 0, stages = 0;
  int slots = 0;            // K rounded up to a multiple of 128
  int64_t n_entries = 0, nnz = 0;
  int32_t* d_seg_off = nullptr;   // [slots*stages+1]
  int32_t* d_seg_nnz = nullptr;   // [slots*stages]
  int32_t* d_position = nullptr;  // [n_entries]
  float* d_values = nullptr;      // [n_entries]
  int32_t* d_oc_order = nullptr;  // [slots], -1 for padding slots
  // (LDS byte offset, value) pairs for one tile geometry, made on first use
  std::map<tetris::BoundKey, int2*> bound;
  std::mutex mu;
  // host mirrors, filled by tetris_g950_host_arrays
  std::vector<int32_t> h_seg_off, h_seg_nnz, h_position, h_oc_order;
  std::vector<float> h_values;
};

struct tetris_spf {
  int C = 0, K = 0, ks = 0, tile_ic = 0;
  int64_t nnz = 0;
  std::vector<int32_t> offsets, stage_len, position, oc_permutation;
  std::vector<float> values;
  int32_t *d_offsets = nullptr, *d_stage_len = nullptr, *d_position = nullptr, *d_oc_permutation = nullptr;
  float* d_values = nullptr;
  std::vector<float> filter;                   // dense copy the kernel's packs are made from
  std::map<int, tetris_g950*> kernel_packs;    // by staged input channels, made at launch
  std::mutex mu;
};

namespace tetris {

// spf_pack_host.cpp
int spf_pack_host(const float* filter, int C, int K, int ks, int tile_ic, bool apply_reorder, bool apply_vectorize,
                  unsigned flags, tetris_spf* out);

// spf_pack_device.hip
int g950_bind(tetris_g950* p, const Geom& g, hipStream_t stream, const int2** entries_out);

// tile_select.cpp
int make_geom(const tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile& t, Geom* g);
int choose_tile(int N, int H, int W, int C, int K, int ks, int stride, int pad, tetris_tile* t);

// spconv2d_kernel.hip
int launch_conv(const Geom& g, const tetris_tile& t, const float* d_in, float* d_out, const int2* entries,
                const int32_t* seg_off, const int32_t* oc_order, hipStream_t stream);
size_t conv_lds_bytes(const Geom& g);

}  // namespace tetris

#endif  // TETRIS_CSRC_COMMON_H_
