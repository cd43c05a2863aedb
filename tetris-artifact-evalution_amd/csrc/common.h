// Internal declarations shared by the translation units of libtetris_spconv2d.so.
#ifndef TETRIS_CSRC_COMMON_H_
#define TETRIS_CSRC_COMMON_H_

#include <hip/hip_runtime.h>

#include <array>
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

constexpr int kBatch = 8;        // entries per 64-byte scalar fetch; every stream is padded to this
constexpr int kRefLanes = 32;    // the reference layout's lane count (Tetris/spconv2d_utils.h:15)
constexpr int kMaxKs = 7;        // 3-bit row/column fields of the position word
constexpr int kSlotPad = 128;    // output-channel slots are padded to a multiple of this
constexpr int kTileBytes = 65536;  // LDS bytes of one workgroup's input tile (all regions), single-buffered kernel
constexpr int kBufBytes = 54272;   // one LDS buffer of the triple-buffered kernel (8-wave workgroups, 3 * 53 KiB)
constexpr int kHalfBufBytes = 27136;  // ... when two 8-wave workgroups of 64-accumulator waves share a CU
constexpr int kBufs = 3;
constexpr int kFlatBufBytes = 65536;      // one of the two LDS buffers of a flat (pointwise) kernel, one workgroup per CU
constexpr int kFlatHalfBufBytes = 32768;  // ... of its 8-wave form with 64 accumulators, two workgroups per CU
constexpr int kMaxChunks = 8;      // (6 in a 16-wave workgroup, whose waves have fewer registers)
constexpr int kMaxChunks16 = 6;
//      // 64-dword LDS chunks of one staged channel a wave may own (triple-buffered kernel)
constexpr int kAccRegs = 128;    // accumulator VGPRs of a wave: oc_per_wave * 4 * quads
constexpr int kFillItems = 8;    // staged 16-byte slots a thread may hold in flight per stage
constexpr int kFlatLanes = 64;   // tetris_tile.lanes_w of the flat (pointwise) tiles
constexpr int kMaxSplit = 8;      // most workgroups that may share an output tile (each reduces a slice of the stages)
// A split layer's scratch starts with its tickets -- one int per (output tile, wave), zero between launches -- and
// the partial sums follow.
constexpr int kTicketBytes = 65536;
constexpr int kMaxTickets = kTicketBytes / 4;

inline int out_extent(int in, int pad, int ks, int stride) { return (in + 2 * pad - ks) / stride + 1; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline unsigned magic_reciprocal(int d) { return d <= 1 ? 0u : (unsigned)((1ull << 32) / (unsigned)d) + 1u; }

// ---- kernel geometry --------------------------------------------------------------------------
// Output pixels are cut into *units* of up to 64 quads: a unit is `lh` virtual rows by 4*lw columns, lane
// (ly, lx) = (lane / lr, lane % lr) owning the four pixels (virtual row ly, columns lx + j*lw, j = 0..3);
// lanes with lx >= lw or ly >= lh idle.  A virtual row v is row v % thi of image v / thi, so that small
// feature maps fold several images into one unit.  A workgroup computes NQ consecutive units (one per
// lane "quad") for waves * G output-channel slots.
//
// Why lr (lanes per row) can exceed lw: a 16-byte-per-lane LDS read runs at the full 256 B/clk only when
// every lane row starts, bank-wise, where the previous one ended, i.e. when the LDS distance between
// consecutive lane rows is 4*lr dwords modulo 64 (measured on MI355X; any other distance halves the
// rate).  A halo'd row holds lw + (ks-1)/stride slots, so the lanes of a row are spread over that many
// lane positions and the pitch is chosen to meet the rule.
//
// LDS holds one region of kTileBytes / NQ bytes per unit: [image][staged channel][input row][pitch]
// floats.  A row stores its columns regrouped so that the four inputs a quad needs for kernel column s
// sit in one aligned 16-byte slot: with u = stride*lx + s, slot (u % stride, u / stride) holds input
// columns u + stride*lw*j, j = 0..3.  Slots of one parity (u % stride) are contiguous, `par` dwords
// per parity, so neighbouring lanes read neighbouring slots for every s and every stride.
struct Geom {
  int N, C, H, W, K, OH, OW, ks, stride, pad;
  int tile_ic, stages;
  int nq, g, waves;    // quads per lane, slots per wave, waves per workgroup
  int lw, lr, lh, thi, nb; // active lanes per row, lane positions per row, lane rows, rows per image, images per unit
  int ng;              // 16-byte slots per parity per row
  int pitch;           // dwords per LDS row (>= stride*ng*4)
  int par;             // dwords between parity planes inside a row (= ng*4)
  int ih;              // staged input rows per image
  int plane;           // dwords per (image, channel) = ih*pitch
  int img_stride;      // dwords per image = tile_ic*plane
  int region;          // bytes per region = kTileBytes / nq
  int units_w, units_h, units_n, units;  // unit grid: columns, row blocks, image blocks, total
  int ugroups;         // workgroups along the units = ceil(units / nq)
  int kblocks;         // workgroups along the output-channel slots
  int kb;              // slots per workgroup = waves*g
  int slots;           // padded slot count of the pack
  // input staging: a thread owns `spt` of the unit group's 16-byte slots and walks the staged channels
  // `cg` at a time
  int slots_per_unit;  // nb*ih*stride*ng
  int fill_slots;      // nq*slots_per_unit
  int spt, cg, fill_iters;
  // triple-buffered kernel (ver == 3): a staged channel of the whole unit group is cut into 64-dword chunks,
  // `cpp` per (unit, image) plane, and wave w fills chunks w, w + waves, ... with loads that write LDS directly
  int ver;             // 2: single LDS tile, register staging; 3: three LDS buffers, direct-to-LDS staging
  int cpp, nchunks, ni;
  int buf_bytes;       // size of one of the three LDS buffers: kBufBytes, or kHalfBufBytes (8 waves of <= 64 accumulators)
  int csplit;          // workgroups that share an output tile, each reducing a slice of the stages into its own copy
                       // of the output (a scratch buffer); reduce_kernel adds the copies.  1 = no split
  // A 1x1 convolution of stride s without padding only reads every s-th row and column: it is run as a stride-1
  // layer on that sub-grid (H, W, stride above then describe the sub-grid) and the staging loads step through the
  // real image: element (row, col) of the sub-grid lies at row*step*in_w + col*step of a plane of in_hw floats.
  int step, in_w, in_hw;
  // Images side by side: a tile whose lanes span the image width twice or four times over (2*lw >= OW, lw >= OW)
  // gives quads j = 0..3 of a lane to `fold` = 2 or 4 different images instead of to four column groups of one:
  // quad j belongs to image j >> jsh of the unit and to column group j & ((1 << jsh) - 1).  fold = 1, jsh = 2 otherwise.
  int fold, jsh;
  int stagers;         // waves 0 .. stagers-1 fill LDS (4 or 8 of an 8-wave workgroup; 4, 8 or 16 of a 16-wave one)
  // Pointwise layers (1x1, stride 1, no padding; ver == 4): no halo, so the pixels of an image are one flat run of H*W
  // floats per channel and a lane owns four CONSECUTIVE pixels (a quad).  Image n holds `qi` = ceil(H*W / 4) quads,
  // the batch N*qi quads, a unit 64 consecutive quads of that sequence (lane l of unit u: quad u*64 + l), and LDS one
  // 1 KiB row per staged channel and unit (lane l at byte 16*l): staging is one 16-byte-per-lane load that writes LDS
  // directly per (channel, unit), reads are aligned 16-byte accesses at consecutive addresses, stores are 16 bytes
  // per lane when H*W is a multiple of four.
  // A strided pointwise layer keeps the flat tile on the sub-grid it reads (H, W above; element (row, col) lies at
  // row*step*in_w + col*step of a plane of in_hw floats): a lane's quad is then staged as four separate dwords.
  int qi, quads_total;
  unsigned m_qi, m_ow;
  // The bound entry array ends with a copy of the first batch (eight entries) of every stream, [group][stage][8],
  // starting at entry `heads_off` (set when the plan is made): a workgroup reads its first batch from there, at an
  // address it knows without having read the stream's offset first.
  int heads_off;
  // What a kernel does to a finished sum before it writes it (set per launch): 0 nothing, 1 ReLU, 2 ReLU and 2x2
  // max-pooling inside the halo'd kernels (the output tensor is then N x K x OH/2 x OW/2).
  int act;
  // Split layers (csplit > 1), set per launch: 1 = every wave, once its partial sums are stored, takes a ticket of its
  // (output tile, wave) pair, and the wave that draws the last one adds the slices itself, in slice order, and writes
  // the finished sums (through `act` 0 or 1); 0 = a second kernel adds the slices.
  int fused;
  // multiply-high reciprocals, floor(2^32 / d) + 1: x / d == umulhi(x, m) whenever x * d < 2^32
  unsigned m_per_unit, m_cpp, m_pitch, m_par, m_upi, m_units_w, m_lr, m_thi, m_kblocks, m_csplit;
  unsigned m_fill_slots, m_slots_per_unit, m_per_img, m_per_row, m_ng;  // single-tile kernel's staging plan
};

// how many images a tile of `lw` lanes per row places side by side on an output OW pixels wide
inline int fold_of(int lw, int OW) { return lw >= OW ? 4 : 2 * lw >= OW ? 2 : 1; }

// Byte offset that the packed entry (ic_local, r, s) adds to a lane's LDS base address.
inline int lds_entry_offset(int plane, int pitch, int par, int stride, int ic_local, int r, int s) {
  return 4 * (ic_local * plane + r * pitch + (s % stride) * par + (s / stride) * 4);
}

struct BoundKey {
  int plane, pitch, par, stride, nq;
  int paired;  // 1: streams rearranged into a segment of pairs and a segment of singles (see g950_bind)
  bool operator<(const BoundKey& o) const {
    if (paired != o.paired) return paired < o.paired;
    if (plane != o.plane) return plane < o.plane;
    if (pitch != o.pitch) return pitch < o.pitch;
    if (par != o.par) return par < o.par;
    if (stride != o.stride) return stride < o.stride;
    return nq < o.nq;
  }
};

}  // namespace tetris

namespace tetris {
// A launch plan: everything run_launch derives from (input shape, tile) for one pack, kept for the next call.
struct Plan {
  int key[11];  // N, H, W, stride, pad, lanes_w, quads, oc_per_wave, waves, tile_ic, csplit
  Geom geom;
  const int2* entries;        // the pack's entries bound to the geometry
  const int32_t* grp_off;     // [groups*stages+1] first entry of every stream in `entries`
  const int32_t* grp_pair;    // [groups*stages] entries of the stream's leading segment of pairs (0 when unpaired)
};
}  // namespace tetris

// gfx950 pack: per (wave group of G slots, input-channel stage) one stream of entries.
struct tetris_g950 {
  int C = 0, K = 0, ks = 0, tile_ic = 0, stages = 0;
  int g = 0;                // slots per wave group
  int slots = 0;            // K rounded up to a multiple of kSlotPad
  int groups = 0;           // slots / g
  int64_t n_entries = 0, nnz = 0;
  int32_t* d_grp_off = nullptr;   // [groups*stages+1] entry index, multiples of 8
  int32_t* d_grp_nnz = nullptr;   // [groups*stages]
  int32_t* d_position = nullptr;  // [n_entries] s | r<<3 | ic_local<<6 | slot-in-group<<24
  float* d_values = nullptr;      // [n_entries]
  int32_t* d_oc_order = nullptr;  // [slots], -1 for padding slots
  // (LDS byte offset | accumulator index << 16 | 0xC << 28, value) pairs for one tile geometry, made on first use
  std::map<tetris::BoundKey, int2*> bound;
  // Paired arrangement of the streams (made on the first paired bind; depends on the pack only): two consecutive
  // entries of a stream that share their position become a pair; per stream first all pairs, padded to a multiple
  // of 8 entries, then the entries left single, padded likewise.
  int32_t* d_pgrp_off = nullptr;   // [groups*stages+1]
  int32_t* d_pgrp_pair = nullptr;  // [groups*stages]
  int32_t* d_zero_pair = nullptr;  // [groups*stages] zeros: the pair counts of the unpaired arrangement
  int64_t n_paired_entries = 0;
  std::vector<tetris::Plan> plans;  // few per pack; searched linearly, most recent first
  // partial sums of layers whose channel reduction is split over workgroups: [csplit][N][K][OH][OW], one buffer per
  // stream the pack is launched on, made by tetris_g950_prepare or by the first such launch; a buffer that had to
  // grow is kept (`retired`) until the pack is destroyed, because a captured graph may still hold its address
  struct Partial {
    float* ptr = nullptr;
    size_t bytes = 0;
  };
  std::map<hipStream_t, Partial> partial;
  std::vector<float*> retired;
  std::mutex mu;
  // host mirrors, filled by tetris_g950_host_arrays
  std::vector<int32_t> h_grp_off, h_grp_nnz, h_position, h_oc_order;
  std::vector<float> h_values;
};

struct tetris_spf {
  int C = 0, K = 0, ks = 0, tile_ic = 0;
  int64_t nnz = 0;
  std::vector<int32_t> offsets, stage_len, position, oc_permutation;
  std::vector<float> values;
  int32_t *d_offsets = nullptr, *d_stage_len = nullptr, *d_position = nullptr, *d_oc_permutation = nullptr;
  float* d_values = nullptr;
  int vec = 0;  // entries per lane and step in `position` / `values`: 4, 1, or 0 for the keep-as-is layout
  std::mutex mu;
};

namespace tetris {

// spf_pack_host.cpp
int spf_pack_host(const float* filter, int C, int K, int ks, int tile_ic, bool apply_reorder, bool apply_vectorize,
                  unsigned flags, tetris_spf* out);

int check_spf_offsets(const int32_t* offsets, int n_off, int lanes, int vec, long long capacity);

// spf_pack_device.hip
// entries of the pack bound to geometry `g`; paired: rearranged into pairs and singles (kernels that walk pairs)
int g950_bind(tetris_g950* p, const Geom& g, bool paired, hipStream_t stream, const int2** entries_out,
              const int32_t** grp_off_out, const int32_t** grp_pair_out, int* heads_off_out);

// spf_pack_device.hip: the reference layout's device arrays as the source of a convolution
// n_ent: entries of d_position / d_values to hash (the caller has read and checked the offsets on the host)
int spf_arrays_hash(const int32_t* d_offsets, int n_off, const int32_t* d_perm, int K, const int32_t* d_position,
                    const float* d_values, long long n_ent, unsigned long long* d_scratch2, hipStream_t stream,
                    unsigned long long* hash_out);
int spf_arrays_decode(const int32_t* d_offsets, const int32_t* d_perm, const int32_t* d_position, const float* d_values,
                      float* d_filter, int C, int K, int ks, int tile_ic, int vec, hipStream_t stream);

// tile_select.cpp
unsigned options();  // TETRIS_OPT_* flags in force (tetris_options_set, or the environment variable TETRIS_OPTIONS)
void set_options(unsigned flags);
int make_geom(const tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile& t, Geom* g);
int choose_tile(int N, int H, int W, int C, int K, int ks, int stride, int pad, tetris_tile* t);
// reads rows in the format of tuned_tiles.inc; choose_tile looks them up before the built-in table
int load_tile_table(const char* path, int* rows_out);
// every tile shape the kernel can run for the layer, cheapest first by the selector's time model
// (density: fraction of non-zero weights when the caller knows the filter, else 0)
int rank_tiles(int N, int H, int W, int C, int K, int ks, int stride, int pad, std::vector<tetris_tile>* ranked,
               double density = 0.0);

// peaks.hip: evicts the caches in front of HBM (a pass over a 512 MiB buffer on `stream`)
int sweep_caches(hipStream_t stream);

// output-channel order (a permutation of 0..K-1) that balances the waves of a workgroup for tile `t`
int balance_oc_order(const float* filter, int C, int K, int ks, const tetris_tile& t, int32_t* order);

// spconv2d_kernel.hip
// launches the conv; when the geometry splits the channel reduction (csplit > 1) the workgroups write their partial
// sums to the scratch ([csplit] outputs) and the slices are added, in slice order, into d_out: by the last wave of
// every (tile, wave) pair to finish (TETRIS_OPT_ADD_IN_KERNEL, on a device whose workgroup placement keeps a tile's
// slices on one XCD, no pooling), or else by a second kernel
// act: 0 = d_out gets the sums; 1 = their ReLU; 2 = ReLU and 2x2 max-pooling (d_out is N x K x OH/2 x OW/2), done by
// the adding kernel of a split layer and otherwise inside the conv kernel where geom_pools_in_kernel allows (else
// TETRIS_EUNSUPPORTED, nothing launched)
// d_scratch (split layers): kTicketBytes of tickets, all zero between launches, then room for csplit outputs
int launch_conv(const Geom& g, const float* d_in, float* d_out, float* d_scratch, const int2* entries,
                const int32_t* grp_off, const int32_t* grp_pair, const int32_t* oc_order, int act, hipStream_t stream);
// whether workgroups with the same blockIdx.x % 8 run on one XCD of the current device (probed once per device):
// what lets the slices of a split layer exchange their partial sums through that XCD's L2
int same_xcd_by_residue(bool* ok);
bool geom_pools_in_kernel(const Geom& g);
// whether the kernel of geometry `g` walks paired streams
bool geom_walks_pairs(const Geom& g);

}  // namespace tetris

#endif  // TETRIS_CSRC_COMMON_H_
