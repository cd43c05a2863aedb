// Filter-sparse direct conv2d for gfx950 (wave64): lanes own output pixels, weights are wave-uniform.
//
// Replaces the reference's SparseConv2dKernel + LoadImg2SharedMem + SparseConv2d launcher
// (Tetris/spconv2d_kernel.cu:13-188), which maps lanes to output channels and pays one LDS read at a
// lane-dependent address per FMA.  Here:
//   * a workgroup stages the halo'd NCHW input of NQ pixel units for `tile_ic` channels in LDS (buffer
//     loads with hardware bounds checking supply the zero padding);
//   * each wave walks ONE stream of packed (LDS offset | accumulator index, weight) entries per stage
//     through the scalar unit (64-byte fetches, eight entries each, one fetch ahead);
//   * an entry costs one VALU add, NQ aligned 16-byte LDS reads (issued a few entries ahead) and 4*NQ FMAs
//     whose weight is an SGPR operand and whose accumulator is selected by the VGPR index register, so
//     the G output channels of a wave need no code replication and no per-channel padding;
//   * the accumulators stay in fixed VGPRs for the whole kernel; the compiler is confined below the
//     registers of the inner loop, which is generated assembly (gen_walk_asm.py).
//
// Four kernels share the loop and the output code:
//   spconv2d_kernel<NQ,SPT>  tiles of 1-4 waves: one 64 KiB LDS tile, input staged through registers one stage
//                            ahead, 128 accumulators, two workgroups per CU;
//   spconv2d_kernel3<NQ>     8 waves, 128 accumulators: three 53 KiB LDS buffers filled by loads that write LDS
//                            directly, two stages ahead; one workgroup per CU;
//   spconv2d_kernel5<NQ>     8 waves, 64 accumulators and at most 128 VGPRs: three 26.5 KiB buffers, two workgroups
//                            per CU (four waves per SIMD);
//   spconv2d_kernel4<NQ>     16 waves, 64 accumulators: three 53 KiB buffers, four waves per SIMD.
// Layers with few pixels per image are cut along the input channels too: each workgroup of a tile reduces a slice of
// the stages into its own copy of the output and reduce_kernel adds the copies (launch_conv).
#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "common.h"

namespace tetris {
namespace {

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
// x / d through the reciprocal made by magic_reciprocal(d) (0 stands for d == 1); exact while x * d < 2^32
__device__ __forceinline__ int fast_div(int x, unsigned m) { return m ? (int)__umulhi((unsigned)x, m) : x; }

// The kernel arguments (nine pointers and the geometry: six 64-byte lines) are read piecemeal by the code below, and
// every first touch of a line is a trip to L2 that the next scalar instruction waits for.  Touching all lines at once
// when the kernel starts turns those trips into one; the later reads hit the scalar cache.
__device__ __forceinline__ void touch_kernel_arguments() {
  typedef const int __attribute__((address_space(4))) * kernarg_ptr;
  kernarg_ptr ka = (kernarg_ptr)__builtin_amdgcn_kernarg_segment_ptr();
  constexpr int kLines = (9 * 8 + (int)sizeof(Geom) + 63) / 64;
  static_assert(kLines == 6, "one load per 64-byte line of the kernel arguments");
  const int a0 = ka[0], a1 = ka[16], a2 = ka[32], a3 = ka[48], a4 = ka[64], a5 = ka[80];
  asm volatile("" ::"s"(a0), "s"(a1), "s"(a2), "s"(a3), "s"(a4), "s"(a5));
}

// Time stamps of a workgroup's life, compiled in by -DTETRIS_STAMPS only (`make stamps`; read with tetris_stamps_read,
// printed by `python -m tetris_amd.stamps`).  Wave 0 of workgroup `logical` records the shader clock where the kernels
// say TETRIS_STAMP(i): 0 kernel entry, 1 kernel arguments touched, 2 first stage's input loads issued, 3 stream offsets
// and first batch in scalar registers, 4 first stage landed and barrier passed, 5 stage loop left, 6 output stores
// issued, 7 output stores acknowledged, 11 staging plan made (just before the first loads go out); slot 8 adds up the
// clocks wave 0 spent inside the walk (12: the largest such sum over the workgroup's waves, 13: the sum over its
// waves), 9 and 10 hold the 100 MHz wall clock at entry and at the end (the clocks' ratio, and when the workgroup ran
// within the launch).
#ifdef TETRIS_STAMPS
constexpr int kStampSlots = 16, kStampWgs = 8192;
__device__ long long g_stamps[kStampWgs * kStampSlots];
#define TETRIS_STAMP_ENTRY() const long long stamp_t0_ = clock64(), stamp_w0_ = wall_clock64(); long long stamp_t1_ = 0, stamp_walk_ = 0
#define TETRIS_STAMP_ARGS() stamp_t1_ = clock64()
#define TETRIS_STAMP(i)                                                                                           \
  do {                                                                                                            \
    if (threadIdx.x == 0 && logical < kStampWgs) g_stamps[logical * kStampSlots + (i)] = clock64();                \
  } while (0)
#define TETRIS_STAMP_WALK(statement)                                                                              \
  do {                                                                                                            \
    const long long w0_ = clock64();                                                                              \
    statement;                                                                                                    \
    stamp_walk_ += clock64() - w0_;                                                                               \
  } while (0)
#define TETRIS_STAMP_END()                                                                                        \
  do {                                                                                                            \
    TETRIS_STAMP(6);                                                                                              \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                              \
    if ((threadIdx.x & 63) == 0 && logical < kStampWgs) {  /* every wave: the busiest wave's walk and the sum */    \
      unsigned long long* u_ = reinterpret_cast<unsigned long long*>(g_stamps + logical * kStampSlots);           \
      atomicMax(u_ + 12, (unsigned long long)stamp_walk_);                                                        \
      atomicAdd(u_ + 13, (unsigned long long)stamp_walk_);                                                        \
    }                                                                                                             \
    if (threadIdx.x == 0 && logical < kStampWgs) {                                                                \
      long long* s_ = g_stamps + logical * kStampSlots;                                                           \
      s_[0] = stamp_t0_; s_[1] = stamp_t1_; s_[7] = clock64(); s_[8] = stamp_walk_; s_[9] = stamp_w0_;            \
      s_[10] = wall_clock64();                                                                                    \
    }                                                                                                             \
  } while (0)
#else
#define TETRIS_STAMP_ENTRY() do {} while (0)
#define TETRIS_STAMP_ARGS() do {} while (0)
#define TETRIS_STAMP(i) do {} while (0)
#define TETRIS_STAMP_WALK(statement) statement
#define TETRIS_STAMP_END() do {} while (0)
#endif

// s36..s51 (the current batch) and s72:s73 (the stream address) are operands of the walk, bound by their constraints
#define TETRIS_S_CLOBBERS                                                                                          \
  "s52", "s53", "s54", "s55", "s56", "s57", "s58", "s59", "s60", "s61", "s62", "s63", "s64", "s65", "s66", "s67", "s68",   \
      "s69", "s70"

#include "walk_asm.inc"  // TETRIS_WALK_ASM_<NQ>, generated by gen_walk_asm.py (entry encoding and register plan there)

// The eight entries at the head of a wave's stream, kept in SGPRs from one stage to the next.
struct Batch {
  unsigned long long c[8];
};

// The first batch of stream `seg` from the copies that end the entry array: lanes 0..7 fetch an entry each (one load
// whose address does not depend on the stream's offset), the wave then spreads them to scalar registers.
__device__ __forceinline__ int2 fetch_head(const int2* __restrict__ entries, const Geom& g, int seg, int lane) {
  return entries[(size_t)g.heads_off + (size_t)seg * kBatch + (lane & 7)];
}
__device__ __forceinline__ void spread_head(Batch& head, int2 e) {
#pragma unroll
  for (int i = 0; i < 8; ++i)
    head.c[i] = (static_cast<unsigned long long>(static_cast<unsigned>(__builtin_amdgcn_readlane(e.y, i))) << 32) |
                static_cast<unsigned>(__builtin_amdgcn_readlane(e.x, i));
}

// Walk `nb` batches of eight entries: `b` holds the first one, `stream` points at the one after it.  On return
// `b` holds the batch that follows the walked ones (the head of the next stage's stream) and `stream` points
// after that.
// VARIANT 2: single LDS tile; 3: three LDS buffers; 4, 5: three LDS buffers and 64 accumulators; 6, 7, 8: the flat
// kernels' two buffers with 64, 128, 64 accumulators (see gen_walk_asm.py)
constexpr bool small_acc(int variant) { return variant == 4 || variant == 5 || variant == 6 || variant == 8; }
// SHARE 2: the batches hold pairs of entries with one LDS offset (four pairs per batch), read once per pair.
template <int NQ, int VARIANT, int SHARE = 1>
__device__ __forceinline__ void walk_stream(Batch& b, const int2*& stream, int nb, int lane_base, int phase) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(stream);
  unsigned plo = uniform(static_cast<unsigned>(a)), phi = uniform(static_cast<unsigned>(a >> 32));
  nb = uniform(nb);
  const int ph = uniform(phase & 3);  // which of the four priority-rotated copies of the loop body to enter
#define TETRIS_WALK_OPERANDS                                                                                       \
  : [c0] "+{s[36:37]}"(b.c[0]), [c1] "+{s[38:39]}"(b.c[1]), [c2] "+{s[40:41]}"(b.c[2]), [c3] "+{s[42:43]}"(b.c[3]),      \
    [c4] "+{s[44:45]}"(b.c[4]), [c5] "+{s[46:47]}"(b.c[5]), [c6] "+{s[48:49]}"(b.c[6]), [c7] "+{s[50:51]}"(b.c[7]),      \
    [plo] "+{s72}"(plo), [phi] "+{s73}"(phi), [nb] "+s"(nb)                                                         \
  : [base] "v"(lane_base), [ph] "s"(ph)                                                                            \
  : "memory", "scc", "m0", TETRIS_S_CLOBBERS
#define TETRIS_WALK_CASE(V, Q)                                                                                     \
  if constexpr (VARIANT == (V == 0 ? 2 : V) && NQ == Q && SHARE == 1)                                              \
    asm volatile(TETRIS_WALK_PASTE(V, _ASM_, Q##_S1) TETRIS_WALK_OPERANDS, TETRIS_WALK_PASTE(V, _ACC_CLOBBERS, ),        \
                 TETRIS_WALK_PASTE(V, _VGPR_CLOBBERS_, Q));
#define TETRIS_WALK_CASE2(V, Q)                                                                                    \
  if constexpr (VARIANT == (V == 0 ? 2 : V) && NQ == Q && SHARE == 2)                                              \
    asm volatile(TETRIS_WALK_PASTE(V, _ASM_, Q##_S2) TETRIS_WALK_OPERANDS, TETRIS_WALK_PASTE(V, _ACC_CLOBBERS, ),        \
                 TETRIS_WALK_PASTE(V, _VGPR_CLOBBERS_, Q));
#define TETRIS_WALK_PASTE(V, mid, Q) TETRIS_WALK_PASTE2(TETRIS_WALK_PREFIX_##V, mid, Q)
#define TETRIS_WALK_PASTE2(pre, mid, Q) TETRIS_WALK_PASTE3(pre, mid, Q)
#define TETRIS_WALK_PASTE3(pre, mid, Q) pre##mid##Q
#define TETRIS_WALK_PREFIX_0 TETRIS_WALK
#define TETRIS_WALK_PREFIX_3 TETRIS_WALK3
#define TETRIS_WALK_PREFIX_4 TETRIS_WALK4
#define TETRIS_WALK_PREFIX_5 TETRIS_WALK5
#define TETRIS_WALK_PREFIX_6 TETRIS_WALK6
#define TETRIS_WALK_PREFIX_7 TETRIS_WALK7
#define TETRIS_WALK_PREFIX_8 TETRIS_WALK8
  TETRIS_WALK_CASE(0, 1)
  TETRIS_WALK_CASE(0, 2)
  TETRIS_WALK_CASE(0, 4)
  TETRIS_WALK_CASE(3, 1)
  TETRIS_WALK_CASE(3, 2)
  TETRIS_WALK_CASE(3, 4)
  TETRIS_WALK_CASE(4, 1)
  TETRIS_WALK_CASE(4, 2)
  TETRIS_WALK_CASE(5, 1)
  TETRIS_WALK_CASE(5, 2)
  TETRIS_WALK_CASE(6, 1)
  TETRIS_WALK_CASE(6, 2)
  TETRIS_WALK_CASE(7, 1)
  TETRIS_WALK_CASE(7, 2)
  TETRIS_WALK_CASE(7, 4)
  TETRIS_WALK_CASE(8, 1)
  TETRIS_WALK_CASE(8, 2)
  TETRIS_WALK_CASE2(0, 1)
  TETRIS_WALK_CASE2(0, 2)
  TETRIS_WALK_CASE2(0, 4)
  TETRIS_WALK_CASE2(3, 1)
  TETRIS_WALK_CASE2(3, 2)
  TETRIS_WALK_CASE2(3, 4)
  TETRIS_WALK_CASE2(4, 1)
  TETRIS_WALK_CASE2(4, 2)
  TETRIS_WALK_CASE2(5, 1)
  TETRIS_WALK_CASE2(5, 2)
#undef TETRIS_WALK_CASE2
#undef TETRIS_WALK_CASE
#undef TETRIS_WALK_OPERANDS
  stream = reinterpret_cast<const int2*>((static_cast<unsigned long long>(phi) << 32) | plo);
}

// Zeroes the first `live` accumulators (a multiple of 16, wave-uniform) with straight-line moves.
template <int VARIANT>
__device__ __forceinline__ void zero_accumulators(int live) {
#define TETRIS_Z4(a) "v_mov_b32 v" #a ", 0\n"
#define TETRIS_ZERO16(b0, b1, b2, b3, b4, b5, b6, b7, b8, b9, b10, b11, b12, b13, b14, b15)                              \
  asm volatile(TETRIS_Z4(b0) TETRIS_Z4(b1) TETRIS_Z4(b2) TETRIS_Z4(b3) TETRIS_Z4(b4) TETRIS_Z4(b5) TETRIS_Z4(b6)       \
               TETRIS_Z4(b7) TETRIS_Z4(b8) TETRIS_Z4(b9) TETRIS_Z4(b10) TETRIS_Z4(b11) TETRIS_Z4(b12) TETRIS_Z4(b13)     \
               TETRIS_Z4(b14) TETRIS_Z4(b15) ::                                                                        \
               : "v" #b0, "v" #b1, "v" #b2, "v" #b3, "v" #b4, "v" #b5, "v" #b6, "v" #b7, "v" #b8, "v" #b9, "v" #b10,   \
                 "v" #b11, "v" #b12, "v" #b13, "v" #b14, "v" #b15)
  if constexpr (small_acc(VARIANT)) {
    TETRIS_ZERO16(64, 65, 66, 67, 68, 69, 70, 71, 72, 73, 74, 75, 76, 77, 78, 79);
    if (live > 16) TETRIS_ZERO16(80, 81, 82, 83, 84, 85, 86, 87, 88, 89, 90, 91, 92, 93, 94, 95);
    if (live > 32) {
      TETRIS_ZERO16(96, 97, 98, 99, 100, 101, 102, 103, 104, 105, 106, 107, 108, 109, 110, 111);
      TETRIS_ZERO16(112, 113, 114, 115, 116, 117, 118, 119, 120, 121, 122, 123, 124, 125, 126, 127);
    }
  } else {
    TETRIS_ZERO16(128, 129, 130, 131, 132, 133, 134, 135, 136, 137, 138, 139, 140, 141, 142, 143);
    if (live > 16) TETRIS_ZERO16(144, 145, 146, 147, 148, 149, 150, 151, 152, 153, 154, 155, 156, 157, 158, 159);
    if (live > 32) {
      TETRIS_ZERO16(160, 161, 162, 163, 164, 165, 166, 167, 168, 169, 170, 171, 172, 173, 174, 175);
      TETRIS_ZERO16(176, 177, 178, 179, 180, 181, 182, 183, 184, 185, 186, 187, 188, 189, 190, 191);
    }
    if (live > 64) {
      TETRIS_ZERO16(192, 193, 194, 195, 196, 197, 198, 199, 200, 201, 202, 203, 204, 205, 206, 207);
      TETRIS_ZERO16(208, 209, 210, 211, 212, 213, 214, 215, 216, 217, 218, 219, 220, 221, 222, 223);
      TETRIS_ZERO16(224, 225, 226, 227, 228, 229, 230, 231, 232, 233, 234, 235, 236, 237, 238, 239);
      TETRIS_ZERO16(240, 241, 242, 243, 244, 245, 246, 247, 248, 249, 250, 251, 252, 253, 254, 255);
    }
  }
#undef TETRIS_ZERO16
#undef TETRIS_Z4
}

template <int VARIANT>
__device__ __forceinline__ float read_accumulator(int i) {  // i is wave-uniform
  float v;
  if constexpr (small_acc(VARIANT))
    asm volatile("s_set_gpr_idx_on %1, 0x1\n v_mov_b32 %0, v64\n s_set_gpr_idx_off\n" : "=v"(v) : "s"(i) : "m0");
  else
    asm volatile("s_set_gpr_idx_on %1, 0x1\n v_mov_b32 %0, v128\n s_set_gpr_idx_off\n" : "=v"(v) : "s"(i) : "m0");
  return v;
}

// Four consecutive accumulators i .. i+3 (i wave-uniform) under one switch of the index mode.
template <int VARIANT>
__device__ __forceinline__ void read_accumulators4(int i, float (&v)[4]) {
  if constexpr (small_acc(VARIANT))
    asm volatile("s_set_gpr_idx_on %4, 0x1\n v_mov_b32 %0, v64\n v_mov_b32 %1, v65\n v_mov_b32 %2, v66\n v_mov_b32 %3, v67\n"
                 "s_set_gpr_idx_off\n"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]) : "s"(i) : "m0");
  else
    asm volatile("s_set_gpr_idx_on %4, 0x1\n v_mov_b32 %0, v128\n v_mov_b32 %1, v129\n v_mov_b32 %2, v130\n v_mov_b32 %3, v131\n"
                 "s_set_gpr_idx_off\n"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]) : "s"(i) : "m0");
}

// Writes a wave's accumulators: slot k of the wave goes to the output channel lane k holds in lane_oc, quad q of a lane to
// the lane's four pixels of unit u0 + q.  The per-pixel byte offsets (inside the image block that starts at
// n_base, channel 0) are formed once; a channel then only adds a scalar offset, and out-of-range pixels carry an
// offset the buffer hardware drops.
template <int NQ, int VARIANT>
__device__ __forceinline__ void store_outputs(float* __restrict__ out, int lane_oc, const Geom& g, int u0, int n_base,
                                              int limg, int lrow, int lx, bool lane_ok) {
  constexpr unsigned kInvalid = 0x80000000u;
  const int upi = g.units_w * g.units_h;
  const int ohw = g.OH * g.OW;
  const long long rec = (long long)(g.N - n_base) * g.K * (long long)ohw * 4;
  const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
      out + (size_t)n_base * g.K * ohw, 0, rec > 0x7fffffffll ? 0x7fffffff : (int)rec, 0x00020000);
  unsigned ooff[NQ][4];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int u = u0 + q;
    const int ub_n = fast_div(u, g.m_upi);
    const int ur = u - ub_n * upi;
    const int ub_h = fast_div(ur, g.m_units_w);
    const int ub_w = ur - ub_h * g.units_w;
    const int n0 = (ub_n * g.nb + limg) * g.fold;  // first of the images this lane's quads belong to
    const int oh = ub_h * g.thi + lrow;
    const int ow = ub_w * (1 << g.jsh) * g.lw + lx;
    const bool ok = lane_ok && u < g.units && oh < g.OH;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + (j >> g.jsh);
      const int col = ow + (j & ((1 << g.jsh) - 1)) * g.lw;
      ooff[q][j] = (ok && n < g.N && col < g.OW) ? 4u * (unsigned)(((n - n_base) * g.K * g.OH + oh) * g.OW + col) : kInvalid;
    }
  }
  const bool relu = g.act != 0 && g.csplit == 1;  // a slice's partial sums are stored as they are
  for (int k = 0; k < g.g; ++k) {
    const int oc = __builtin_amdgcn_readlane(lane_oc, k);  // lane k fetched the slot's channel when the kernel began
    if (oc < 0) continue;  // padding slot
    const int soff = oc * ohw * 4;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j)
      {
        float v = read_accumulator<VARIANT>((k * NQ + q) * 4 + j);
        if (relu) v = fmaxf(v, 0.f);
        if (ooff[q][j] != kInvalid)
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), orsrc, (int)ooff[q][j], soff, 0);
      }
  }
}

// The same with ReLU and 2x2 max-pooling on the way out: the output is N x K x OH/2 x OW/2 (an odd last row or column
// is dropped).  Needs lw and thi even (the launcher checks): pixel j of a lane lies in column base + lx + lw*j' with
// an even base, so the lane right of an even lx holds the next column of the same row, and the lane lr further on
// the row below of the same image.  Every lane takes the maximum with its right neighbour, then with the lane below;
// lanes of even row and even column write.
template <int NQ, int VARIANT>
__device__ __forceinline__ void store_pooled(float* __restrict__ out, int lane_oc, const Geom& g, int u0, int n_base,
                                             int limg, int lrow, int lx, bool lane_ok) {
  constexpr unsigned kInvalid = 0x80000000u;
  const int upi = g.units_w * g.units_h;
  const int poh = g.OH >> 1, pow_ = g.OW >> 1;
  const int phw = poh * pow_;
  const long long rec = (long long)(g.N - n_base) * g.K * (long long)phw * 4;
  const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
      out + (size_t)n_base * g.K * phw, 0, rec > 0x7fffffffll ? 0x7fffffff : (int)rec, 0x00020000);
  const int lane = threadIdx.x & 63;
  const int right = 4 * min(lane + 1, 63), below = 4 * min(lane + g.lr, 63);  // byte addresses for ds_bpermute
  unsigned ooff[NQ][4];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int u = u0 + q;
    const int ub_n = fast_div(u, g.m_upi);
    const int ur = u - ub_n * upi;
    const int ub_h = fast_div(ur, g.m_units_w);
    const int ub_w = ur - ub_h * g.units_w;
    const int n0 = (ub_n * g.nb + limg) * g.fold;
    const int oh = ub_h * g.thi + lrow;
    const int ow = ub_w * (1 << g.jsh) * g.lw + lx;
    const bool ok = lane_ok && u < g.units && !(lrow & 1) && !(lx & 1) && (oh >> 1) < poh;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + (j >> g.jsh);
      const int col = ow + (j & ((1 << g.jsh) - 1)) * g.lw;
      ooff[q][j] = (ok && n < g.N && (col >> 1) < pow_)
                       ? 4u * (unsigned)(((n - n_base) * g.K * poh + (oh >> 1)) * pow_ + (col >> 1)) : kInvalid;
    }
  }
  for (int k = 0; k < g.g; ++k) {
    const int oc = __builtin_amdgcn_readlane(lane_oc, k);
    if (oc < 0) continue;  // padding slot
    const int soff = oc * phw * 4;
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j)
      {
        float v = fmaxf(read_accumulator<VARIANT>((k * NQ + q) * 4 + j), 0.f);
        v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(right, __builtin_bit_cast(int, v))));
        v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(below, __builtin_bit_cast(int, v))));
        if (ooff[q][j] != kInvalid)
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), orsrc, (int)ooff[q][j], soff, 0);
      }
  }
}


// ---- split layers: the last wave to finish adds the slices ---------------------------------------------------------
// The workgroups that share an output tile (the slices of its channel reduction) have consecutive logical ids inside
// one XCD's range, so they run on one XCD and meet in its L2.  Wave w of every slice holds the same output channels
// and pixels.  Once its partial sums are stored and acknowledged by L2 (vmcnt(0)), a wave takes a ticket of the
// (tile, wave) pair with an atomic add that L2 executes; the wave that draws ticket csplit - 1 knows that the same
// wave of every other slice has stored its sums before taking its ticket, reads all slices back with loads that
// bypass the CU's vector cache (sc1) and adds them in slice order.  Nobody waits for anybody.  The ticket is put
// back to zero by the wave that used it up.
__device__ __forceinline__ bool drew_last_ticket(int* __restrict__ tickets, int tile_id, int wave, const Geom& g) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's partial sums have reached L2
  int* t = tickets + tile_id * g.waves + wave;
  int old = 0;
  if ((threadIdx.x & 63) == 0) old = __hip_atomic_fetch_add(t, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  old = __builtin_amdgcn_readfirstlane(old);
  if (old != g.csplit - 1) return false;
  if ((threadIdx.x & 63) == 0) __hip_atomic_store(t, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return true;
}
constexpr int kBypassL1 = 16;  // cache policy of a buffer load: sc1 (agent scope), never served by the CU's vector cache

// The halo'd kernels' counterpart of store_outputs for the wave that drew the last ticket: out[...] = act(sum over the
// slices, in slice order, of the partial sums at the same offsets).
template <int NQ>
__device__ __forceinline__ void add_slices(const float* __restrict__ partial, float* __restrict__ out, int lane_oc,
                                           const Geom& g, int u0, int n_base, int limg, int lrow, int lx, bool lane_ok) {
  constexpr unsigned kInvalid = 0x80000000u;
  const int upi = g.units_w * g.units_h;
  const int ohw = g.OH * g.OW;
  const size_t out_elems = (size_t)g.N * g.K * ohw;
  const long long rec = (long long)(g.N - n_base) * g.K * (long long)ohw * 4;
  const int records = rec > 0x7fffffffll ? 0x7fffffff : (int)rec;
  const __amdgpu_buffer_rsrc_t orsrc =
      __builtin_amdgcn_make_buffer_rsrc(out + (size_t)n_base * g.K * ohw, 0, records, 0x00020000);
  unsigned ooff[NQ][4];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int u = u0 + q;
    const int ub_n = fast_div(u, g.m_upi);
    const int ur = u - ub_n * upi;
    const int ub_h = fast_div(ur, g.m_units_w);
    const int ub_w = ur - ub_h * g.units_w;
    const int n0 = (ub_n * g.nb + limg) * g.fold;
    const int oh = ub_h * g.thi + lrow;
    const int ow = ub_w * (1 << g.jsh) * g.lw + lx;
    const bool ok = lane_ok && u < g.units && oh < g.OH;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + (j >> g.jsh);
      const int col = ow + (j & ((1 << g.jsh) - 1)) * g.lw;
      ooff[q][j] = (ok && n < g.N && col < g.OW) ? 4u * (unsigned)(((n - n_base) * g.K * g.OH + oh) * g.OW + col) : kInvalid;
    }
  }
  const bool relu = g.act != 0;
  for (int k = 0; k < g.g; ++k) {
    const int oc = __builtin_amdgcn_readlane(lane_oc, k);
    if (oc < 0) continue;  // padding slot
    const int soff = oc * ohw * 4;
    float sum[NQ][4];
    for (int s = 0; s < g.csplit; ++s) {
      const __amdgpu_buffer_rsrc_t prsrc = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<float*>(partial) + (size_t)s * out_elems + (size_t)n_base * g.K * ohw, 0, records, 0x00020000);
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // an offset out of range reads as zero
          const float v = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(prsrc, (int)ooff[q][j], soff, kBypassL1));
          sum[q][j] = s == 0 ? v : sum[q][j] + v;
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (ooff[q][j] != kInvalid)
          __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, relu ? fmaxf(sum[q][j], 0.f) : sum[q][j]), orsrc,
                                                (int)ooff[q][j], soff, 0);
  }
}

// SPT: 16-byte LDS slots of the unit group a thread stages (1 or 2)
template <int NQ, int SPT>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(88))) void spconv2d_kernel(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  TETRIS_STAMP_ENTRY();
  touch_kernel_arguments();
  TETRIS_STAMP_ARGS();
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = uniform(tid >> 6);
  const int nthreads = blockDim.x;

  // Workgroup -> (unit group, channel block).  Consecutive workgroup ids go round-robin to the eight XCDs;
  // give each XCD a contiguous range of logical ids so that the channel blocks of one unit group, which read
  // the same input, share an L2.
  const int total = g.ugroups * g.kblocks * g.csplit;
  const int per_xcd = gridDim.x >> 3;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const int tile_id = fast_div(logical, g.m_csplit);  // slices of one output tile are neighbours: same XCD, same L2
  const int slice = logical - tile_id * g.csplit;
  const int ugroup = fast_div(tile_id, g.m_kblocks);
  const int kblock = tile_id - ugroup * g.kblocks;
  const int u0 = ugroup * NQ;
  // this workgroup's stages (multiply-high division: make_geom checks its range)
  const int st0 = fast_div(slice * g.stages, g.m_csplit), st1 = fast_div((slice + 1) * g.stages, g.m_csplit);
  // a slice of a split reduction writes its partial sums to its own copy of the output (`out` is then that scratch)
  const size_t out_elems = (size_t)g.N * g.K * g.OH * g.OW;
  const int upi = g.units_w * g.units_h;  // units per image block
  const int n_base = fast_div(u0, g.m_upi) * g.nb * g.fold;   // first image this workgroup touches

  zero_accumulators<2>(g.g * 4 * NQ);

  // ---- input staging set-up: which global columns feed each 16-byte LDS slot this thread owns -------------
  const size_t hw = (size_t)g.in_hw;  // floats per (image, channel) plane in memory
  const float* in_base = in + (size_t)n_base * g.C * hw;
  const long long rec = (long long)(g.N - n_base) * g.C * (long long)hw * 4;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(in_base), 0, rec > 0x7fffffffll ? 0x7fffffff : (int)rec, 0x00020000);
  constexpr unsigned kInvalid = 0x80000000u;  // beyond num_records: the load returns 0
  unsigned voff[SPT][4];
  int dst[SPT];
  bool owns[SPT];
  const int cgi = (SPT == 1) ? fast_div(tid, g.m_fill_slots) : 0;  // which channel of each group of `cg` this thread stages
  {
    const int per_row = g.stride * g.ng;
    const int per_img = g.ih * per_row;
#pragma unroll
    for (int k = 0; k < SPT; ++k) {
      const int fs = (SPT == 1) ? tid - cgi * g.fill_slots : tid + k * nthreads;
      owns[k] = fs < g.fill_slots && cgi < g.cg;
      const int q = fast_div(fs, g.m_slots_per_unit);
      int r = fs - q * g.slots_per_unit;
      const int img = fast_div(r, g.m_per_img);
      r -= img * per_img;
      const int row = fast_div(r, g.m_per_row);
      r -= row * per_row;
      const int par = fast_div(r, g.m_ng);
      const int m = r - par * g.ng;
      const int u = u0 + q;
      const int ub_n = fast_div(u, g.m_upi);
      const int ur = u - ub_n * upi;
      const int ub_h = fast_div(ur, g.m_units_w);
      const int ub_w = ur - ub_h * g.units_w;
      const int n0 = (ub_n * g.nb + img) * g.fold;  // quad j of the slot belongs to image n0 + (j >> jsh)
      const int ihh = ub_h * g.thi * g.stride - g.pad + row;
      const int col0 = ub_w * (1 << g.jsh) * g.lw * g.stride - g.pad + par + g.stride * m;
      const bool row_ok = owns[k] && u < g.units && ihh >= 0 && ihh < g.H;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + (j >> g.jsh);
        const int c = col0 + (j & ((1 << g.jsh) - 1)) * g.stride * g.lw;
        const unsigned b = (unsigned)(((n - n_base) * g.C + cgi) * (int)hw + ihh * g.step * g.in_w) * 4u;
        voff[k][j] = (row_ok && n < g.N && c >= 0 && c < g.W) ? b + 4u * (unsigned)(c * g.step) : kInvalid;
      }
      dst[k] = q * g.region + 4 * (img * g.img_stride + cgi * g.plane + row * g.pitch + par * g.par + m * 4);
    }
  }

  // ---- lane -> pixels: the same for every quad, which only differ by their LDS region ---------------------
  const int ly = fast_div(lane, g.m_lr);
  const int lx = lane - ly * g.lr;
  const int limg = fast_div(ly, g.m_thi);
  const int lrow = ly - limg * g.thi;
  const bool row_ok = ly < g.lh && limg < g.nb;
  const bool lane_ok = row_ok && lx < g.lw;
  // idle lane positions of a live row keep the row's address pattern (they read slots nobody needs)
  // Lanes of rows that do not exist keep walking the same address pattern (their results are never stored): a lane
  // parked at one fixed address would collide with a live lane's banks in every read (measured: 20-38 % of the LDS
  // cycles of such tiles were bank conflicts).
  int lane_base = 4 * ((g.nb > 1 ? limg * g.img_stride + lrow * g.stride * g.pitch : ly * g.stride * g.pitch) + lx * 4);

  const int grp = kblock * g.waves + wave;  // this wave's stream group
  const int lane_oc = lane < g.g ? oc_order[grp * g.g + lane] : -1;  // fetched now, used when the outputs are written
  constexpr int ITERS = kFillItems / SPT;
  float stage_buf[SPT][ITERS][4];

  // Issue the global loads of stage `st` into registers.  The range check of a buffer load covers the scalar offset
  // too (measured on MI355X), so a staged channel past C in the last stage of a ragged C reads zeros at the tensor's
  // end and, inside the tensor, the next image's data, which no entry refers to.
  auto fetch = [&](int st) {
    const int soff0 = st * g.tile_ic * (int)hw * 4;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      if (it < g.fill_iters) {
        const int soff = soff0 + it * g.cg * (int)hw * 4;
#pragma unroll
        for (int k = 0; k < SPT; ++k)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            stage_buf[k][it][j] =
                __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voff[k][j], soff, 0));
      }
    }
  };
  auto commit = [&]() {  // write the fetched registers into LDS
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      if (it < g.fill_iters) {
#pragma unroll
        for (int k = 0; k < SPT; ++k) {
          if (owns[k] && it * g.cg + cgi < g.tile_ic) {
            float4 v = make_float4(stage_buf[k][it][0], stage_buf[k][it][1], stage_buf[k][it][2], stage_buf[k][it][3]);
            *reinterpret_cast<float4*>(smem + dst[k] + 4 * it * g.cg * g.plane) = v;
          }
        }
      }
    }
  };

  // the wave's streams of consecutive stages lie back to back: keep the head batch of the next one in SGPRs
  const int32_t* go = grp_off + grp * g.stages;
  const int32_t* gp = grp_pair + grp * g.stages;
  const int2 head_entry = fetch_head(entries, g, grp * g.stages + st0, lane);  // in flight together with the offsets
  int o0 = uniform(go[st0]), o1 = uniform(go[st0 + 1]), o2 = uniform(go[min(st0 + 2, g.stages)]);
  const int o_end = uniform(go[st1]);
  const int2* stream = entries + o0 + 8;
  Batch head;
  spread_head(head, head_entry);
  TETRIS_STAMP(3);

  // The scalar loads of the walk run only one 64-byte fetch ahead, far too little to cover a miss in L2.  So each
  // wave touches the stream of the stage after next with one vector load (a dword per 128-byte line, 8 KB at most)
  // whose value is only consumed after the next staging wait.
  const int* words = reinterpret_cast<const int*>(entries);
  auto touch = [&](int from, int to) {
    const int e = from + lane * 16;
    return e < to ? __builtin_nontemporal_load(words + 2 * (size_t)e) : 0;
  };
  int sink = touch(o0 + 8, o_end);  // as much of the wave's whole stream as one touch covers (8 KB)
  int touched = 0;

  TETRIS_STAMP(11);
  fetch(st0);
  TETRIS_STAMP(2);
  for (int st = st0; st < st1; ++st) {
    commit();
    sink ^= touched;
    __syncthreads();
    if (st == st0) TETRIS_STAMP(4);
    if (st + 1 < st1) fetch(st + 1);  // in flight while this stage is computed
    const int o3 = uniform(go[min(st + 3, g.stages)]);  // stream bounds two stages ahead
    touched = touch(o2, o3);
    const int nb = (o1 - o0) >> 3;
    const int np = uniform(gp[st]) >> 3;  // the stream's batches of pairs come first
    if (np > 0) TETRIS_STAMP_WALK((walk_stream<NQ, 2, 2>(head, stream, np, lane_base, (wave >> 2) * 2 + st)));
    if (nb - np > 0) TETRIS_STAMP_WALK((walk_stream<NQ, 2, 1>(head, stream, nb - np, lane_base, (wave >> 2) * 2 + st + 1)));
    o0 = o1; o1 = o2; o2 = o3;
    __syncthreads();  // everyone is done reading the tile
  }
  TETRIS_STAMP(5);

  // ---- write the outputs -------------------------------------------------------------------------------------
  if (g.N < 0) out[0] = __builtin_bit_cast(float, sink ^ touched);  // never true: keeps the touching loads alive
  if (g.act == 2) store_pooled<NQ, 2>(out, lane_oc, g, u0, n_base, limg, lrow, lx, lane_ok);
  else store_outputs<NQ, 2>(out + (size_t)slice * out_elems, lane_oc, g, u0, n_base, limg, lrow, lx, lane_ok);
  if (g.fused && drew_last_ticket(tickets, tile_id, wave, g))
    add_slices<NQ>(out, final_out, lane_oc, g, u0, n_base, limg, lrow, lx, lane_ok);
  TETRIS_STAMP_END();
}

static_assert(TETRIS_WALK_TILE_BYTES == kTileBytes && TETRIS_WALK_BUF_BYTES == kBufBytes &&
                  TETRIS_WALK_HALF_BUF_BYTES == kHalfBufBytes && TETRIS_WALK_FLAT_BUF_BYTES == kFlatBufBytes &&
                  TETRIS_WALK_FLAT_HALF_BUF_BYTES == kFlatHalfBufBytes,
              "the generated inner loop was made for other LDS sizes");

// Triple-buffered variants: one workgroup per CU with 3 * kBufBytes of its 160 KiB LDS.
//   * Input goes from global memory straight into LDS (buffer loads with the LDS bit: 64 lanes fill 64
//     consecutive dwords, each from its own bounds-checked global address), two stages ahead of the compute, so
//     no registers hold staged data and nothing is copied by the waves.
//   * One barrier per stage, placed in the MIDDLE of the stage's walk: it certifies that every wave's loads for
//     the next stage have landed and that every wave has left the previous stage, so the buffer two stages ahead
//     can be refilled.  A wave that finishes a stage early walks on into the next one.
//   * In an 8-wave workgroup half of the waves issue their loads right after the barrier, the other half at the
//     end of the stage; every SIMD holds a wave of each half, so one computes while the other issues loads.
// WAVES == 8: 128 accumulators per wave, two waves per SIMD.  WAVES == 16: 64 accumulators and at most 128 VGPRs
// per wave, four waves per SIMD, which hides more of the LDS latency (the loop alone runs about 1.3x faster).
template <int NQ, int WAVES, int VARIANT>
__device__ __forceinline__ void conv3_body(const float* __restrict__ in, float* __restrict__ out,
                                           const int2* __restrict__ entries, const int32_t* __restrict__ grp_off,
                                           const int32_t* __restrict__ grp_pair, const int32_t* __restrict__ oc_order,
                                           float* __restrict__ final_out, int* __restrict__ tickets, const Geom& g) {
  constexpr int MAXC = VARIANT == 3 ? kMaxChunks : kMaxChunks16;
  constexpr int BUF = VARIANT == 5 ? kHalfBufBytes : kBufBytes;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  TETRIS_STAMP_ENTRY();
  touch_kernel_arguments();
  TETRIS_STAMP_ARGS();
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = uniform(tid >> 6);

  const int total = g.ugroups * g.kblocks * g.csplit;
  const int per_xcd = gridDim.x >> 3;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const int tile_id = fast_div(logical, g.m_csplit);  // slices of one output tile are neighbours: same XCD, same L2
  const int slice = logical - tile_id * g.csplit;
  const int ugroup = fast_div(tile_id, g.m_kblocks);
  const int kblock = tile_id - ugroup * g.kblocks;
  const int u0 = ugroup * NQ;
  // this workgroup's stages (multiply-high division: make_geom checks its range)
  const int st0 = fast_div(slice * g.stages, g.m_csplit), st1 = fast_div((slice + 1) * g.stages, g.m_csplit);
  // a slice of a split reduction writes its partial sums to its own copy of the output (`out` is then that scratch)
  const size_t out_elems = (size_t)g.N * g.K * g.OH * g.OW;
  const int upi = g.units_w * g.units_h;
  const int n_base = fast_div(u0, g.m_upi) * g.nb * g.fold;

  const size_t hw = (size_t)g.in_hw;  // floats per (image, channel) plane in memory
  const float* in_base = in + (size_t)n_base * g.C * hw;
  const long long rec = (long long)(g.N - n_base) * g.C * (long long)hw * 4;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(in_base), 0, rec > 0x7fffffffll ? 0x7fffffff : (int)rec, 0x00020000);
  constexpr unsigned kInvalid = 0x80000000u;

  // ---- staging plan: chunk x = wave + stagers * i of every staged channel belongs to wave < stagers.  A 16-wave
  // workgroup stages with waves 0-3 alone when it can: they are the oldest wave of their SIMD, which the hardware
  // serves first, so they finish their share of a stage early and would otherwise idle at the barrier (-5 %).
  unsigned voff[MAXC];   // global byte offset of this lane's dword (channel 0 of the stage), or kInvalid
  int loff[MAXC];        // LDS byte offset of the chunk inside a buffer (channel 0), wave-uniform
  bool writes[MAXC];     // this lane's dword lies inside the plane (the last chunk of a plane may overhang)
  // chunks this wave stages: x = wave, wave + stagers, ... below nchunks -- a wave-uniform count, so that the plan
  // and every issue() skip the other slots with scalar branches (a load under an empty exec mask still costs its issue)
  TETRIS_STAMP(11);
  const int stager_shift = g.stagers == 16 ? 4 : g.stagers == 8 ? 3 : 2;  // stagers is 4, 8 or 16
  const int n_live = wave < g.stagers ? min(g.ni, (g.nchunks - wave + g.stagers - 1) >> stager_shift) : 0;
  // The plan of a chunk costs some hundred cycles of index arithmetic, and the loads of a stage keep the CU's address
  // unit busy for about as long as the whole plan takes: so the first stage's loads of chunk i go out as soon as chunk
  // i's plan is made, and the address unit works while the plan of chunk i + 1 is computed.
  {
    const int per_unit = g.nb * g.cpp;
    unsigned char* buf0 = smem + (st0 % kBufs) * BUF;
    const int c00 = st0 * g.tile_ic;
    const int nch0 = min(g.tile_ic, g.C - c00);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      writes[i] = false;
      voff[i] = kInvalid;
      loff[i] = 0;
      if (i >= n_live) continue;
      const int x = wave + g.stagers * i;
      const int q = fast_div(x, g.m_per_unit);
      const int rem = x - q * per_unit;
      const int img = fast_div(rem, g.m_cpp);
      const int chunk = rem - img * g.cpp;
      const int p = chunk * 64 + lane;  // dword inside the (unit, image, channel) plane
      const int row = fast_div(p, g.m_pitch);
      const int within = p - row * g.pitch;
      const int par = fast_div(within, g.m_par);
      const int wp = within - par * g.par;
      const int m = wp >> 2, j = wp & 3;
      const int u = u0 + q;
      const int ub_n = fast_div(u, g.m_upi);
      const int ur = u - ub_n * upi;
      const int ub_h = fast_div(ur, g.m_units_w);
      const int ub_w = ur - ub_h * g.units_w;
      const int n = (ub_n * g.nb + img) * g.fold + (j >> g.jsh);  // quad j: image j >> jsh, column group j & mask
      const int ihh = ub_h * g.thi * g.stride - g.pad + row;
      const int col = ub_w * (1 << g.jsh) * g.lw * g.stride - g.pad + par + g.stride * (m + (j & ((1 << g.jsh) - 1)) * g.lw);
      writes[i] = p < g.plane;
      const bool ok = writes[i] && par < g.stride && u < g.units && n < g.N && ihh >= 0 && ihh < g.H && col >= 0 &&
                      col < g.W;
      voff[i] = ok ? (unsigned)(((n - n_base) * g.C) * (int)hw + ihh * g.step * g.in_w + col * g.step) * 4u : kInvalid;
      loff[i] = uniform(q * g.region + 4 * (img * g.img_stride + chunk * 64));
      if (writes[i])
        for (int ch = 0; ch < nch0; ++ch)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              rsrc, (__attribute__((address_space(3))) void*)(buf0 + loff[i] + 4 * ch * g.plane), 4, (int)voff[i],
              (c00 + ch) * (int)hw * 4, 0, 0);
    }
  }
  auto issue = [&](int st) {  // start the loads of stage `st` into buffer st % 3
    if (st >= st1 || n_live == 0) return;
    unsigned char* buf = smem + (st % kBufs) * BUF;
    const int c0 = st * g.tile_ic;
    const int nch = min(g.tile_ic, g.C - c0);
    for (int ch = 0; ch < nch; ++ch) {
      const int soff = (c0 + ch) * (int)hw * 4;
      const int chan = 4 * ch * g.plane;
#pragma unroll
      for (int i = 0; i < MAXC; ++i)
        if (i < n_live && writes[i])
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              rsrc, (__attribute__((address_space(3))) void*)(buf + loff[i] + chan), 4, (int)voff[i],
              soff, 0, 0);
    }
  };

  // which waves issue their loads right after the barrier, and which at the end of the stage
  const int prio_phase = WAVES == 16 ? wave >> 2 : (wave >> 2) * 2;  // waves of one SIMD start in different phases
  const bool split = g.stagers == WAVES;  // everybody stages: one half early, one half late
  const bool early = wave < g.stagers && (!split || (wave & 4) == 0);
  const bool late = split && (wave & 4) != 0;
  // When only the oldest waves stage, the workgroup starts on stage st0 as soon as its loads have landed; those of
  // stage st0 + 1 are issued then and land during the first half of the walk (-1 % per launch).  When everybody
  // stages it pays to have both stages in flight before the first wait (measured both ways).
  const bool early_start = WAVES == 16 || !split;
  // The first stage's loads have gone out (with the plan, above) before anything else is fetched (the streams'
  // offsets and head entries, the wave's channels), so that those round trips run under the input's.
  if (!early_start) issue(st0 + 1);
  TETRIS_STAMP(2);
  zero_accumulators<VARIANT>(g.g * 4 * NQ);

  // ---- lane -> pixels -------------------------------------------------------------------------------------------
  const int ly = fast_div(lane, g.m_lr);
  const int lx = lane - ly * g.lr;
  const int limg = fast_div(ly, g.m_thi);
  const int lrow = ly - limg * g.thi;
  const bool row_ok = ly < g.lh && limg < g.nb;
  const bool lane_ok = row_ok && lx < g.lw;
  // Lanes of rows that do not exist keep walking the same address pattern (their results are never stored): a lane
  // parked at one fixed address would collide with a live lane's banks in every read.
  const int lane_base = 4 * ((g.nb > 1 ? limg * g.img_stride + lrow * g.stride * g.pitch : ly * g.stride * g.pitch) + lx * 4);

  const int grp = kblock * g.waves + wave;
  const int lane_oc = lane < g.g ? oc_order[grp * g.g + lane] : -1;  // fetched now, used when the outputs are written
  const int32_t* go = grp_off + grp * g.stages;
  const int32_t* gp = grp_pair + grp * g.stages;
  const int2 head_entry = fetch_head(entries, g, grp * g.stages + st0, lane);  // in flight together with the offsets
  int o0 = uniform(go[st0]), o1 = uniform(go[st0 + 1]), o2 = uniform(go[min(st0 + 2, g.stages)]);
  int o3 = uniform(go[min(st0 + 3, g.stages)]);
  const int o_end = uniform(go[st1]);
  const int2* stream = entries + o0 + 8;
  Batch head;
  spread_head(head, head_entry);
  TETRIS_STAMP(3);

  const int* words = reinterpret_cast<const int*>(entries);
  auto touch = [&](int from, int to) {  // pull a stream range into L2: a dword per 128-byte line, 8 KB at most
    const int e = from + lane * 16;
    return e < to ? __builtin_nontemporal_load(words + 2 * (size_t)e) : 0;
  };
  int sink = touch(o0 + 8, o_end);  // as much of the wave's whole stream as one touch covers (8 KB)

  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0); the expcnt and lgkmcnt fields stay at their maxima
  __syncthreads();
  TETRIS_STAMP(4);
  if (early_start) issue(st0 + 1);
  for (int st = st0; st < st1; ++st) {
    const int o4 = uniform(go[min(st + 4, g.stages)]);  // fetched an iteration before it is needed
    const int nb = (o1 - o0) >> 3;
    const int np = uniform(gp[st]) >> 3;  // the stream's batches of pairs come first
    const int base = lane_base + (st % kBufs) * BUF;
    // The barrier sits between the two parts of the stage's walk: after the pairs when the stream has them (they are
    // about half of a typical stream), else in the middle of the singles.
    const int first = np > 0 ? 0 : nb >> 1;
    // The touching load is issued and its result consumed inside one iteration, behind the wait that is due anyway: a
    // result carried into the next iteration may be given a register copy at the loop's end, and that copy waits for
    // every load in flight, the next stage's included.
    const int touched = touch(o2, o3);
    if (np > 0) TETRIS_STAMP_WALK((walk_stream<NQ, VARIANT, 2>(head, stream, np, base, prio_phase + 2 * st)));
    if (first > 0) TETRIS_STAMP_WALK((walk_stream<NQ, VARIANT, 1>(head, stream, first, base, prio_phase + 2 * st)));
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): my loads of stage st + 1 have landed
    sink ^= touched;
    __syncthreads();                     // ... and so have everyone's; nobody reads the buffer of stage st - 1 any more
    if (early) issue(st + 2);
    if (nb - np - first > 0)
      TETRIS_STAMP_WALK((walk_stream<NQ, VARIANT, 1>(head, stream, nb - np - first, base, prio_phase + 2 * st + 1)));
    if (late) issue(st + 2);
    o0 = o1; o1 = o2; o2 = o3; o3 = o4;
  }
  TETRIS_STAMP(5);

  // ---- write the outputs -------------------------------------------------------------------------------------
  if (g.N < 0) out[0] = __builtin_bit_cast(float, sink);  // never true: keeps the touching loads alive
  if (g.act == 2) store_pooled<NQ, VARIANT>(out, lane_oc, g, u0, n_base, limg, lrow, lx, lane_ok);
  else store_outputs<NQ, VARIANT>(out + (size_t)slice * out_elems, lane_oc, g, u0, n_base, limg, lrow, lx, lane_ok);
  if (g.fused && drew_last_ticket(tickets, tile_id, wave, g))
    add_slices<NQ>(out, final_out, lane_oc, g, u0, n_base, limg, lrow, lx, lane_ok);
  TETRIS_STAMP_END();
}

template <int NQ>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(TETRIS_WALK3_FIRST_RESERVED_4))) void spconv2d_kernel3(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  conv3_body<NQ, 8, 3>(in, out, entries, grp_off, grp_pair, oc_order, final_out, tickets, g);
}

template <int NQ>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_num_vgpr(TETRIS_WALK4_FIRST_RESERVED_2))) void spconv2d_kernel4(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  conv3_body<NQ, 16, 4>(in, out, entries, grp_off, grp_pair, oc_order, final_out, tickets, g);
}

template <int NQ>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(TETRIS_WALK5_FIRST_RESERVED_2))) void spconv2d_kernel5(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  conv3_body<NQ, 8, 5>(in, out, entries, grp_off, grp_pair, oc_order, final_out, tickets, g);
}

// Pointwise layers (1x1, stride 1, no padding) with flat tiles: a lane owns four consecutive pixels of one image
// (a quad), a unit is 64 consecutive quads of the batch, and LDS holds one 1 KiB row per staged channel and unit.
//   * Staging is ONE 16-byte-per-lane buffer load that writes LDS directly per (channel, unit): the address unit
//     spends the same 16 cycles on a wave's load whether its lanes carry 4 or 16 bytes, so this stages at four times
//     the rate of the dword loads the halo'd tiles need.
//   * Two LDS buffers; a stage is ONE walk followed by ONE barrier (these layers' stages hold few entries per wave,
//     and every walk call costs a scalar fetch that nothing overlaps): after the barrier of stage st the buffer it
//     used is refilled with stage st + 2, which has the whole walk of stage st + 1 to land.
//   * The walk is the same generated loop (entry offset = channel * 1 KiB); a lane stores 16 contiguous bytes per
//     output channel when H*W is a multiple of four.
// VARIANT 6: 16 waves, 64 accumulators; 7: 8 waves, 128 accumulators (64 KiB buffers, one workgroup per CU);
// 8: 8 waves, 64 accumulators, 32 KiB buffers, two workgroups per CU.
template <int NQ, int WAVES, int VARIANT>
__device__ __forceinline__ void flat_body(const float* __restrict__ in, float* __restrict__ out,
                                          const int2* __restrict__ entries, const int32_t* __restrict__ grp_off,
                                          const int32_t* __restrict__ grp_pair, const int32_t* __restrict__ oc_order,
                                          float* __restrict__ final_out, int* __restrict__ tickets, const Geom& g) {
  constexpr int BUF = VARIANT == 8 ? kFlatHalfBufBytes : kFlatBufBytes;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  TETRIS_STAMP_ENTRY();
  touch_kernel_arguments();
  TETRIS_STAMP_ARGS();
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = uniform(tid >> 6);

  const int total = g.ugroups * g.kblocks * g.csplit;
  const int per_xcd = gridDim.x >> 3;
  const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (logical >= total) return;
  const int tile_id = fast_div(logical, g.m_csplit);
  const int slice = logical - tile_id * g.csplit;
  const int ugroup = fast_div(tile_id, g.m_kblocks);
  const int kblock = tile_id - ugroup * g.kblocks;
  const int u0 = ugroup * NQ;
  const int st0 = fast_div(slice * g.stages, g.m_csplit), st1 = fast_div((slice + 1) * g.stages, g.m_csplit);
  const size_t out_elems = (size_t)g.N * g.K * g.OH * g.OW;
  const int hw = g.in_hw;        // floats per (image, channel) plane of the input in memory
  const int ohw = g.OH * g.OW;   // ... of the output: the same, unless the layer is strided
  const int n_base = fast_div(u0 * 64, g.m_qi);  // first image this workgroup touches

  // ---- input staging: issued first, so that the loads run under the rest of the set-up -----------------------------
  const float* in_base = in + (size_t)n_base * g.C * hw;
  const long long rec = (long long)(g.N - n_base) * g.C * (long long)hw * 4;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(in_base), 0, rec > 0x7fffffffll ? 0x7fffffff : (int)rec, 0x00020000);
  constexpr unsigned kInvalid = 0x80000000u;
  unsigned voff[NQ], ooff[NQ];
  int npx[NQ];  // pixels of the lane's quad that exist (the last quad of an image may be short)
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int qd = (u0 + q) * 64 + lane;
    const int n = fast_div(qd, g.m_qi);
    const int qq = qd - n * g.qi;
    const bool ok = qd < g.quads_total;
    voff[q] = ok ? 4u * (unsigned)((n - n_base) * g.C * hw + 4 * qq) : kInvalid;
    ooff[q] = ok ? 4u * (unsigned)((n - n_base) * g.K * ohw + 4 * qq) : kInvalid;
    npx[q] = ok ? min(4, ohw - 4 * qq) : 0;
  }
  // A strided layer's quad is four pixels of the sub-grid, `step` apart in memory (and possibly in two rows): dword
  // 64 k + lane of a unit's LDS row is element (64 k + lane) % 4 of quad (64 k + lane) / 4 of the unit.
  const bool strided = g.step != 1;
  unsigned soffs[NQ][4];
#pragma unroll
  for (int q = 0; q < NQ; ++q)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      soffs[q][k] = kInvalid;
      if (strided) {
        const int d = 64 * k + lane;
        const int qd = (u0 + q) * 64 + (d >> 2);
        const int n = fast_div(qd, g.m_qi);
        const int px = 4 * (qd - n * g.qi) + (d & 3);
        const int row = fast_div(px, g.m_ow);
        const int col = px - row * g.OW;
        if (qd < g.quads_total && px < ohw)
          soffs[q][k] = 4u * (unsigned)((n - n_base) * g.C * hw + row * g.step * g.in_w + col * g.step);
      }
    }
  // channels ch = wave, wave + stagers, ... of a stage are staged by wave < stagers: NQ loads of 1 KiB per channel
  auto issue = [&](int st) {
    if (st >= st1 || wave >= g.stagers) return;
    unsigned char* buf = smem + (st & 1) * BUF;
    const int c0 = st * g.tile_ic;
    const int nch = min(g.tile_ic, g.C - c0);
    for (int ch = wave; ch < nch; ch += g.stagers) {
      const int soff = (c0 + ch) * hw * 4;
      if (!strided) {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(
              rsrc, (__attribute__((address_space(3))) void*)(buf + q * g.region + ch * 1024), 16, (int)voff[q], soff, 0, 0);
      } else {
#pragma unroll
        for (int q = 0; q < NQ; ++q)
#pragma unroll
          for (int k = 0; k < 4; ++k)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rsrc, (__attribute__((address_space(3))) void*)(buf + q * g.region + ch * 1024 + k * 256), 4,
                (int)soffs[q][k], soff, 0, 0);
      }
    }
  };
  TETRIS_STAMP(11);
  issue(st0);
  issue(st0 + 1);
  TETRIS_STAMP(2);

  // ---- the wave's streams.  Lane i keeps the stream offset of stage chunk0 + i, so a stage costs no memory access
  // for them (reloaded every 60 stages).
  const int grp = kblock * g.waves + wave;
  const int lane_oc = lane < g.g ? oc_order[grp * g.g + lane] : -1;
  const int32_t* go = grp_off + grp * g.stages;
  int chunk0 = st0;
  int gov = go[min(chunk0 + lane, g.stages)];
  const int2 head_entry = fetch_head(entries, g, grp * g.stages + st0, lane);  // in flight together with the offsets
  auto off_at = [&](int st) { return __builtin_amdgcn_readlane(gov, min(st, g.stages) - chunk0); };

  zero_accumulators<VARIANT>(g.g * 4 * NQ);

  int o0 = off_at(st0), o1 = off_at(st0 + 1);
  const int2* stream = entries + o0 + 8;
  Batch head;
  spread_head(head, head_entry);
  TETRIS_STAMP(3);
  const int* words = reinterpret_cast<const int*>(entries);
  auto touch = [&](int from, int to) {  // pull a stream range into L2: a dword per 128-byte line, 8 KB at most
    const int e = from + lane * 16;
    return e < to ? __builtin_nontemporal_load(words + 2 * (size_t)e) : 0;
  };
  // The whole stream is asked for now, 8 KB per load and 32 KB at most (4096 entries: more than a wave of a pointwise
  // layer holds): a touching load inside the stage loop would make the compiler wait for every load in flight, the
  // staged input included, before it reuses the load's destination register at the top of the next iteration.
  int sink = 0;
  {
    const int end = off_at(min(st1, st0 + 63));
#pragma unroll
    for (int k = 0; k < 4; ++k) sink ^= touch(o0 + 8 + k * 1024, end);
  }

  const int lane_base = lane * 16;
  const int prio_phase = WAVES == 16 ? wave >> 2 : (wave >> 2) * 2;
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): stages st0 and st0 + 1 have landed
  __syncthreads();
  TETRIS_STAMP(4);
  for (int st = st0; st < st1; ++st) {
    if (st + 3 - chunk0 > 63) {  // the lanes' stream offsets run out: fetch the next 64
      chunk0 = st;
      gov = go[min(chunk0 + lane, g.stages)];
      // waited for here, once in 60 stages: left pending, every read of a lane of gov in the loop would be preceded
      // by a wait for all loads in flight, the staged input included
      __builtin_amdgcn_s_waitcnt(0x0f70);
    }
    const int nb = (o1 - o0) >> 3;
    if (nb > 0) TETRIS_STAMP_WALK((walk_stream<NQ, VARIANT>(head, stream, nb, lane_base + (st & 1) * BUF, prio_phase + st)));
    o0 = o1;
    o1 = off_at(st + 2);
    if (st + 1 < st1) {
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): my loads of stage st + 1 have landed
      __syncthreads();                     // ... and everyone's; nobody reads the buffer of stage st any more
      issue(st + 2);
    }
  }
  TETRIS_STAMP(5);

  // ---- write the outputs ------------------------------------------------------------------------------------------
  if (g.N < 0) out[0] = __builtin_bit_cast(float, sink);  // never true: keeps the touching loads alive
  float* obase = out + (size_t)slice * out_elems + (size_t)n_base * g.K * ohw;
  const long long orec = (long long)(g.N - n_base) * g.K * (long long)ohw * 4;
  const __amdgpu_buffer_rsrc_t orsrc =
      __builtin_amdgcn_make_buffer_rsrc(obase, 0, orec > 0x7fffffffll ? 0x7fffffff : (int)orec, 0x00020000);
  // 16-byte stores need every quad whole and 16-byte aligned addresses
  const bool vec = (ohw & 3) == 0 && (reinterpret_cast<size_t>(out) & 15) == 0;
  const bool relu = g.act != 0 && g.csplit == 1;  // a slice's partial sums are stored as they are
  typedef float f4 __attribute__((ext_vector_type(4)));
  typedef unsigned u4 __attribute__((ext_vector_type(4)));
  for (int k = 0; k < g.g; ++k) {
    const int oc = __builtin_amdgcn_readlane(lane_oc, k);
    if (oc < 0) continue;  // padding slot
    const int soff = oc * ohw * 4;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      float v[4];
      read_accumulators4<VARIANT>((k * NQ + q) * 4, v);
      if (ooff[q] == kInvalid) continue;
      if (relu) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = fmaxf(v[j], 0.f);
      }
      if (vec) {
        const f4 d = {v[0], v[1], v[2], v[3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, d), orsrc, (int)ooff[q], soff, 0);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (j < npx[q])
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v[j]), orsrc, (int)ooff[q] + 4 * j, soff, 0);
      }
    }
  }
  if (!(g.fused && drew_last_ticket(tickets, tile_id, wave, g))) {
    TETRIS_STAMP_END();
    return;
  }
  // This wave adds the slices (see drew_last_ticket): the same quads and channels at the same offsets of every slice.
  const bool fvec = vec && (reinterpret_cast<size_t>(final_out) & 15) == 0;
  const __amdgpu_buffer_rsrc_t frsrc = __builtin_amdgcn_make_buffer_rsrc(
      final_out + (size_t)n_base * g.K * ohw, 0, orec > 0x7fffffffll ? 0x7fffffff : (int)orec, 0x00020000);
  const bool frelu = g.act != 0;
  for (int k = 0; k < g.g; ++k) {
    const int oc = __builtin_amdgcn_readlane(lane_oc, k);
    if (oc < 0) continue;
    const int soff = oc * ohw * 4;
    float sum[NQ][4];
    for (int s = 0; s < g.csplit; ++s) {
      const __amdgpu_buffer_rsrc_t prsrc = __builtin_amdgcn_make_buffer_rsrc(
          out + (size_t)s * out_elems + (size_t)n_base * g.K * ohw, 0, orec > 0x7fffffffll ? 0x7fffffff : (int)orec, 0x00020000);
#pragma unroll
      for (int q = 0; q < NQ; ++q) {
        float v[4];
        if (vec) {  // an offset out of range reads as zero
          const f4 d = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(prsrc, (int)ooff[q], soff, kBypassL1));
          v[0] = d.x; v[1] = d.y; v[2] = d.z; v[3] = d.w;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            v[j] = j < npx[q] ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                    prsrc, (int)ooff[q] + 4 * j, soff, kBypassL1)) : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) sum[q][j] = s == 0 ? v[j] : sum[q][j] + v[j];
      }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (ooff[q] == kInvalid) continue;
      if (frelu) {
#pragma unroll
        for (int j = 0; j < 4; ++j) sum[q][j] = fmaxf(sum[q][j], 0.f);
      }
      if (fvec) {
        const f4 d = {sum[q][0], sum[q][1], sum[q][2], sum[q][3]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, d), frsrc, (int)ooff[q], soff, 0);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (j < npx[q])
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, sum[q][j]), frsrc, (int)ooff[q] + 4 * j, soff, 0);
      }
    }
  }
  TETRIS_STAMP_END();
}

template <int NQ>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_num_vgpr(TETRIS_WALK6_FIRST_RESERVED_2))) void spconv2d_flat6(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  flat_body<NQ, 16, 6>(in, out, entries, grp_off, grp_pair, oc_order, final_out, tickets, g);
}

template <int NQ>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(TETRIS_WALK7_FIRST_RESERVED_4))) void spconv2d_flat7(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  flat_body<NQ, 8, 7>(in, out, entries, grp_off, grp_pair, oc_order, final_out, tickets, g);
}

template <int NQ>
__global__ __launch_bounds__(512) __attribute__((amdgpu_num_vgpr(TETRIS_WALK8_FIRST_RESERVED_2))) void spconv2d_flat8(
    const float* __restrict__ in, float* __restrict__ out, const int2* __restrict__ entries,
    const int32_t* __restrict__ grp_off, const int32_t* __restrict__ grp_pair,
    const int32_t* __restrict__ oc_order, float* __restrict__ final_out, int* __restrict__ tickets, const Geom g) {
  flat_body<NQ, 8, 8>(in, out, entries, grp_off, grp_pair, oc_order, final_out, tickets, g);
}

// Adds the `slices` partial outputs of a split reduction, in slice order (so the result does not depend on timing);
// relu: the sum goes through max(., 0) before it is written.
__global__ __launch_bounds__(256) void reduce_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                     long long n, int slices, int relu) {
  const long long step = (long long)gridDim.x * blockDim.x;
  const long long n4 = n >> 2;
  const float4* p4 = reinterpret_cast<const float4*>(partial);
  const bool vec = (n & 3) == 0 && (reinterpret_cast<size_t>(out) & 15) == 0;  // slices then start 16-byte aligned too
  if (vec) {
    for (long long k = (long long)blockIdx.x * blockDim.x + threadIdx.x; k < n4; k += step) {
      float4 a = p4[k];
      for (int s = 1; s < slices; ++s) {
        const float4 b = p4[(long long)s * n4 + k];
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
      }
      if (relu) { a.x = fmaxf(a.x, 0.f); a.y = fmaxf(a.y, 0.f); a.z = fmaxf(a.z, 0.f); a.w = fmaxf(a.w, 0.f); }
      reinterpret_cast<float4*>(out)[k] = a;
    }
  } else {
    for (long long k = (long long)blockIdx.x * blockDim.x + threadIdx.x; k < n; k += step) {
      float a = partial[k];
      for (int s = 1; s < slices; ++s) a += partial[(long long)s * n + k];
      out[k] = relu ? fmaxf(a, 0.f) : a;
    }
  }
}

// The same followed by ReLU and 2x2 max-pooling: out[p][y][x] = max(0, sums of [p][2y..2y+1][2x..2x+1]) over `planes`
// planes of OH x OW sums per slice (an odd last row or column is dropped).  vec: OW is a multiple of four and the
// pointers are 16-byte aligned, a thread then makes two neighbouring outputs from two 16-byte loads per slice.
__global__ __launch_bounds__(256) void reduce_pool_kernel(const float* __restrict__ partial, float* __restrict__ out,
                                                          long long planes, int OH, int OW, int slices, int vec) {
  const int ph = OH >> 1, pw = OW >> 1;
  const long long n = planes * OH * OW;  // floats per slice
  const long long step = (long long)gridDim.x * blockDim.x;
  const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (vec) {
    const int pairs = pw >> 1;
    const long long total = planes * ph * pairs;
    for (long long i = t; i < total; i += step) {
      const long long row = i / pairs;  // plane * ph + y
      const int xp = (int)(i - row * pairs);
      const long long p = row / ph;
      const int y = (int)(row - p * ph);
      const float* src = partial + (p * OH + 2 * y) * OW + 4 * xp;
      float4 a = *reinterpret_cast<const float4*>(src);
      float4 b = *reinterpret_cast<const float4*>(src + OW);
      for (int s = 1; s < slices; ++s) {
        const float4 c = *reinterpret_cast<const float4*>(src + s * n);
        const float4 d = *reinterpret_cast<const float4*>(src + s * n + OW);
        a.x += c.x; a.y += c.y; a.z += c.z; a.w += c.w;
        b.x += d.x; b.y += d.y; b.z += d.z; b.w += d.w;
      }
      float2 r;
      r.x = fmaxf(fmaxf(fmaxf(a.x, a.y), fmaxf(b.x, b.y)), 0.f);
      r.y = fmaxf(fmaxf(fmaxf(a.z, a.w), fmaxf(b.z, b.w)), 0.f);
      *reinterpret_cast<float2*>(out + row * pw + 2 * xp) = r;
    }
  } else {
    const long long total = planes * ph * pw;
    for (long long i = t; i < total; i += step) {
      const long long row = i / pw;
      const int x = (int)(i - row * pw);
      const long long p = row / ph;
      const int y = (int)(row - p * ph);
      const float* src = partial + (p * OH + 2 * y) * OW + 2 * x;
      float a = src[0], b = src[1], c = src[OW], d = src[OW + 1];
      for (int s = 1; s < slices; ++s) {
        const float* q = src + s * n;
        a += q[0]; b += q[1]; c += q[OW]; d += q[OW + 1];
      }
      out[i] = fmaxf(fmaxf(fmaxf(a, b), fmaxf(c, d)), 0.f);
    }
  }
}

// Workgroup ids go round-robin to the eight XCDs and the kernels turn them into logical ids that are contiguous per
// XCD (logical = (id % 8) * grid / 8 + id / 8); the slices of an output tile are `csplit` consecutive logical ids.
// Every XCD's range holds a whole number of tiles, so the slices of a tile always share an XCD.
int grid_size(const Geom& g) {
  const int tiles = g.ugroups * g.kblocks;
  return 8 * ((tiles + 7) / 8) * g.csplit;
}

template <int NQ, int WAVES, int VARIANT>
int launch_three(const Geom& g, const float* d_in, float* d_out, const int2* entries, const int32_t* grp_off,
                 const int32_t* grp_pair, const int32_t* oc_order, float* d_final, int* d_tickets, hipStream_t stream) {
  void (*kern)(const float*, float*, const int2*, const int32_t*, const int32_t*, const int32_t*, float*, int*, const Geom);
  constexpr int LDS = VARIANT == 5 ? kBufs * kHalfBufBytes : VARIANT == 8 ? 2 * kFlatHalfBufBytes
                      : VARIANT >= 6 ? 2 * kFlatBufBytes : kBufs * kBufBytes;
  if constexpr (VARIANT == 4) kern = spconv2d_kernel4<NQ>;
  else if constexpr (VARIANT == 5) kern = spconv2d_kernel5<NQ>;
  else if constexpr (VARIANT == 6) kern = spconv2d_flat6<NQ>;
  else if constexpr (VARIANT == 7) kern = spconv2d_flat7<NQ>;
  else if constexpr (VARIANT == 8) kern = spconv2d_flat8<NQ>;
  else kern = spconv2d_kernel3<NQ>;
  static std::atomic<bool> lds_set{false};  // per instantiation; setting the attribute twice is harmless
  if (!lds_set.load(std::memory_order_acquire)) {
    TETRIS_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
    lds_set.store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(grid_size(g)), dim3(WAVES * 64), LDS, stream, d_in, d_out, entries, grp_off, grp_pair,
                     oc_order, d_final, d_tickets, g);
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}

template <int NQ, int SPT>
int launch_one(const Geom& g, const float* d_in, float* d_out, const int2* entries, const int32_t* grp_off,
               const int32_t* grp_pair, const int32_t* oc_order, float* d_final, int* d_tickets, hipStream_t stream) {
  auto kern = spconv2d_kernel<NQ, SPT>;
  static std::atomic<bool> lds_set{false};  // per instantiation; setting the attribute twice is harmless
  if (!lds_set.load(std::memory_order_acquire)) {
    TETRIS_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   kTileBytes));
    lds_set.store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(grid_size(g)), dim3(g.waves * 64), kTileBytes, stream, d_in, d_out, entries, grp_off,
                     grp_pair, oc_order, d_final, d_tickets, g);
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}

}  // namespace

static int launch_kernel(const Geom& g, const float* d_in, float* d_out, const int2* entries, const int32_t* grp_off,
                         const int32_t* grp_pair, const int32_t* oc_order, float* d_final, int* d_tickets,
                         hipStream_t stream) {
  if (g.ver == 4) {  // flat tiles of pointwise layers
    if ((g.waves != 8 && g.waves != 16) || g.g * 4 * g.nq > (g.waves == 16 ? 64 : 128) || g.ks != 1 || g.stride != 1 ||
        g.pad != 0 || g.step < 1 || g.OH != g.H || g.OW != g.W || g.plane != 256 || g.region * g.nq != g.buf_bytes || 1024 * g.tile_ic > g.region ||
        (g.buf_bytes != kFlatBufBytes && (g.buf_bytes != kFlatHalfBufBytes || g.waves != 8 || g.g * 4 * g.nq > 64 || g.nq > 2)) ||
        g.qi != (g.H * g.W + 3) / 4 || (g.step == 1 && g.in_hw != g.H * g.W) || (long long)g.quads_total != (long long)g.N * g.qi || g.stagers < 1 ||
        g.stagers > g.waves || g.ugroups * g.nq * 64ll < g.quads_total)
      return fail(TETRIS_EINVAL, "inconsistent kernel geometry (flat kernel)");
    if (g.waves == 16) {
      if (g.nq == 1) return launch_three<1, 16, 6>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 2) return launch_three<2, 16, 6>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
    } else if (g.buf_bytes == kFlatHalfBufBytes) {
      if (g.nq == 1) return launch_three<1, 8, 8>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 2) return launch_three<2, 8, 8>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
    } else {
      if (g.nq == 1) return launch_three<1, 8, 7>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 2) return launch_three<2, 8, 7>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 4) return launch_three<4, 8, 7>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
    }
    return fail(TETRIS_EINVAL, "no flat kernel for quads=%d waves=%d", g.nq, g.waves);
  }
  if (g.ver == 3) {
    if ((g.waves != 8 && g.waves != 16) || g.g * 4 * g.nq > (g.waves == 16 ? 64 : 128) ||
        (g.buf_bytes != kBufBytes && (g.buf_bytes != kHalfBufBytes || g.waves != 8 || g.g * 4 * g.nq > 64 || g.nq > 2)) ||
        g.region * g.nq != g.buf_bytes || g.cpp * 64 < g.plane || g.nchunks != g.nq * g.nb * g.cpp ||
        g.stagers < 4 || g.stagers > g.waves || g.ni * g.stagers < g.nchunks || g.ni > (g.waves == 16 || g.buf_bytes == kHalfBufBytes ? kMaxChunks16 : kMaxChunks))
      return fail(TETRIS_EINVAL, "inconsistent kernel geometry (triple-buffered kernel)");
    if (g.waves == 16) {
      if (g.nq == 1) return launch_three<1, 16, 4>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 2) return launch_three<2, 16, 4>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
    } else if (g.buf_bytes == kHalfBufBytes) {
      if (g.nq == 1) return launch_three<1, 8, 5>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 2) return launch_three<2, 8, 5>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
    } else {
      if (g.nq == 1) return launch_three<1, 8, 3>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 2) return launch_three<2, 8, 3>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
      if (g.nq == 4) return launch_three<4, 8, 3>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
    }
    return fail(TETRIS_EINVAL, "no kernel for quads=%d waves=%d", g.nq, g.waves);
  }
  if (g.region * g.nq != kTileBytes || g.spt * g.fill_iters > kFillItems || g.fill_slots > g.spt * g.waves * 64)
    return fail(TETRIS_EINVAL, "inconsistent kernel geometry");
#define TETRIS_CASE(NQ, SPT) \
  if (g.nq == NQ && g.spt == SPT) return launch_one<NQ, SPT>(g, d_in, d_out, entries, grp_off, grp_pair, oc_order, d_final, d_tickets, stream);
  TETRIS_CASE(1, 1)
  TETRIS_CASE(1, 2)
  TETRIS_CASE(2, 1)
  TETRIS_CASE(2, 2)
  TETRIS_CASE(4, 1)
  TETRIS_CASE(4, 2)
#undef TETRIS_CASE
  return fail(TETRIS_EINVAL, "no kernel for quads=%d slots-per-thread=%d", g.nq, g.spt);
}

// The halo'd kernels walk streams arranged as pairs + singles when a wave holds enough channels for pairs to be
// common; the flat kernels' waves hold few channels and walk the pack's own arrangement.
bool geom_walks_pairs(const Geom& g) { return (options() & TETRIS_OPT_PAIRS) && g.ver != 4 && g.g >= 4; }

// whether the kernel of geometry `g` can pool its own outputs (store_pooled's conditions)
bool geom_pools_in_kernel(const Geom& g) {
  return g.ver != 4 && g.csplit == 1 && (g.thi & 1) == 0 && ((g.lw & 1) == 0 || g.jsh == 0);
}

// ---- which XCD a workgroup runs on ---------------------------------------------------------------------------------
namespace {
__global__ void xcc_probe_kernel(int* __restrict__ out) {
  // XCC_ID hardware register (id 20), all 32 bits; its low four bits number the XCD this wave runs on
  const int id = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (31 << 11)) & 0xf;
  if (threadIdx.x == 0) out[blockIdx.x] = id;
}
}  // namespace

int same_xcd_by_residue(bool* ok) {
  constexpr int kMaxDev = 64, kBlocks = 1024;
  static std::mutex mu;
  static signed char known[kMaxDev];  // 0 not asked, 1 yes, 2 no
  int dev = 0;
  TETRIS_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDev) return fail(TETRIS_EINVAL, "device %d out of range", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!known[dev]) {
    // more workgroups than the GPU runs at once, twice: every residue of blockIdx.x % 8 must report one XCD throughout
    int* d = nullptr;
    TETRIS_HIP(hipMalloc(&d, sizeof(int) * kBlocks));
    std::vector<int> h(kBlocks);
    bool same = true;
    int first[8];
    for (int round = 0; round < 2 && same; ++round) {
      hipLaunchKernelGGL(xcc_probe_kernel, dim3(kBlocks), dim3(round ? 1024 : 64), 0, 0, d);
      hipError_t e = hipMemcpy(h.data(), d, sizeof(int) * kBlocks, hipMemcpyDeviceToHost);
      if (e != hipSuccess) {
        (void)hipFree(d);
        return fail(TETRIS_EHIP, "XCD probe failed: %s", hipGetErrorString(e));
      }
      for (int i = 0; i < kBlocks; ++i) {
        if (round == 0 && i < 8) first[i] = h[i];
        same = same && h[i] == first[i & 7];
      }
    }
    (void)hipFree(d);
    known[dev] = same ? 1 : 2;
  }
  *ok = known[dev] == 1;
  return TETRIS_OK;
}

int launch_conv(const Geom& g0, const float* d_in, float* d_user_out, float* d_scratch, const int2* entries,
                const int32_t* grp_off, const int32_t* grp_pair, const int32_t* oc_order, int act, hipStream_t stream) {
  // what the kernel's indexing assumes, checked once more before anything is launched
  if (g0.g * 4 * g0.nq > kAccRegs || g0.nb * g0.img_stride * 4 > g0.region || g0.lr * g0.lh > 64 || g0.lw > g0.lr ||
      g0.kblocks * g0.kb > g0.slots || g0.waves < 1 || g0.waves > 16 || g0.csplit < 1 || g0.csplit > kMaxSplit ||
      (g0.csplit > 1 && (g0.stages < 2 * g0.csplit || !d_scratch)) || g0.heads_off < kBatch)
    return fail(TETRIS_EINVAL, "inconsistent kernel geometry");
  if (act < 0 || act > 2) return fail(TETRIS_EINVAL, "unknown activation %d", act);
  if (act == 2 && (g0.OH < 2 || g0.OW < 2)) return fail(TETRIS_EINVAL, "2x2 pooling needs an output of at least 2 x 2");
  if (act == 2 && g0.csplit == 1 && !geom_pools_in_kernel(g0))
    return fail(TETRIS_EUNSUPPORTED, "this tile cannot pool its outputs (lanes_w %d, %d rows per unit): launch with ReLU "
                "and pool with tetris_relu_maxpool", g0.lw, g0.thi);
  Geom g = g0;
  g.fused = 0;
  if (g.csplit == 1) {
    g.act = act;
    return launch_kernel(g, d_in, d_user_out, entries, grp_off, grp_pair, oc_order, nullptr, nullptr, stream);
  }
  // A split layer.  Its scratch: the tickets, then one copy of the output per slice.
  int* d_tickets = reinterpret_cast<int*>(d_scratch);
  float* d_partial = d_scratch + kTicketBytes / sizeof(float);
  if (act != 2 && (options() & TETRIS_OPT_ADD_IN_KERNEL) &&
      (long long)g.ugroups * g.kblocks * g.waves <= kMaxTickets) {
    bool ok = false;
    const int rc = same_xcd_by_residue(&ok);  // asked once per device (the first time from tetris_g950_prepare or an
    if (rc) return rc;                        // eager launch, never under capture: planning a split layer allocates)
    g.fused = ok ? 1 : 0;
  }
  g.act = g.fused ? act : 0;  // otherwise the sums are finished by the adding kernel
  const int rc = launch_kernel(g, d_in, d_partial, entries, grp_off, grp_pair, oc_order, d_user_out, d_tickets, stream);
  if (rc != TETRIS_OK || g.fused) return rc;
  const long long n = (long long)g.N * g.K * g.OH * g.OW;
  if (act == 2) {
    const int vec = (g.OW & 3) == 0 && (reinterpret_cast<size_t>(d_user_out) & 15) == 0;
    const long long items = (long long)g.N * g.K * (g.OH / 2) * (vec ? g.OW / 4 : g.OW / 2);
    const int blocks = (int)std::min<long long>((items + 255) / 256, 2048);
    hipLaunchKernelGGL(reduce_pool_kernel, dim3(blocks), dim3(256), 0, stream, d_partial, d_user_out,
                       (long long)g.N * g.K, g.OH, g.OW, g.csplit, vec);
  } else {
    const int blocks = (int)std::min<long long>(((n + 3) / 4 + 255) / 256, 2048);
    hipLaunchKernelGGL(reduce_kernel, dim3(blocks), dim3(256), 0, stream, d_partial, d_user_out, n, g.csplit, act);
  }
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}

}  // namespace tetris

#ifdef TETRIS_STAMPS
// Copies the stamps of the first `n_wg` workgroups of the last launches (16 values each, see TETRIS_STAMP) to the
// host and clears them.  Only in the library `make stamps` builds.
extern "C" int tetris_stamps_read(long long* out, int n_wg) {
  using namespace tetris;
  if (!out || n_wg < 1 || n_wg > kStampWgs) return fail(TETRIS_EINVAL, "bad argument");
  TETRIS_HIP(hipDeviceSynchronize());
  TETRIS_HIP(hipMemcpyFromSymbol(out, HIP_SYMBOL(g_stamps), sizeof(long long) * kStampSlots * (size_t)n_wg));
  std::vector<long long> zero((size_t)kStampSlots * n_wg, 0);
  TETRIS_HIP(hipMemcpyToSymbol(HIP_SYMBOL(g_stamps), zero.data(), sizeof(long long) * zero.size()));
  return TETRIS_OK;
}
#endif
