// Tile-shape selection for the gfx950 conv kernel: turns a layer shape plus a tetris_tile into the
// kernel geometry, and picks a tetris_tile when the caller leaves it to the library.
//
// Takes the place of the reference's exhaustive search over 185 compiled {KS, STRIDE, TILE_IC, TILE_H,
// TILE_W} instantiations (Tetris/spconv2d.cc:90-329, 130 launches and one re-pack per candidate).
#include <algorithm>
#include <atomic>
#include <climits>
#include <cstdlib>
#include <cmath>
#include <cstdio>
#include <mutex>
#include <utility>

#include "common.h"

namespace tetris {

namespace {
std::atomic<unsigned> g_options{~0u};  // ~0: not set yet
}

unsigned options() {
  unsigned v = g_options.load();
  if (v == ~0u) {
    const char* e = std::getenv("TETRIS_OPTIONS");
    v = e ? (unsigned)std::strtoul(e, nullptr, 0) & 0xffffu : 0u;
    g_options.store(v);
  }
  return v;
}
void set_options(unsigned flags) { g_options.store(flags & 0xffffu); }

// Compute units of the current device (256 on MI355X), asked once; 256 when no device can be asked (packing and
// tile selection also run on machines without a GPU).
int cu_count() {
  static std::atomic<int> cached{0};
  int v = cached.load();
  if (v == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached.store(v = n);
  }
  return v;
}

namespace {

struct Shape {
  int lw, lr, lh, thi, nb, ng, par, pitch, ih;
};

// Period (in dwords) of the bank rule for `lr` lane positions per row: 64, except that rows of 1, 2 or 4
// lanes repeat every 8 * lr dwords (measured with 16-byte reads on MI355X).
inline int bank_period(int lr) { return (lr == 1 || lr == 2 || lr == 4) ? 8 * lr : 64; }

// Lane rows and LDS pitch for `lw` active lanes per row.  The LDS distance between consecutive lane rows,
// stride * pitch dwords, must equal 4 * lr modulo the bank period for full-rate 16-byte reads; among the
// (lr, pitch) pairs that satisfy it, take the one that wastes the least: idle lane positions cost compute
// time one for one, a padded pitch only costs LDS room.
Shape unit_shape(int lw, int OH, int N, int ks, int stride) {
  Shape s;
  s.lw = lw;
  s.ng = lw + (ks - 1) / stride;
  s.par = 4 * s.ng;
  const int min_pitch = stride * s.par;
  double best = 1e300;
  s.lr = lw;
  s.pitch = min_pitch;
  const bool rule = !(options() & TETRIS_OPT_NO_BANK_RULE);
  for (int lr = lw; lr <= 64 && lr <= lw + 16; ++lr)
    for (int pitch = min_pitch; pitch <= min_pitch + 64; pitch += 4) {
      if (rule && (stride * pitch - 4 * lr) % bank_period(lr) != 0) continue;
      const int lh = 64 / lr;
      const int thi = std::min(lh, OH);
      const int rows = std::max(1, std::min(lh / thi, N)) * thi;  // lane rows that can hold pixels
      const double cost = (64.0 / (rows * lw)) * (1.0 + 0.25 * ((double)pitch / min_pitch - 1.0));
      if (cost < best - 1e-9) {
        best = cost;
        s.lr = lr;
        s.pitch = pitch;
      }
      break;  // larger pitches with this lr only cost more
    }
  s.lh = 64 / s.lr;
  s.thi = std::min(s.lh, OH);
  s.nb = std::max(1, std::min(s.lh / s.thi, N));
  s.ih = stride * (s.thi - 1) + ks;
  return s;
}

// Dwords per image of a unit's region: at least tile_ic planes, padded so that the step from the last lane
// row of one image to the first of the next also meets the bank rule.
int image_stride(const Shape& s, int tile_ic, int stride) {
  int v = tile_ic * s.ih * s.pitch;
  if (s.nb > 1 && !(options() & TETRIS_OPT_NO_BANK_RULE))
    while ((v - (s.thi - 1) * stride * s.pitch - 4 * s.lr) % bank_period(s.lr) != 0) v += 4;
  return v;
}

}  // namespace

// How many workgroups share an output tile.  The tile may say (1 = none, up to kMaxSplit, every slice at least two
// stages); 0 leaves it to the rule: small feature maps leave most of the CUs without a workgroup, so double the
// slices while fewer than half of the wave slots (`room`) would be used and every slice keeps at least four stages.
static int choose_csplit(const tetris_tile& t, long long waves_total, long long room, int stages, int* out) {
  if (t.csplit < 0 || t.csplit > kMaxSplit) return fail(TETRIS_EINVAL, "bad tile: csplit=%d (0..%d)", t.csplit, kMaxSplit);
  if (t.csplit > 1 && stages < 2 * t.csplit)
    return fail(TETRIS_EINVAL, "bad tile: %d slices of %d stages (every slice needs at least two)", t.csplit, stages);
  int cs = 1;
  if (t.csplit > 0) cs = t.csplit;
  else while (cs < kMaxSplit && waves_total * cs * 2 <= room && stages >= 8 * cs) cs *= 2;
  *out = cs;
  return TETRIS_OK;
}

// Geometry of a flat tile (lanes_w == 64) for a pointwise layer; `g` holds the layer and the tile's quads, slots and waves.
static int make_flat_geom(const tetris_g950* p, Geom g, const tetris_tile& t, Geom* out) {
  if (p->ks != 1 || g.stride != 1 || g.pad != 0 || g.step < 1)  // a strided layer arrives as stride 1 on its sub-grid
    return fail(TETRIS_EINVAL, "flat tiles (lanes_w = %d) are for 1x1 layers without padding", kFlatLanes);
  if (t.waves != 8 && t.waves != 16) return fail(TETRIS_EINVAL, "bad tile: flat tiles take 8 or 16 waves (got %d)", t.waves);
  if (g.nq != 1 && g.nq != 2 && g.nq != 4) return fail(TETRIS_EINVAL, "bad tile: quads=%d", g.nq);
  if (t.oc_per_wave != p->g)
    return fail(TETRIS_EINVAL, "tile wants %d output channels per wave, the pack was made for %d", t.oc_per_wave, p->g);
  const int acc_regs = t.waves == 16 ? kAccRegs / 2 : kAccRegs;
  if (g.g * 4 * g.nq > acc_regs || (t.waves == 16 && g.nq > 2))
    return fail(TETRIS_EINVAL, "oc_per_wave * 4 * quads = %d exceeds the %d accumulators of a wave", g.g * 4 * g.nq, acc_regs);
  g.ver = 4;
  const long long hw = (long long)g.H * g.W;
  g.qi = (int)((hw + 3) / 4);
  const long long quads = (long long)g.N * g.qi;
  if (quads * g.qi >= (1ll << 32) || quads >= (1ll << 30))
    return fail(TETRIS_EINVAL, "too many pixels for the kernel's index arithmetic");
  g.quads_total = (int)quads;
  g.m_qi = magic_reciprocal(g.qi);
  if (hw * g.W >= (1ll << 32)) return fail(TETRIS_EINVAL, "too many pixels for the kernel's index arithmetic");
  g.m_ow = magic_reciprocal(g.W);
  g.buf_bytes = (t.waves == 8 && g.g * 4 * g.nq <= kAccRegs / 2 && g.nq <= 2) ? kFlatHalfBufBytes : kFlatBufBytes;
  g.region = g.buf_bytes / g.nq;
  g.plane = 256; g.pitch = 0; g.par = 0; g.lw = g.lr = 64; g.lh = 1; g.thi = 1; g.nb = 1; g.ng = 64; g.ih = 1;
  g.img_stride = g.tile_ic * g.plane;
  g.fold = 1; g.jsh = 2;
  if (4ll * g.img_stride > g.region)
    return fail(TETRIS_EINVAL, "a pixel unit needs %lld bytes of LDS for %d staged channels (region is %d): lower tile_ic "
                "or quads", 4ll * g.img_stride, g.tile_ic, g.region);
  g.units = (int)((quads + 63) / 64);
  g.units_w = g.units; g.units_h = 1; g.units_n = 1;
  g.ugroups = ceil_div(g.units, g.nq);
  g.kb = t.waves * g.g;
  g.kblocks = ceil_div(p->K, g.kb);
  if (g.kblocks * g.kb > p->slots) return fail(TETRIS_EINVAL, "channel block %d does not divide the slot padding", g.kb);
  if ((long long)g.ugroups * g.kblocks > (1ll << 28)) return fail(TETRIS_EINVAL, "grid too large");
  // a workgroup reaches its images through one 2 GB window on the input and one on the output
  const long long span = (64ll * g.nq + g.qi - 1) / g.qi + 2;  // images a workgroup's quads can touch, and a spare
  if (4ll * std::max((long long)g.in_hw * p->C, hw * p->K) * span >= (1ll << 31))
    return fail(TETRIS_EINVAL, "images too large for the 2 GB window of a workgroup");
  if ((long long)g.N * p->K * hw >= (1ll << 40)) return fail(TETRIS_EINVAL, "output too large");
  const bool four = t.waves == 16 || g.buf_bytes == kFlatHalfBufBytes;
  const long long room = (long long)cu_count() * (four ? 16 : 8);
  const long long waves_total = (long long)g.ugroups * g.kblocks * t.waves;
  if (int rc = choose_csplit(t, waves_total, room, g.stages, &g.csplit)) return rc;
  if ((long long)g.ugroups * g.kblocks * g.csplit * g.kblocks * g.csplit >= (1ll << 32) ||
      (long long)g.stages * (g.csplit + 1) * g.csplit >= (1ll << 32))
    return fail(TETRIS_EINVAL, "grid too large");
  if (g.csplit > 1 && 4ll * g.csplit * g.N * p->K * hw > (1ll << 30))
    return fail(TETRIS_EINVAL, "%d slices of this layer's output are more than 1 GiB of partial sums", g.csplit);
  g.m_kblocks = magic_reciprocal(g.kblocks);
  g.m_csplit = magic_reciprocal(g.csplit);
  // Every load a wave issues waits its turn at the CU's address unit, and a wave that issues does not walk.  In a
  // 16-wave workgroup the eight oldest waves (two per SIMD, served first) stage for all: the other eight walk meanwhile
  // (MobileNet pass -1.9 %, ResNet-50 -1.0 % against all sixteen staging; four stagers: +4 % and 0 %).
  g.stagers = t.waves == 16 ? 8 : t.waves;
  g.spt = 1; g.cg = 1; g.fill_iters = 1;
  *out = g;
  return TETRIS_OK;
}

int make_geom(const tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile& t, Geom* out) {
  Geom g{};
  if (N <= 0 || H <= 0 || W <= 0 || stride <= 0 || pad < 0)
    return fail(TETRIS_EINVAL, "bad conv shape N=%d H=%d W=%d stride=%d pad=%d", N, H, W, stride, pad);
  g.step = 1; g.in_w = W; g.in_hw = H * W;
  if (p->ks == 1 && stride > 1 && pad == 0) {  // only every stride-th row and column is read: stage just those
    g.step = stride;
    H = (H - 1) / stride + 1;
    W = (W - 1) / stride + 1;
    stride = 1;
  }
  g.N = N; g.C = p->C; g.H = H; g.W = W; g.K = p->K; g.ks = p->ks; g.stride = stride; g.pad = pad;
  g.OH = out_extent(H, pad, p->ks, stride);
  g.OW = out_extent(W, pad, p->ks, stride);
  if (H + 2 * pad < p->ks || W + 2 * pad < p->ks || g.OH <= 0 || g.OW <= 0)
    return fail(TETRIS_EINVAL, "kernel %d does not fit the padded %dx%d image", p->ks, H, W);
  g.tile_ic = p->tile_ic;
  g.stages = p->stages;
  g.slots = p->slots;

  g.nq = t.quads;
  g.g = p->g;
  g.waves = t.waves;
  if (t.lanes_w == kFlatLanes) return make_flat_geom(p, g, t, out);
  if (t.lanes_w < 1 || t.lanes_w > 64 || (g.nq != 1 && g.nq != 2 && g.nq != 4))
    return fail(TETRIS_EINVAL, "bad tile: lanes_w=%d quads=%d", t.lanes_w, g.nq);
  if (t.oc_per_wave != p->g)
    return fail(TETRIS_EINVAL, "tile wants %d output channels per wave, the pack was made for %d", t.oc_per_wave, p->g);
  if (t.waves != 1 && t.waves != 2 && t.waves != 4 && t.waves != 8 && t.waves != 16)
    return fail(TETRIS_EINVAL, "bad tile: waves=%d (1, 2, 4, 8 or 16)", t.waves);
  const int acc_regs = t.waves == 16 ? kAccRegs / 2 : kAccRegs;  // 16-wave workgroups run four waves per SIMD
  if (g.g * 4 * g.nq > acc_regs)
    return fail(TETRIS_EINVAL, "oc_per_wave * 4 * quads = %d exceeds the %d accumulators of a wave", g.g * 4 * g.nq,
                acc_regs);
  g.fold = fold_of(t.lanes_w, g.OW);
  g.jsh = g.fold == 4 ? 0 : g.fold == 2 ? 1 : 2;
  const Shape s = unit_shape(t.lanes_w, g.OH, ceil_div(N, g.fold), p->ks, stride);
  g.lw = s.lw; g.lr = s.lr; g.lh = s.lh; g.thi = s.thi; g.nb = s.nb; g.ng = s.ng; g.par = s.par; g.ih = s.ih;
  g.ver = t.waves >= 8 ? 3 : 2;
  // 8 waves that need at most 64 accumulators each leave room for a second workgroup on the CU
  g.buf_bytes = (t.waves == 8 && g.g * 4 * g.nq <= kAccRegs / 2 && g.nq <= 2) ? kHalfBufBytes : kBufBytes;
  g.region = (g.ver == 3 ? g.buf_bytes : kTileBytes) / g.nq;
  g.pitch = s.pitch;
  g.plane = g.ih * g.pitch;
  g.img_stride = image_stride(s, g.tile_ic, stride);
  if (4ll * g.nb * g.img_stride > g.region)
    return fail(TETRIS_EINVAL, "a pixel unit needs %lld bytes of LDS for %d staged channels (region is %d): lower tile_ic "
                "or quads", 4ll * g.nb * g.img_stride, g.tile_ic, g.region);
  g.units_w = ceil_div(g.OW, (4 / g.fold) * g.lw);
  g.units_h = ceil_div(g.OH, g.thi);
  g.units_n = ceil_div(N, g.nb * g.fold);
  const long long units = (long long)g.units_w * g.units_h * g.units_n;
  g.kb = t.waves * g.g;
  g.kblocks = ceil_div(p->K, g.kb);
  if (g.kblocks * g.kb > p->slots) return fail(TETRIS_EINVAL, "channel block %d does not divide the slot padding", g.kb);
  if (units * g.kblocks > (1ll << 30)) return fail(TETRIS_EINVAL, "grid too large");
  g.units = (int)units;
  g.ugroups = ceil_div(g.units, g.nq);
  // a workgroup addresses its images through one 2 GB buffer window
  const long long img_bytes = 4ll * p->C * g.in_hw;
  if (img_bytes * ((long long)g.nq * g.nb * g.fold + 2) >= (1ll << 31))
    return fail(TETRIS_EINVAL, "images too large for the 2 GB input window of a workgroup");
  if ((long long)N * p->K * g.OH * g.OW >= (1ll << 40)) return fail(TETRIS_EINVAL, "output too large");
  // ... and writes its outputs through one as well
  if (4ll * p->K * g.OH * g.OW * ((long long)g.nq * g.nb * g.fold + 2) >= (1ll << 31))
    return fail(TETRIS_EINVAL, "images too large for the 2 GB output window of a workgroup");
  // staging plan
  g.slots_per_unit = g.nb * g.ih * stride * g.ng;
  g.fill_slots = g.nq * g.slots_per_unit;
  const int threads = t.waves * 64;
  {
    // the kernels divide by these with a multiply-high, exact while dividend * divisor < 2^32
    const long long upi = (long long)g.units_w * g.units_h;
    if (units * upi >= (1ll << 32)) return fail(TETRIS_EINVAL, "too many pixel units for the kernel's index arithmetic");
    g.m_upi = magic_reciprocal((int)upi);
    g.m_units_w = magic_reciprocal(g.units_w);
    g.m_lr = magic_reciprocal(g.lr);
    g.m_thi = magic_reciprocal(g.thi);
    // Small feature maps leave most of the 256 CUs without a workgroup: then several workgroups share an output
    // tile, each reducing a slice of the input-channel stages (at least four stages each, at most eight slices).
    const bool four = t.waves == 16 || g.buf_bytes == kHalfBufBytes;  // waves per SIMD the kernel variant allows
    const long long room = (long long)cu_count() * (g.ver == 3 && four ? 16 : 8);
    const long long waves_total = (long long)g.ugroups * g.kblocks * t.waves;
    if (int rc = choose_csplit(t, waves_total, room, g.stages, &g.csplit)) return rc;
    if ((long long)g.ugroups * g.kblocks * g.csplit * g.kblocks * g.csplit >= (1ll << 32) ||
        (long long)g.stages * (g.csplit + 1) * g.csplit >= (1ll << 32))
      return fail(TETRIS_EINVAL, "grid too large");
    if (g.csplit > 1 && 4ll * g.csplit * N * p->K * g.OH * g.OW > (1ll << 30))
      return fail(TETRIS_EINVAL, "%d slices of this layer's output are more than 1 GiB of partial sums", g.csplit);
    g.m_kblocks = magic_reciprocal(g.kblocks);
    g.m_csplit = magic_reciprocal(g.csplit);
  }
  if (g.ver == 3) {
    g.cpp = ceil_div(g.plane, 64);
    g.nchunks = g.nq * g.nb * g.cpp;
    // a workgroup of 8 or 16 waves leaves the staging to its four oldest waves when they can hold the plan (the
    // hardware serves the oldest wave of a SIMD first: they finish their walk early and would idle at the barrier)
    g.stagers = t.waves;
    const int max_chunks = (t.waves == 16 || g.buf_bytes == kHalfBufBytes) ? kMaxChunks16 : kMaxChunks;
    if (t.waves == 16) g.stagers = g.nchunks <= 4 * max_chunks ? 4 : g.nchunks <= 8 * max_chunks ? 8 : 16;
    if (t.waves == 8 && g.nchunks <= 4 * max_chunks) g.stagers = 4;
    g.ni = ceil_div(g.nchunks, g.stagers);
    if (64ll * (g.cpp + 1) * g.pitch >= (1ll << 32))
      return fail(TETRIS_EINVAL, "too many pixel units for the kernel's index arithmetic");
    g.m_per_unit = magic_reciprocal(g.nb * g.cpp);
    g.m_cpp = magic_reciprocal(g.cpp);
    g.m_pitch = magic_reciprocal(g.pitch);
    g.m_par = magic_reciprocal(g.par);
    g.spt = 1; g.cg = 1; g.fill_iters = 1;
    if (g.ni > max_chunks)
      return fail(TETRIS_EINVAL, "a staged channel takes %d LDS chunks per wave (limit %d): use fewer quads or a narrower "
                  "tile", g.ni, max_chunks);
    *out = g;
    return TETRIS_OK;
  }
  g.m_fill_slots = magic_reciprocal(g.fill_slots);
  g.m_slots_per_unit = magic_reciprocal(g.slots_per_unit);
  g.m_per_img = magic_reciprocal(g.ih * stride * g.ng);
  g.m_per_row = magic_reciprocal(stride * g.ng);
  g.m_ng = magic_reciprocal(g.ng);
  if (g.fill_slots <= threads) {
    g.spt = 1;
    g.cg = std::min(threads / g.fill_slots, g.tile_ic);
  } else {
    g.spt = 2;
    g.cg = 1;
    if (g.fill_slots > 2 * threads)
      return fail(TETRIS_EINVAL, "%d LDS slots per stage are more than %d threads can stage: use more waves or fewer "
                  "quads", g.fill_slots, threads);
  }
  g.fill_iters = ceil_div(g.tile_ic, g.cg);
  if (g.spt * g.fill_iters > kFillItems)
    return fail(TETRIS_EINVAL, "staging %d channels takes %d loads per thread (limit %d): lower tile_ic or use more "
                "waves", g.tile_ic, g.spt * g.fill_iters, kFillItems);
  *out = g;
  return TETRIS_OK;
}

// Largest tile_ic (a power of two, or C itself when smaller) that a tile shape can stage.
static int max_tile_ic(const Shape& s, int nq, int g, int waves, int stride, int C) {
  const bool v3 = waves >= 8;
  const bool half = waves == 8 && g * 4 * nq <= kAccRegs / 2 && nq <= 2;
  const int region = (v3 ? (half ? kHalfBufBytes : kBufBytes) : kTileBytes) / nq;
  const int threads = waves * 64;
  const int fill_slots = nq * s.nb * s.ih * stride * s.ng;
  if (v3) {
    if (ceil_div(nq * s.nb * ceil_div(s.ih * s.pitch, 64), waves) > (waves == 16 || half ? kMaxChunks16 : kMaxChunks)) return 0;
  } else if (fill_slots > 2 * threads) {
    return 0;
  }
  int best = 0;
  for (int t = 1; t <= 256; t *= 2) {
    const int tic = std::min(t, C);
    if (4ll * s.nb * image_stride(s, tic, stride) > region) break;
    int spt = 1, cg = tic;
    if (!v3) {
      if (fill_slots <= threads) { spt = 1; cg = std::min(threads / fill_slots, tic); } else { spt = 2; cg = 1; }
    }
    if (spt * ceil_div(tic, cg) > kFillItems) break;
    best = tic;
    if (tic == C) break;
  }
  return best;
}

int rank_tiles(int N, int H, int W, int C, int K, int ks, int stride, int pad, std::vector<tetris_tile>* ranked,
               double density) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs || stride <= 0 || pad < 0)
    return fail(TETRIS_EINVAL, "bad layer shape");
  const bool pointwise = ks == 1 && pad == 0;  // what the flat tiles take (a strided one on the sub-grid it reads)
  if (ks == 1 && stride > 1 && pad == 0) {  // run as a stride-1 layer on the sub-grid it reads (see make_geom)
    H = (H - 1) / stride + 1;
    W = (W - 1) / stride + 1;
    stride = 1;
  }
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
  if (OH <= 0 || OW <= 0) return fail(TETRIS_EINVAL, "empty output");
  // Score every candidate with a small time model calibrated on MI355X and keep the cheapest:
  //   a wave spends about 35 + 41 * quads cycles per entry when two waves share a SIMD (one LDS dword per
  //   FMA is what binds it) and about 0.62 of that when it has the SIMD to itself; a stage costs about 2000
  //   cycles of barriers and stream start-up plus 60 per 16-byte slot a thread stages, and the waves of a
  //   workgroup wait for the slowest one at every stage; a CU holds eight waves.
  static const int kQuadG[][2] = {{2, 16}, {4, 8}, {1, 32}, {2, 8}, {1, 16}, {4, 4}, {1, 8}, {2, 4}, {1, 4}, {2, 2}, {1, 2}, {4, 2}, {1, 1}};
  static const int kWaves[] = {16, 8, 4, 2, 1};
  if (!(density > 0.0) || density > 1.0) density = 0.15;  // mask unknown: typical of the pruned layers this runs
  std::vector<std::pair<double, tetris_tile>> scored;
  for (int lw = 1; lw <= 62; ++lw) {
    if (lw > OW && lw > 1) break;  // wider than four images side by side could use
    if (4 * lw < (OW >= 28 ? 28 : (OW + 1) / 2)) continue;  // narrow tiles stage their halo'd rows poorly (measured)
    const int fold = fold_of(lw, OW);
    // wider than the image only to place 2 or 4 images side by side, and then only as wide as that needs
    if (4 * (lw - 1) >= OW && lw > 1 && (fold == 1 || N < fold || (fold == 2 && 2 * (lw - 1) >= OW) || (fold == 4 && lw - 1 >= OW)))
      continue;
    const Shape s = unit_shape(lw, OH, ceil_div(N, fold), ks, stride);
    const long long units = (long long)ceil_div(OW, (4 / fold) * lw) * ceil_div(OH, s.thi) * ceil_div(N, s.nb * fold);
    for (const auto& qg : kQuadG) {
      const int nq = qg[0], g = qg[1];
      for (int waves : kWaves) {
        const int kb = waves * g;
        if (kb > kSlotPad) continue;
        if (waves == 16 && (g * 4 * nq > kAccRegs / 2 || nq > 2)) continue;
        const int tic_max = max_tile_ic(s, nq, g, waves, stride, C);
        if (tic_max <= 0) continue;
        for (int tic = tic_max, tries = 0; tic >= 1 && tries < 3; tic /= 2, ++tries) {  // fewer channels, more stages
        const long long ugroups = (units + nq - 1) / nq;
        const int kblocks = ceil_div(K, kb);
        const int stages = ceil_div(C, tic);
        const double entries = g * tic * ks * ks * density + 4.0;  // per wave and stage, with stream padding
        // waves of a workgroup meet at a barrier every stage: the slowest of them sets the pace
        const double straggle = waves > 1 ? 1.4 * std::sqrt(entries) : 0.0;
        const double items = (double)tic * nq * s.nb * s.ih * stride * s.ng / (waves * 64);  // staged slots per thread
        // cycles per entry: two waves per SIMD, or four (16-wave workgroups: 110 and 180 measured for one and two quads)
        const bool four = waves == 16 || (waves == 8 && g * 4 * nq <= kAccRegs / 2 && nq <= 2);  // waves per SIMD
        const double per_entry = four ? 40.0 + 70.0 * nq : 35.0 + 41.0 * nq;
        const double per_wave = stages * ((entries + straggle) * per_entry + 2000.0 + 60.0 * items);
        const double waves_total = (double)ugroups * kblocks * waves;
        const double rounds = waves_total / ((double)cu_count() * (four ? 16.0 : 8.0));
        // input re-read by every channel block, in units of the per-wave cycle count (a weak tie-breaker)
        const double reread = 1.0 + 0.02 * kblocks;
        const double cost = per_wave * std::max(rounds, 0.62) * reread;
        tetris_tile t{};
        t.lanes_w = lw; t.quads = nq; t.oc_per_wave = g; t.waves = waves; t.tile_ic = tic;
        scored.emplace_back(cost, t);
        }
      }
    }
  }
  if (pointwise) {
    // Flat tiles of pointwise layers (lanes_w = 64): a unit is 64 consecutive 4-pixel quads of the batch, two LDS
    // buffers of 64 KiB (32 KiB for 8 waves of at most 64 accumulators, two workgroups per CU), 1 KiB per staged
    // channel and unit.  A stage is one walk and one barrier; a walk call costs about 600 cycles before its first entry.
    static const int kFlatG[] = {32, 16, 8, 4, 2, 1};
    const long long quads = (long long)N * ((H * W + 3) / 4);
    for (int waves : {16, 8})
      for (int nq : {1, 2, 4})
        for (int g : kFlatG) {
          const int acc = g * 4 * nq;
          if (acc > (waves == 16 ? kAccRegs / 2 : kAccRegs) || (waves == 16 && nq > 2) || waves * g > kSlotPad) continue;
          const bool half = waves == 8 && acc <= kAccRegs / 2 && nq <= 2;
          const int buf = half ? kFlatHalfBufBytes : kFlatBufBytes;
          for (int tic = 64; tic >= 8; tic /= 2) {
            const int t = std::min(tic, C);
            if (1024 * t * nq > buf) continue;
            const bool four = waves == 16 || half;
            const long long ugroups = ((quads + 63) / 64 + nq - 1) / nq;
            const int kblocks = ceil_div(K, waves * g);
            const int stages = ceil_div(C, t);
            const double entries = std::ceil((g * t * density + 0.5) / 8.0) * 8.0;
            const double per_entry = four ? 40.0 + 70.0 * nq : 35.0 + 41.0 * nq;
            const double per_wave = stages * (entries * per_entry + 600.0 + 900.0) + 6000.0;
            const double rounds = (double)ugroups * kblocks * waves / ((double)cu_count() * (four ? 16.0 : 8.0));
            const double cost = per_wave * std::max(rounds, 0.62) * (1.0 + 0.02 * kblocks);
            tetris_tile tt{};
            tt.lanes_w = kFlatLanes; tt.quads = nq; tt.oc_per_wave = g; tt.waves = waves; tt.tile_ic = t;
            scored.emplace_back(cost, tt);
            if (t == C) break;
          }
        }
  }
  if (scored.empty()) return fail(TETRIS_EINVAL, "no tile shape fits this layer");
  std::stable_sort(scored.begin(), scored.end(),
                   [](const std::pair<double, tetris_tile>& a, const std::pair<double, tetris_tile>& b) { return a.first < b.first; });
  ranked->clear();
  for (const auto& e : scored) ranked->push_back(e.second);
  return TETRIS_OK;
}

namespace {
// Tiles measured on MI355X (tetris_tile_autotune over the benchmark suites), keyed by layer shape.  They play the
// part of the reference's per-layer table of template instantiations (Tetris/spconv2d.cc:90-329).
struct Tuned {
  int N, H, W, C, K, ks, stride, pad;
  tetris_tile tile;
};
const Tuned kTuned[] = {
#include "tuned_tiles.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, {0, 0, 0, 0, 0, 0}}};

// Rows a caller loaded at run time (tetris_tile_table_load); they are looked up before the built-in ones.
std::mutex g_loaded_mu;
std::vector<Tuned> g_loaded;

// trust a table row only as far as the kernel's own checks go
bool usable(const Tuned& e) {
  tetris_g950 shape;
  shape.C = e.C; shape.K = e.K; shape.ks = e.ks; shape.tile_ic = e.tile.tile_ic; shape.g = e.tile.oc_per_wave;
  if (e.tile.tile_ic <= 0 || e.tile.oc_per_wave <= 0) return false;
  shape.stages = ceil_div(e.C, e.tile.tile_ic);
  shape.slots = ceil_div(e.K, kSlotPad) * kSlotPad;
  Geom g;
  return make_geom(&shape, e.N, e.H, e.W, e.stride, e.pad, e.tile, &g) == TETRIS_OK;
}

bool same_shape(const Tuned& e, int N, int H, int W, int C, int K, int ks, int stride, int pad) {
  return e.N == N && e.H == H && e.W == W && e.C == C && e.K == K && e.ks == ks && e.stride == stride && e.pad == pad;
}
}  // namespace

int load_tile_table(const char* path, int* rows_out) {
  FILE* fp = std::fopen(path, "r");
  if (!fp) return fail(TETRIS_EIO, "cannot open tile table %s", path);
  std::vector<Tuned> rows;
  char line[512];
  while (std::fgets(line, sizeof line, fp)) {
    Tuned e{};
    // the tile's sixth number (csplit) is optional: a row without it leaves the split to the library's rule
    const int n = std::sscanf(line, " {%d, %d, %d, %d, %d, %d, %d, %d, {%d, %d, %d, %d, %d, %d}}", &e.N, &e.H, &e.W, &e.C, &e.K,
                              &e.ks, &e.stride, &e.pad, &e.tile.lanes_w, &e.tile.quads, &e.tile.oc_per_wave, &e.tile.waves,
                              &e.tile.tile_ic, &e.tile.csplit);
    if (n == 13) e.tile.csplit = 0;
    if (n >= 13) rows.push_back(e);
  }
  std::fclose(fp);
  std::lock_guard<std::mutex> lock(g_loaded_mu);
  g_loaded.insert(g_loaded.begin(), rows.begin(), rows.end());
  if (rows_out) *rows_out = (int)rows.size();
  return TETRIS_OK;
}

int choose_tile(int N, int H, int W, int C, int K, int ks, int stride, int pad, tetris_tile* t) {
  {
    std::lock_guard<std::mutex> lock(g_loaded_mu);
    for (const Tuned& e : g_loaded)
      if (same_shape(e, N, H, W, C, K, ks, stride, pad) && usable(e)) {
        *t = e.tile;
        return TETRIS_OK;
      }
  }
  for (const Tuned& e : kTuned)
    if (same_shape(e, N, H, W, C, K, ks, stride, pad)) {
      if (usable(e)) {
        *t = e.tile;
        return TETRIS_OK;
      }
      break;
    }
  // Not measured: borrow the tile of the most similar measured layer of the same kernel size and stride (image
  // width first -- it fixes the lane layout --, then pixels per launch, then channel counts), if the kernel accepts
  // it for this shape.  The cycle model below ranks 16-wave tiles too high on small feature maps; the nearest measured
  // neighbour is within 10 % of a measured choice where the model is 1.5x off.
  {
    auto lg = [](double a, double b) { return std::fabs(std::log2(a / b)); };
    const int OW = out_extent(W, pad, ks, stride), OH = out_extent(H, pad, ks, stride);
    std::vector<std::pair<double, const Tuned*>> near;
    for (const Tuned& e : kTuned) {
      if (e.N == 0 || e.ks != ks || e.stride != stride) continue;
      const int eow = out_extent(e.W, e.pad, e.ks, e.stride), eoh = out_extent(e.H, e.pad, e.ks, e.stride);
      const double d = 4.0 * lg(OW, eow) + 2.0 * lg((double)N * OH * OW, (double)e.N * eoh * eow) + lg(C, e.C) + lg(K, e.K) +
                       0.5 * lg(N, e.N);
      near.emplace_back(d, &e);
    }
    std::sort(near.begin(), near.end(), [](const std::pair<double, const Tuned*>& a, const std::pair<double, const Tuned*>& b) { return a.first < b.first; });
    for (size_t i = 0; i < near.size() && i < 6 && near[i].first < 6.0; ++i) {
      Tuned cand = *near[i].second;
      // same number of units across the image as in the neighbour, at this image's width
      const int eow = out_extent(cand.W, cand.pad, cand.ks, cand.stride);
      const int per_image = 4 / fold_of(cand.tile.lanes_w, eow);  // column groups of a lane that belong to one image
      const int units_w = ceil_div(eow, per_image * cand.tile.lanes_w);
      cand.tile.lanes_w = ceil_div(OW, per_image * units_w);
      cand.N = N; cand.H = H; cand.W = W; cand.C = C; cand.K = K; cand.pad = pad;
      cand.tile.tile_ic = std::min(cand.tile.tile_ic, C);
      if (usable(cand)) {
        *t = cand.tile;
        return TETRIS_OK;
      }
    }
  }
  std::vector<tetris_tile> ranked;
  const int rc = rank_tiles(N, H, W, C, K, ks, stride, pad, &ranked);
  if (rc) return rc;
  for (const tetris_tile& cand : ranked) {  // the model ranks shapes the kernel's own checks may still refuse
    Tuned e{N, H, W, C, K, ks, stride, pad, cand};
    if (usable(e)) {
      *t = cand;
      return TETRIS_OK;
    }
  }
  return fail(TETRIS_EINVAL, "no tile shape the kernel accepts for this layer");
}

// Output-channel order that evens out the work inside a workgroup.  A wave walks the entries of its
// `oc_per_wave` slots stage by stage and the waves of a workgroup meet at a barrier after every stage.  Waves
// w, w + 4, w + 8, ... run on the same SIMD and share its issue slots, so what a stage costs is the entry count of
// the busiest SIMD; the busiest wave only matters at the end of a stage, when a SIMD is left with one wave that
// cannot fill it alone.  (Measured against file order, whole VGG19-shaped stack at batch 16: -4 % with the masks
// of a shipped pruned network, -1.7 % with uniform random masks.)  Pruned networks have output channels of very different density (some
// are empty): in file order the busiest wave of a stage carries 1.2-1.5x the mean.
// The channels are sorted by their number of non-zeros and dealt to the workgroups' blocks of
// waves*oc_per_wave slots in serpentine order (blocks of equal total work: no straggler workgroup); inside a
// block each channel, heaviest first, goes to the wave where it raises, summed over the stages, the busiest SIMD's
// count the least, then the busiest wave's.  Plays the part of ReorderOutChannel
// (Tetris/spconv2d_utils.h:275-420), whose own objective -- lanes of a warp with alike channels -- does not fit a
// wave that sums its channels.
int balance_oc_order(const float* filter, int C, int K, int ks, const tetris_tile& t, int32_t* order) {
  const int G = t.oc_per_wave, waves = t.waves, tile_ic = t.tile_ic;
  if (G <= 0 || waves <= 0 || tile_ic <= 0) return fail(TETRIS_EINVAL, "bad tile");
  const int S = ceil_div(C, tile_ic), B = G * waves, nblocks = ceil_div(K, B), taps = ks * ks;
  std::vector<int32_t> per((size_t)K * S, 0);
  std::vector<int64_t> total(K, 0);
  for (int k = 0; k < K; ++k)
    for (int c = 0; c < C; ++c) {
      const float* w = filter + ((size_t)k * C + c) * taps;
      int n = 0;
      for (int i = 0; i < taps; ++i) n += w[i] != 0.f;
      per[(size_t)k * S + c / tile_ic] += n;
      total[k] += n;
    }
  std::vector<int32_t> sorted(K);
  for (int k = 0; k < K; ++k) sorted[k] = k;
  std::stable_sort(sorted.begin(), sorted.end(), [&](int32_t a, int32_t b) { return total[a] > total[b]; });
  // serpentine deal; the last block may hold fewer than B channels
  std::vector<std::vector<int32_t>> blocks(nblocks);
  {
    int b = 0, d = 1;
    for (int32_t k : sorted) {
      while ((int)blocks[b].size() >= std::min(B, K - b * B)) {
        b += d;
        if (b < 0 || b >= nblocks) { d = -d; b += d; }
      }
      blocks[b].push_back(k);
      b += d;
      if (b < 0 || b >= nblocks) { d = -d; b += d; }
    }
  }
  const int nsimd = std::min(4, waves);  // wave w runs on SIMD w % 4
  std::vector<int64_t> load((size_t)waves * S), busiest(S), simd_load((size_t)nsimd * S), busiest_simd(S);
  std::vector<std::vector<int32_t>> members(waves);
  int32_t* o = order;
  for (const std::vector<int32_t>& blk : blocks) {
    std::fill(load.begin(), load.end(), 0);
    std::fill(busiest.begin(), busiest.end(), 0);
    std::fill(simd_load.begin(), simd_load.end(), 0);
    std::fill(busiest_simd.begin(), busiest_simd.end(), 0);
    for (auto& m : members) m.clear();
    const int len = (int)blk.size();
    for (int32_t k : blk) {
      int best = -1;
      int64_t best_simd = 0, best_wave = 0, best_sum = 0;
      for (int w = 0; w < waves; ++w) {
        const int cap = std::min(G, std::max(0, len - w * G));  // slots of this wave that hold a channel
        if ((int)members[w].size() >= cap) continue;
        const int sd = w % nsimd;
        int64_t cost_simd = 0, cost_wave = 0, sum = 0;
        for (int s = 0; s < S; ++s) {
          const int64_t add = per[(size_t)k * S + s];
          cost_simd += std::max(busiest_simd[s], simd_load[(size_t)sd * S + s] + add);
          cost_wave += std::max(busiest[s], load[(size_t)w * S + s] + add);
          sum += load[(size_t)w * S + s];
        }
        if (best < 0 || cost_simd < best_simd || (cost_simd == best_simd && (cost_wave < best_wave ||
            (cost_wave == best_wave && sum < best_sum)))) {
          best = w; best_simd = cost_simd; best_wave = cost_wave; best_sum = sum;
        }
      }
      const int sd = best % nsimd;
      for (int s = 0; s < S; ++s) {
        const int64_t add = per[(size_t)k * S + s];
        load[(size_t)best * S + s] += add;
        busiest[s] = std::max(busiest[s], load[(size_t)best * S + s]);
        simd_load[(size_t)sd * S + s] += add;
        busiest_simd[s] = std::max(busiest_simd[s], simd_load[(size_t)sd * S + s]);
      }
      members[best].push_back(k);
    }
    for (int w = 0; w < waves; ++w)
      for (int32_t k : members[w]) *o++ = k;
  }
  // The deal is a heuristic: keep the file order when it is no worse by the measure the deal aims at (what the waves
  // of a workgroup wait for: per block and stage the busiest wave's entries, summed).
  auto wait_cost = [&](auto channel_at) {
    int64_t sum = 0;
    for (int b = 0; b < nblocks; ++b)
      for (int s = 0; s < S; ++s) {
        int64_t worst = 0;
        for (int w = 0; w < waves; ++w) {
          int64_t n = 0;
          for (int i = 0; i < G; ++i) {
            const int slot = b * B + w * G + i;
            if (slot < K) n += per[(size_t)channel_at(slot) * S + s];
          }
          worst = std::max(worst, n);
        }
        sum += worst;
      }
    return sum;
  };
  if (wait_cost([&](int slot) { return slot; }) <= wait_cost([&](int slot) { return order[slot]; }))
    for (int k = 0; k < K; ++k) order[k] = k;
  return TETRIS_OK;
}

}  // namespace tetris
