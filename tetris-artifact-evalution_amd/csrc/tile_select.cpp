// Tile-shape selection for the gfx950 conv kernel: turns a layer shape plus a tetris_tile into the
// kernel geometry, and picks a tetris_tile when the caller leaves it to the library.
//
// Takes the place of the reference's exhaustive search over 185 compiled {KS, STRIDE, TILE_IC, TILE_H,
// TILE_W} instantiations (Tetris/spconv2d.cc:90-329, 130 launches and one re-pack per candidate).
#include <algorithm>
#include <climits>

#include "common.h"

namespace tetris {

namespace {

constexpr int kLdsLimit = 160 * 1024;

// LDS serves a 16-byte-per-lane read in groups of lanes over 64 four-byte banks.  Score a row pitch by
// the worst bank multiplicity inside each group of 16 consecutive lanes (1 = conflict free).
int bank_cost(int lw, int lh, int stride, int pitch) {
  int cost = 0;
  for (int g0 = 0; g0 < 64; g0 += 16) {
    int banks[64] = {0};
    for (int l = g0; l < g0 + 16; ++l) {
      const int lx = l % lw, ly = l / lw;
      if (ly >= lh) continue;
      const int dw = ly * stride * pitch + lx * 4;
      for (int j = 0; j < 4; ++j) banks[(dw + j) & 63] += 1;
    }
    cost += *std::max_element(banks, banks + 64);
  }
  return cost;
}

}  // namespace

int make_geom(const tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile& t, Geom* out) {
  Geom g{};
  if (N <= 0 || H <= 0 || W <= 0 || stride <= 0 || pad < 0)
    return fail(TETRIS_EINVAL, "bad conv shape N=%d H=%d W=%d stride=%d pad=%d", N, H, W, stride, pad);
  g.N = N; g.C = p->C; g.H = H; g.W = W; g.K = p->K; g.ks = p->ks; g.stride = stride; g.pad = pad;
  g.OH = out_extent(H, pad, p->ks, stride);
  g.OW = out_extent(W, pad, p->ks, stride);
  if (H + 2 * pad < p->ks || W + 2 * pad < p->ks || g.OH <= 0 || g.OW <= 0)
    return fail(TETRIS_EINVAL, "kernel %d does not fit the padded %dx%d image", p->ks, H, W);
  if ((long long)N * p->C * H * W >= INT_MAX || (long long)N * p->K * g.OH * g.OW >= (1ll << 40))
    return fail(TETRIS_EINVAL, "tensor too large for 32-bit in-tile offsets");
  g.tile_ic = p->tile_ic;
  g.stages = p->stages;
  g.slots = p->slots;

  const int nq = t.quads;
  if (t.lanes_w < 1 || t.lanes_w > 64 || (nq != 1 && nq != 2 && nq != 4))
    return fail(TETRIS_EINVAL, "bad tile: lanes_w=%d quads=%d", t.lanes_w, nq);
  if ((t.oc_per_wave != 4 && t.oc_per_wave != 8 && t.oc_per_wave != 16) ||
      (t.waves != 1 && t.waves != 2 && t.waves != 4 && t.waves != 8))
    return fail(TETRIS_EINVAL, "bad tile: oc_per_wave=%d waves=%d", t.oc_per_wave, t.waves);
  g.lw = t.lanes_w;
  g.lh = 64 / g.lw;
  const int vrows = nq * g.lh;
  g.thi = std::min(vrows, g.OH);
  g.nb = std::max(1, std::min(vrows / g.thi, N));
  g.ng = g.lw + (p->ks - 1) / stride;
  g.par = 4 * g.ng;
  const int min_pitch = stride * g.par;
  int best_pitch = min_pitch, best_cost = INT_MAX;
  for (int pitch = min_pitch; pitch <= min_pitch + min_pitch / 4 + 4; pitch += 4) {
    const int c = bank_cost(g.lw, g.lh, stride, pitch);
    if (c < best_cost) {
      best_cost = c;
      best_pitch = pitch;
    }
  }
  g.pitch = best_pitch;
  g.ih = stride * (g.thi - 1) + p->ks;
  g.plane = g.ih * g.pitch;
  g.img_stride = g.tile_ic * g.plane;
  g.fill_slots = g.nb * g.ih * stride * g.ng;
  g.tiles_w = ceil_div(g.OW, 4 * g.lw);
  g.tiles_h = ceil_div(g.OH, g.thi);
  g.tiles_n = ceil_div(N, g.nb);
  g.kb = t.waves * t.oc_per_wave;
  g.kblocks = ceil_div(p->K, g.kb);
  if (g.kblocks * g.kb > p->slots) return fail(TETRIS_EINVAL, "channel block %d does not divide the slot padding", g.kb);
  const long long lds = 4ll * g.nb * g.img_stride + 20ll * g.fill_slots;
  if (lds > kLdsLimit)
    return fail(TETRIS_EINVAL, "tile needs %lld bytes of LDS (limit %d): lower tile_ic, quads or lanes_w", lds,
                kLdsLimit);
  g.lds_bytes = (int)lds;
  if ((long long)g.tiles_n * g.tiles_h * g.tiles_w * g.kblocks > (1ll << 30))
    return fail(TETRIS_EINVAL, "grid too large");
  *out = g;
  return TETRIS_OK;
}

int choose_tile(int N, int H, int W, int C, int K, int ks, int stride, int pad, tetris_tile* t) {
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs || stride <= 0 || pad < 0)
    return fail(TETRIS_EINVAL, "bad layer shape");
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
  if (OH <= 0 || OW <= 0) return fail(TETRIS_EINVAL, "empty output");
  tetris_tile best{};
  best.quads = 2;
  best.oc_per_wave = 8;
  best.waves = 4;
  while (best.waves > 1 && best.waves * best.oc_per_wave / 2 >= K) best.waves /= 2;
  // lanes across: least padded pixel slots, then the widest rows
  long long best_slots = LLONG_MAX;
  const int cand[] = {16, 14, 13, 8, 7, 4, 2, 1};
  for (int lw : cand) {
    const int lh = 64 / lw, vrows = best.quads * lh;
    const int thi = std::min(vrows, OH);
    const int nb = std::max(1, std::min(vrows / thi, N));
    const long long tiles = (long long)ceil_div(OW, 4 * lw) * ceil_div(OH, thi) * ceil_div(N, nb);
    const long long slots = tiles * 64 * best.quads * 4;
    if (slots < best_slots) {
      best_slots = slots;
      best.lanes_w = lw;
    }
  }
  // input channels per stage: the most that keeps three workgroups per CU resident
  const int lw = best.lanes_w, lh = 64 / lw, vrows = best.quads * lh;
  const int thi = std::min(vrows, OH), nb = std::max(1, std::min(vrows / thi, N));
  const int ih = stride * (thi - 1) + ks;
  const int pitch = stride * 4 * (lw + (ks - 1) / stride);
  const long long per_ic = 4ll * nb * ih * (pitch + pitch / 8);
  int tile_ic = 64;
  while (tile_ic > 4 && per_ic * tile_ic > 50 * 1024) tile_ic /= 2;
  while (tile_ic > 4 && tile_ic / 2 >= C) tile_ic /= 2;
  best.tile_ic = tile_ic;
  *t = best;
  return TETRIS_OK;
}

}  // namespace tetris
