// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's spconv2d / spf path.
//
// Nothing shipped may link, load or call this file: it exists so that tests, the smoke check and
// the benchmark's cpu_baseline leg can compare the HIP engine with the algorithm the reference
// defines.  Every function names the reference lines it follows (paths relative to the reference
// checkout, directory Tetris/).
//
// How each function is pinned (see tests/test_oracle_*.py):
//   orc_host_conv2d            torch.nn.functional.conv2d, closed forms (all-ones, one-hot filter),
//                              and the reference's own tensor_utils.cc compiled unmodified
//                              (oracle/_ref, when the reference checkout is present)
//   orc_read_weight_file       the compiled reference reader (oracle/_ref) on shipped weight files
//   orc_spf_pack               plain step 1: the scan order the text fixes, invariants, decode == filter non-zeros;
//                              Bank-SR and ReorderOutChannel: hand-worked cases derived step by step from the text
//                              of spconv2d_utils.h:99-199 and :275-420 (broadcast pass, free-bank pass, wait-list
//                              pads, the entry-index-as-bank comparison of :184, cost function with duplicates and
//                              padding term, ties, two stages, K % 8 != 0), per-step invariants on random filters,
//                              and both-flags == Bank-SR on the permuted filter (tests/test_oracle_handworked.py);
//                              as a cross-check, FNV-1a answers recorded from a compiled reference for six shipped
//                              layers (tests/golden/spf_known_answers.json)
//   orc_host_spconv2d*,        decode(pack(filter)) convolved == orc_host_conv2d
//   orc_g950_*                 layout defined by this project (no reference counterpart); pinned by
//                              multiset equality with the filter's non-zeros and by conv equality
//
// Build: make -C oracle   (g++ -O2 -fopenmp -shared -fPIC)

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr int kLanes = 32;   // spconv2d_utils.h:15   WARP_SIZE
constexpr int kBitS = 3;     // spconv2d_utils.h:19
constexpr int kBitR = 3;     // spconv2d_utils.h:20
constexpr int kSubGroup = 8; // spconv2d_utils.h:299  GROUP_SIZE

inline int out_extent(int in, int pad, int ks, int stride) { return (in + 2 * pad - ks) / stride + 1; }

inline int32_t make_pos(int s, int r, int ic) { return s + (r << kBitS) + (ic << (kBitS + kBitR)); }

}  // namespace

struct OrcPack {
  int C = 0, K = 0, ks = 0, tile_ic = 0, stages = 0;
  int apply_reorder = 0, vec = 1;
  int64_t nnz = 0;        // counted only on the keep-as-is path, like the reference's nnz_
  int64_t bank_oob = 0;   // times Bank-SR's entry-index-as-bank read would have left the 32 flags
  std::vector<int32_t> perm, stage_len, offsets, position;
  std::vector<float> values;
};

namespace {

// spconv2d_utils.h:275-420  ReorderOutChannel
void reorder_out_channel(OrcPack& P, const float* filter) {
  const int C = P.C, K = P.K, ks = P.ks, T = P.tile_ic, S = P.stages;
  const int kk = ks * ks;
  std::vector<int> cnt((size_t)K * S, 0);
  std::vector<std::vector<int>> nzpos((size_t)K * S);
  for (int o = 0; o < K; ++o)
    for (int i = 0; i < C; i += T) {
      const int sid = o * S + i / T;
      for (int j = i; j < std::min(i + T, C); ++j)
        for (int r = 0; r < ks; ++r)
          for (int s = 0; s < ks; ++s)
            if (filter[(size_t)o * C * kk + (size_t)j * kk + r * ks + s] != 0.f) {
              cnt[sid] += 1;
              nzpos[sid].push_back(make_pos(s, r, j));  // :289 global channel index
            }
    }

  struct Sub {
    int l, r, cost;
    bool operator<(const Sub& b) const { return cost != b.cost ? cost > b.cost : l < b.l; }  // :303-307
  };
  std::set<Sub> waiting;
  for (int i = 0; i < K; i += kSubGroup) {
    const int l = i, r = std::min(K, i + kSubGroup);
    int cost = 0;
    for (int j = 0; j < S; ++j) {
      int m = 0;
      for (int t = l; t < r; ++t) m = std::max(m, cnt[t * S + j]);
      cost += m;
    }
    waiting.insert(Sub{l, r, cost});
  }

  P.perm.clear();
  while (!waiting.empty()) {
    std::vector<int> group;
    std::vector<int> cur_mx(S, 0);
    std::vector<int> cur_bank((size_t)S * kLanes, 0);
    std::unordered_map<int, int> seen;
    const Sub seed = *waiting.begin();
    waiting.erase(waiting.begin());
    for (int t = seed.l; t < seed.r; ++t) group.push_back(t);

    auto upd_mx = [&](int oc) {
      for (int i = 0; i < S; ++i) cur_mx[i] = std::max(cur_mx[i], cnt[oc * S + i]);
    };
    auto upd_bank = [&](int l, int r) {  // :345-358
      for (int oc = l; oc < r; ++oc)
        for (int i = 0; i < S; ++i)
          for (int pos : nzpos[oc * S + i]) {
            const int bank = (pos >> (kBitS + kBitR)) % kLanes;
            if (!seen.count(pos)) {
              cur_bank[i * kLanes + bank] += 1;
              seen[pos] = 1;
            }
          }
    };
    auto cost_of = [&](int l, int r) -> float {  // :360-391
      float total = 0;
      for (int i = 0; i < S; ++i) {
        std::vector<int> bank(kLanes, 0);
        int mx = 0;
        for (int oc = l; oc < r; ++oc) {
          mx = std::max(mx, cnt[oc * S + i]);
          for (int pos : nzpos[oc * S + i])
            if (!seen.count(pos)) bank[(pos >> (kBitS + kBitR)) % kLanes] += 1;
        }
        const int padding = mx - cur_mx[i] > 0 ? mx - cur_mx[i] : cur_mx[i] - mx;
        int mx_bank = bank[0] + cur_bank[i * kLanes];
        for (int t = 0; t < kLanes; ++t) mx_bank = std::max(mx_bank, bank[t] + cur_bank[i * kLanes + t]);
        total += std::max(mx_bank - std::max(mx, cur_mx[i]), padding);
      }
      return total;
    };

    for (int t = seed.l; t < seed.r; ++t) upd_mx(t);
    upd_bank(seed.l, seed.r);

    while (!waiting.empty() && group.size() < (size_t)kLanes) {  // :399-417
      float best_cost = 1e18;
      Sub best{-1, -1, -1};
      for (const Sub& c : waiting) {
        const float v = cost_of(c.l, c.r);
        if (v < best_cost) {
          best_cost = v;
          best = c;
        }
      }
      waiting.erase(best);
      upd_bank(best.l, best.r);
      for (int t = best.l; t < best.r; ++t) {
        upd_mx(t);
        group.push_back(t);
      }
    }
    P.perm.insert(P.perm.end(), group.begin(), group.end());
  }
}

// spconv2d_utils.h:38-61  keep-as-is (CSR-like) format
void pack_plain_rows(OrcPack& P, const float* filter) {
  const int C = P.C, K = P.K, ks = P.ks, T = P.tile_ic;
  const int kk = ks * ks;
  for (int o = 0; o < K; ++o)
    for (int i = 0; i < C; ++i) {
      if (i % T == 0) P.offsets.push_back(P.offsets.back());
      for (int r = 0; r < ks; ++r)
        for (int s = 0; s < ks; ++s) {
          const float v = filter[(size_t)o * C * kk + (size_t)i * kk + r * ks + s];
          if (v != 0.f) {
            P.nnz += 1;
            P.values.push_back(v);
            P.position.push_back(make_pos(s, r, i % T));
            P.offsets.back() += 1;
          }
        }
    }
}

struct LaneList {
  std::vector<float> v;
  std::vector<int32_t> p;
};

// scan-order entries of packed lane `o` in stage starting at channel i  (:85-94 / :107-117)
void scan_stage(const OrcPack& P, const float* filter, int o, int i, LaneList& out) {
  const int C = P.C, ks = P.ks, T = P.tile_ic, kk = ks * ks;
  const int src = P.perm[o];
  for (int j = i; j < std::min(i + T, C); ++j)
    for (int r = 0; r < ks; ++r)
      for (int s = 0; s < ks; ++s) {
        const float v = filter[(size_t)src * C * kk + (size_t)j * kk + r * ks + s];
        if (v != 0.f) {
          out.v.push_back(v);
          out.p.push_back(make_pos(s, r, j % T));
        }
      }
}

// spconv2d_utils.h:100-198  Bank-SR ordering of one (group, stage)
void bank_sr_stage(OrcPack& P, const float* filter, int g, int i, std::vector<LaneList>& lists) {
  const int K = P.K, C = P.C, ks = P.ks, S = P.stages, T = P.tile_ic, kk = ks * ks;
  LaneList tmp[kLanes];
  int pad_left[kLanes];
  int longest = 0;
  for (int o = g; o < std::min(g + kLanes, K); ++o) {
    scan_stage(P, filter, o, i, tmp[o - g]);
    longest = std::max(longest, (int)tmp[o - g].v.size());
  }
  for (int l = 0; l < kLanes; ++l) pad_left[l] = longest - (int)tmp[l].v.size();

  for (int t = 0; t < longest; ++t) {
    std::vector<int> bank_flag(kLanes, 0);
    std::vector<int> tap_flag((size_t)C * kk, 0);
    std::vector<int> wait;
    for (int l = 0; l < kLanes; ++l) {
      LaneList& L = tmp[l];
      int pick = -1;
      for (size_t j = 0; j < L.p.size(); ++j) {  // :131-141 already-broadcast tap
        const int pos = L.p[j];
        const int ic = pos >> (kBitS + kBitR), y = pos & 7, x = (pos >> kBitS) & 7;
        if (tap_flag[ic * kk + x * ks + y] == 1) {
          pick = (int)j;
          break;
        }
      }
      for (size_t j = 0; j < L.p.size(); ++j) {  // :143-155 first entry on a free bank
        const int pos = L.p[j];
        const int ic = pos >> (kBitS + kBitR), y = pos & 7, x = (pos >> kBitS) & 7;
        const int bank = ic % kLanes;
        if (bank_flag[bank] == 0 && pick == -1) {
          pick = (int)j;
          bank_flag[bank] = 1;
          tap_flag[ic * kk + x * ks + y] = 1;
          break;
        }
      }
      if (pick != -1) {
        LaneList& dst = lists[(size_t)(g + l) * S + i / T];
        dst.v.push_back(L.v[pick]);
        dst.p.push_back(L.p[pick]);
        L.v.erase(L.v.begin() + pick);
        L.p.erase(L.p.begin() + pick);
      } else {
        wait.push_back(l);
      }
    }
    for (int l : wait) {  // :167-195
      LaneList& L = tmp[l];
      LaneList& dst = lists[(size_t)(g + l) * S + i / T];
      if (pad_left[l] > 0) {
        for (int b = 0; b < kLanes; ++b)
          if (bank_flag[b] == 0) {
            bank_flag[b] = 1;
            pad_left[l] -= 1;
            dst.v.push_back(0.0f);
            dst.p.push_back(b << (kBitS + kBitR));
            break;
          }
      } else {
        int pick = -1;
        for (size_t j = 0; j < L.p.size(); ++j) {
          const int bank = (L.p[j] >> (kBitS + kBitR)) % kLanes;
          // :184 compares bank_flag[pick] -- the flags indexed by the ENTRY index -- as written.
          int lhs = 0;
          if (pick != -1) {
            if (pick >= kLanes) {
              P.bank_oob += 1;  // the reference would read past its 32-int vector here
              lhs = 0;
            } else {
              lhs = bank_flag[pick];
            }
          }
          if (pick == -1 || lhs > bank_flag[bank]) pick = (int)j;
        }
        const int bank = (L.p[pick] >> (kBitS + kBitR)) % kLanes;
        bank_flag[bank] += 1;
        dst.v.push_back(L.v[pick]);
        dst.p.push_back(L.p[pick]);
        L.v.erase(L.v.begin() + pick);
        L.p.erase(L.p.begin() + pick);
      }
    }
  }
}

// spconv2d_utils.h:62-246  reorder path (SPF)
void pack_spf(OrcPack& P, const float* filter, int bank_optimize, int reorder_oc) {
  const int K = P.K, C = P.C, S = P.stages, T = P.tile_ic;
  if (reorder_oc) reorder_out_channel(P, filter);  // :66-70
  const int groups = (K - 1) / kLanes + 1;
  const int padK = groups * kLanes;
  P.offsets.assign((size_t)groups * S + 1, 0);      // :75
  P.stage_len.assign((size_t)groups * kLanes * S, 0);  // :76
  std::vector<LaneList> lists((size_t)padK * S + 1);

  for (int g = 0; g < K; g += kLanes)
    for (int i = 0; i < C; i += T) {
      if (!bank_optimize) {
        for (int o = g; o < std::min(g + kLanes, K); ++o) scan_stage(P, filter, o, i, lists[(size_t)o * S + i / T]);
      } else {
        bank_sr_stage(P, filter, g, i, lists);
      }
    }

  const int vec = P.vec;
  for (int w = 0; w < K; w += kLanes)  // :207-244
    for (int i = 0; i < C; i += T) {
      int longest = 0;
      for (int o = w; o < std::min(K, w + kLanes); ++o) {
        const int n = (int)lists[(size_t)o * S + i / T].v.size();
        longest = std::max(longest, (n + vec - 1) / vec * vec);
      }
      const int oid = w / kLanes * S + i / T;
      P.offsets[oid + 1] = P.offsets[oid] + longest;
      for (int o = w; o < std::min(K, w + kLanes); ++o)
        P.stage_len[(size_t)w * S + (size_t)(i / T) * kLanes + o % kLanes] = (int)lists[(size_t)o * S + i / T].v.size();
      for (int t = 0; t < longest; t += vec)
        for (int o = w; o < w + kLanes; ++o) {
          const LaneList& L = lists[(size_t)o * S + i / T];
          for (int it = 0; it < vec; ++it) {
            if ((size_t)(t + it) < L.v.size()) {
              P.values.push_back(L.v[t + it]);
              P.position.push_back(L.p[t + it]);
            } else {
              P.values.push_back(0.0f);
              P.position.push_back(0);
            }
          }
        }
    }
}

}  // namespace

extern "C" {

// tensor_utils.cc:136-170  HostConv2d (dense, NCHW / OIHW, zero padding, floor output extent)
// `threads` > 1 splits the (n, oc) loop only, which leaves each output's summation order alone.
void orc_host_conv2d(const float* input, const float* filter, float* output, int N, int H, int W, int C, int K,
                     int ks, int stride, int pad, int threads) {
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
#pragma omp parallel for collapse(2) schedule(dynamic) num_threads(threads > 0 ? threads : 1)
  for (int n = 0; n < N; ++n)
    for (int oc = 0; oc < K; ++oc)
      for (int h = 0; h < OH; ++h)
        for (int w = 0; w < OW; ++w) {
          float* o = &output[(((size_t)n * K + oc) * OH + h) * OW + w];
          *o = 0.f;
          for (int ic = 0; ic < C; ++ic)
            for (int x = 0; x < ks; ++x)
              for (int y = 0; y < ks; ++y) {
                const int ih = h * stride + x, iw = w * stride + y;
                if (ih < pad || ih >= H + pad) continue;
                if (iw < pad || iw >= W + pad) continue;
                *o += input[(((size_t)n * C + ic) * H + (ih - pad)) * W + (iw - pad)] *
                      filter[(((size_t)oc * C + ic) * ks + x) * ks + y];
              }
        }
}

// tensor_utils.cc:17-19
int orc_float_equal(float x, float y) { return fabs(x - y) <= 1e-5 * (fabs(x) + fabs(y)) + 1e-5; }

// tensor_utils.cc:21-34; returns the first differing index or -1
int64_t orc_tensor_first_mismatch(const float* a, const float* b, int64_t len) {
  for (int64_t i = 0; i < len; ++i)
    if (!orc_float_equal(a[i], b[i])) return i;
  return -1;
}

// tensor_utils.cc:55-82; header order H W IC OC KS PAD STRIDE GROUPS, then OC*IC*KS*KS floats.
// hdr receives the eight header ints in file order.  Returns 0, or 1 when the file cannot be opened
// (where the reference prints "Open file error." and exits).
int orc_read_weight_file(const char* path, int32_t* hdr, float** filter_out, int64_t* nnz_out) {
  std::ifstream in(path);
  if (!in.is_open()) return 1;
  for (int i = 0; i < 8; ++i) in >> hdr[i];
  const int64_t n = (int64_t)hdr[3] * hdr[2] * hdr[4] * hdr[4];
  float* f = (float*)malloc((size_t)n * sizeof(float));
  int64_t nnz = 0;
  for (int64_t i = 0; i < n; ++i) {
    in >> f[i];
    if (f[i] != 0) nnz += 1;
  }
  *filter_out = f;
  *nnz_out = nnz;
  return 0;
}

void orc_free(void* p) { free(p); }

// tensor_utils.cc:87-99 (NCHW2NHWC) / :101-113 (NHWC2NCHW); out of place here, the reference works in place
void orc_nchw_to_nhwc(const float* src, float* dst, int N, int C, int H, int W) {
  for (int n = 0; n < N; ++n)
    for (int h = 0; h < H; ++h)
      for (int w = 0; w < W; ++w)
        for (int c = 0; c < C; ++c)
          dst[(((size_t)n * H + h) * W + w) * C + c] = src[(((size_t)n * C + c) * H + h) * W + w];
}
void orc_nhwc_to_nchw(const float* src, float* dst, int N, int C, int H, int W) {
  for (int n = 0; n < N; ++n)
    for (int c = 0; c < C; ++c)
      for (int h = 0; h < H; ++h)
        for (int w = 0; w < W; ++w)
          dst[(((size_t)n * C + c) * H + h) * W + w] = src[(((size_t)n * H + h) * W + w) * C + c];
}

// spconv2d_utils.h:25-246  SparseFilter constructor; the two compile-time macros are arguments here.
OrcPack* orc_spf_pack(const float* filter, int C, int K, int ks, int tile_ic, int apply_reorder, int apply_vectorize,
                      int bank_optimize, int reorder_out_channel) {
  OrcPack* P = new OrcPack;
  P->C = C; P->K = K; P->ks = ks; P->tile_ic = tile_ic;
  P->stages = (C - 1) / tile_ic + 1;
  P->apply_reorder = apply_reorder;
  P->vec = apply_vectorize ? 4 : 1;
  P->offsets.push_back(0);
  for (int o = 0; o < K; ++o) P->perm.push_back(o);
  if (!apply_reorder) {
    P->vec = 1;
    pack_plain_rows(*P, filter);
  } else {
    pack_spf(*P, filter, bank_optimize, reorder_out_channel);
  }
  return P;
}

void orc_pack_free(OrcPack* p) { delete p; }
void orc_pack_sizes(const OrcPack* p, int64_t* n) {
  n[0] = (int64_t)p->offsets.size(); n[1] = (int64_t)p->stage_len.size(); n[2] = (int64_t)p->position.size();
  n[3] = (int64_t)p->values.size(); n[4] = (int64_t)p->perm.size(); n[5] = p->nnz; n[6] = p->bank_oob; n[7] = p->stages;
}
const int32_t* orc_pack_offsets(const OrcPack* p) { return p->offsets.data(); }
const int32_t* orc_pack_stage_len(const OrcPack* p) { return p->stage_len.data(); }
const int32_t* orc_pack_position(const OrcPack* p) { return p->position.data(); }
const float* orc_pack_values(const OrcPack* p) { return p->values.data(); }
const int32_t* orc_pack_perm(const OrcPack* p) { return p->perm.data(); }

// spconv2d_utils.h:422-455  HostSpconv2d: decodes the keep-as-is format
void orc_host_spconv2d(const OrcPack* p, const float* input, float* output, int N, int H, int W, int pad, int stride,
                       int threads) {
  const int C = p->C, K = p->K, ks = p->ks, S = p->stages, T = p->tile_ic;
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
#pragma omp parallel for collapse(2) schedule(dynamic) num_threads(threads > 0 ? threads : 1)
  for (int n = 0; n < N; ++n)
    for (int oc = 0; oc < K; ++oc)
      for (int h = 0; h < OH; ++h)
        for (int w = 0; w < OW; ++w) {
          float* o = &output[(((size_t)n * K + oc) * OH + h) * OW + w];
          *o = 0.f;
          for (int sid = S * oc, t = 0; sid < S * (oc + 1); ++sid, ++t)
            for (int k = p->offsets[sid]; k < p->offsets[sid + 1]; ++k) {
              const int pos = p->position[k];
              const int y = pos & 7, x = (pos >> kBitS) & 7, ic = (pos >> (kBitS + kBitR)) + t * T;
              const int ih = h * stride + x, iw = w * stride + y;
              if (ih < pad || ih >= H + pad) continue;
              if (iw < pad || iw >= W + pad) continue;
              *o += input[(((size_t)n * C + ic) * H + (ih - pad)) * W + (iw - pad)] * p->values[k];
            }
        }
}

// spconv2d_utils.h:457-493 HostReorderSpconv2d generalised over the vector width: entry e of lane l in
// (group, stage) sits at 32*offsets[g*S+i] + (e/vec)*32*vec + l*vec + e%vec, which is the host decoder's
// start + k*32 + lane for vec = 1 (:475-476) and the kernel's start + k*32 + lane*4 + it for vec = 4
// (spconv2d_kernel.cu:96-100).  Result goes to output channel perm[oc] (:485, kernel.cu:148-153).
void orc_host_reorder_spconv2d(const OrcPack* p, const float* input, float* output, int N, int H, int W, int pad,
                               int stride, int threads) {
  const int C = p->C, K = p->K, ks = p->ks, S = p->stages, T = p->tile_ic, vec = p->vec;
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
#pragma omp parallel for collapse(2) schedule(dynamic) num_threads(threads > 0 ? threads : 1)
  for (int n = 0; n < N; ++n)
    for (int oc = 0; oc < K; ++oc)
      for (int h = 0; h < OH; ++h)
        for (int w = 0; w < OW; ++w) {
          float sum = 0;
          const int lane = oc % kLanes;
          for (int j = 0; j < S; ++j) {
            const int oid = oc / kLanes * S + j;
            const int len = p->offsets[oid + 1] - p->offsets[oid];
            const size_t start = (size_t)p->offsets[oid] * kLanes;
            for (int e = 0; e < len; ++e) {
              const size_t at = start + (size_t)(e / vec) * kLanes * vec + (size_t)lane * vec + e % vec;
              const int pos = p->position[at];
              const float v = p->values[at];
              const int y = pos & 7, x = (pos >> kBitS) & 7, ic = (pos >> (kBitS + kBitR)) + j * T;
              const int ih = h * stride + x, iw = w * stride + y;
              if (ih < pad || ih >= H + pad) continue;
              if (iw < pad || iw >= W + pad) continue;
              if (ic >= C) continue;  // Bank-SR pads name a bank, not a channel; their value is 0
              sum += input[(((size_t)n * C + ic) * H + (ih - pad)) * W + (iw - pad)] * v;
            }
          }
          output[(((size_t)n * K + p->perm[oc]) * OH + h) * OW + w] = sum;
        }
}

// ---- gfx950 layout (defined by this project; no reference counterpart) --------------------------
// Slots = K rounded up to a multiple of 128; slot i computes output channel order[i] (identity when
// order == NULL), padding slots hold -1.  Slots are taken G at a time (one group per wave of the HIP
// kernel).  Per (group, stage) one stream: for every position of the stage in (channel, row, column)
// order -- the scan order of spconv2d_utils.h:85-94 -- and every slot l of the group in ascending
// order, the non-zero weight with the position word of spconv2d_utils.h:91 plus l << 24; then
// (0, 0.0f) entries up to a multiple of 8.  grp_off is the running sum of the padded stream lengths.
struct OrcG950 {
  int C = 0, K = 0, ks = 0, tile_ic = 0, stages = 0, slots = 0, G = 0, groups = 0;
  std::vector<int32_t> grp_off, grp_nnz, position, order;
  std::vector<float> values;
};

OrcG950* orc_g950_pack(const float* filter, int C, int K, int ks, int tile_ic, int G, const int32_t* order) {
  OrcG950* P = new OrcG950;
  P->C = C; P->K = K; P->ks = ks; P->tile_ic = tile_ic; P->G = G;
  P->stages = (C - 1) / tile_ic + 1;
  P->slots = (K + 127) / 128 * 128;
  P->groups = P->slots / G;
  P->order.assign(P->slots, -1);
  for (int i = 0; i < K; ++i) P->order[i] = order ? order[i] : i;
  P->grp_off.push_back(0);
  const int kk = ks * ks;
  for (int grp = 0; grp < P->groups; ++grp)
    for (int st = 0; st < P->stages; ++st) {
      int n = 0;
      for (int j = st * tile_ic; j < std::min((st + 1) * tile_ic, C); ++j)
        for (int r = 0; r < ks; ++r)
          for (int s = 0; s < ks; ++s)
            for (int l = 0; l < G; ++l) {
              const int oc = P->order[grp * G + l];
              if (oc < 0) continue;
              const float v = filter[(size_t)oc * C * kk + (size_t)j * kk + r * ks + s];
              if (v != 0.f) {
                P->position.push_back(make_pos(s, r, j % tile_ic) + (l << 24));
                P->values.push_back(v);
                ++n;
              }
            }
      P->grp_nnz.push_back(n);
      for (int i = n; i % 8 != 0; ++i) {
        P->position.push_back(0);
        P->values.push_back(0.0f);
      }
      P->grp_off.push_back((int32_t)P->position.size());
    }
  return P;
}
void orc_g950_free(OrcG950* p) { delete p; }
void orc_g950_sizes(const OrcG950* p, int64_t* n) {
  n[0] = (int64_t)p->grp_off.size(); n[1] = (int64_t)p->grp_nnz.size(); n[2] = (int64_t)p->position.size();
  n[3] = p->slots; n[4] = p->stages;
}
const int32_t* orc_g950_grp_off(const OrcG950* p) { return p->grp_off.data(); }
const int32_t* orc_g950_grp_nnz(const OrcG950* p) { return p->grp_nnz.data(); }
const int32_t* orc_g950_position(const OrcG950* p) { return p->position.data(); }
const float* orc_g950_values(const OrcG950* p) { return p->values.data(); }
const int32_t* orc_g950_order(const OrcG950* p) { return p->order.data(); }

// Convolution straight from the gfx950 arrays: every output accumulates its slot's entries in stream
// order (stage by stage) -- the order the HIP kernel adds in, without its fused multiply-add.
void orc_g950_conv(const OrcG950* p, const float* input, float* output, int N, int H, int W, int pad, int stride,
                   int threads) {
  const int C = p->C, K = p->K, ks = p->ks, S = p->stages, T = p->tile_ic, G = p->G;
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
#pragma omp parallel for collapse(2) schedule(dynamic) num_threads(threads > 0 ? threads : 1)
  for (int n = 0; n < N; ++n)
    for (int grp = 0; grp < p->groups; ++grp) {
      std::vector<float> acc((size_t)G * OH * OW, 0.f);
      for (int st = 0; st < S; ++st)
        for (int e = p->grp_off[grp * S + st]; e < p->grp_off[grp * S + st + 1]; ++e) {
          const int pos = p->position[e];
          const float v = p->values[e];
          if (v == 0.f) continue;  // padding
          const int y = pos & 7, x = (pos >> kBitS) & 7, ic = ((pos >> (kBitS + kBitR)) & 0x3ffff) + st * T;
          const int l = (pos >> 24) & 0xff;
          const float* img = &input[((size_t)n * C + ic) * H * W];
          float* a = &acc[(size_t)l * OH * OW];
          for (int h = 0; h < OH; ++h) {
            const int ih = h * stride + x - pad;
            if (ih < 0 || ih >= H) continue;
            for (int w = 0; w < OW; ++w) {
              const int iw = w * stride + y - pad;
              if (iw < 0 || iw >= W) continue;
              a[h * OW + w] += img[(size_t)ih * W + iw] * v;
            }
          }
        }
      for (int l = 0; l < G; ++l) {
        const int oc = p->order[grp * G + l];
        if (oc < 0) continue;
        std::copy(acc.begin() + (size_t)l * OH * OW, acc.begin() + (size_t)(l + 1) * OH * OW,
                  &output[((size_t)n * K + oc) * OH * OW]);
      }
    }
}

// FNV-1a 64 over raw bytes; pass the previous return value as `h` to chain buffers
// (the known-answer table starts from 1469598103934665603, see oracle_py.py).
uint64_t orc_fnv1a(const void* data, int64_t len, uint64_t h) {
  const unsigned char* b = (const unsigned char*)data;
  for (int64_t i = 0; i < len; ++i) {
    h ^= b[i];
    h *= 0x100000001b3ULL;
  }
  return h;
}

int orc_max_threads() {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // extern "C"
