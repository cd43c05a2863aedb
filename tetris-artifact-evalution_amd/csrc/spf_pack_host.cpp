// Host-side weight preprocessing into the reference's packed layout ("SPF"), byte-identical to
// struct SparseFilter<float,int,int> (Tetris/spconv2d_utils.h:25-265) for every combination of its
// constructor arguments and its two compile-time macros (BANK_OPTIMIZE :80, REORDER_OUT_CHANNEL :66).
//
// The results are the reference's; the data structures are not.  Bank-SR (:99-199) is run on per-lane
// linked lists with per-bank queues instead of vector::erase scans, and the channel regrouping
// (:275-420) tests positions against a flat bitmap instead of a hash map.  Both greedy procedures
// are sequential by nature and stay on the host, where the reference has them.
#include <algorithm>
#include <set>

#include "common.h"

namespace tetris {
namespace {

constexpr int L = kRefLanes;

inline int32_t pos_word(int s, int r, int ic) { return s + (r << 3) + (ic << 6); }

struct Lane {  // one packed lane's entries for one stage, in (channel, row, column) order
  std::vector<int32_t> pos;
  std::vector<float> val;
};

void scan_lane(const float* filter, int C, int ks, int T, int src_oc, int c0, Lane& out) {
  const int kk = ks * ks;
  const int c1 = std::min(c0 + T, C);
  const float* w = filter + ((size_t)src_oc * C + c0) * kk;
  for (int j = c0; j < c1; ++j)
    for (int r = 0; r < ks; ++r)
      for (int s = 0; s < ks; ++s, ++w)
        if (*w != 0.f) {
          out.pos.push_back(pos_word(s, r, j % T));
          out.val.push_back(*w);
        }
}

// ---- Bank-SR for one (32-lane group, stage) -----------------------------------------------------
// in[l]: scan-order entries of lane l; out[l]: the order Bank-SR emits (with its zero-valued pads).
// Returns false when the reference would index its 32 bank flags with an entry index >= 32.
bool bank_sr(const Lane* in, Lane* out) {
  int longest = 0;
  for (int l = 0; l < L; ++l) longest = std::max(longest, (int)in[l].pos.size());
  if (longest == 0) return true;

  struct State {
    std::vector<int> next, prev;          // alive entries as a doubly linked list, sentinel = n
    std::vector<char> alive;
    std::vector<int> queue[L];            // entry indices per bank, ascending
    int head[L];
    int pads;
  };
  std::vector<State> st(L);
  for (int l = 0; l < L; ++l) {
    State& s = st[l];
    const int n = (int)in[l].pos.size();
    s.next.resize(n + 1);
    s.prev.resize(n + 1);
    s.alive.assign(n, 1);
    for (int i = 0; i <= n; ++i) {
      s.next[i] = i + 1 <= n ? i + 1 : 0;
      s.prev[i] = i ? i - 1 : n;
    }
    s.next[n] = 0;  // sentinel -> first
    for (int i = 0; i < n; ++i) s.queue[(in[l].pos[i] >> 6) % L].push_back(i);
    std::fill(s.head, s.head + L, 0);
    s.pads = longest - n;
    out[l].pos.reserve(longest);
    out[l].val.reserve(longest);
  }
  auto take = [&](int l, int i) {
    State& s = st[l];
    out[l].pos.push_back(in[l].pos[i]);
    out[l].val.push_back(in[l].val[i]);
    s.alive[i] = 0;
    s.next[s.prev[i]] = s.next[i];
    s.prev[s.next[i]] = s.prev[i];
  };

  std::vector<int32_t> flagged;  // taps selected through a free bank in this step
  for (int t = 0; t < longest; ++t) {
    int bank_flag[L] = {0};
    flagged.clear();
    int waiting[L], n_wait = 0;
    for (int l = 0; l < L; ++l) {
      State& s = st[l];
      const int n = (int)in[l].pos.size();
      int pick = n;  // smallest alive index that qualifies
      // (a) an entry whose tap another lane already reads in this step (broadcast)
      for (int32_t tap : flagged) {
        auto it = std::lower_bound(in[l].pos.begin(), in[l].pos.end(), tap);
        if (it != in[l].pos.end() && *it == tap) {
          const int i = (int)(it - in[l].pos.begin());
          if (s.alive[i]) pick = std::min(pick, i);
        }
      }
      if (pick == n) {  // (b) the first entry on a bank nobody uses yet
        int bank_of_pick = -1;
        for (int b = 0; b < L; ++b) {
          if (bank_flag[b]) continue;
          int& h = s.head[b];
          const std::vector<int>& q = s.queue[b];
          while (h < (int)q.size() && !s.alive[q[h]]) ++h;
          if (h < (int)q.size() && q[h] < pick) {
            pick = q[h];
            bank_of_pick = b;
          }
        }
        if (pick != n) {
          bank_flag[bank_of_pick] = 1;
          flagged.push_back(in[l].pos[pick]);
        }
      }
      if (pick != n) take(l, pick);
      else waiting[n_wait++] = l;
    }
    for (int w = 0; w < n_wait; ++w) {
      const int l = waiting[w];
      State& s = st[l];
      if (s.pads > 0) {
        for (int b = 0; b < L; ++b)
          if (!bank_flag[b]) {
            bank_flag[b] = 1;
            s.pads -= 1;
            out[l].pos.push_back(b << 6);
            out[l].val.push_back(0.0f);
            break;
          }
      } else {
        // The reference walks the remaining entries keeping `select`, and compares
        // bank_flag[select] -- indexed by the entry's list position -- with the bank flag of entry j.
        const int n = (int)in[l].pos.size();
        int sel_idx = -1, sel_at = -1;
        int j = 0;
        for (int i = s.next[n]; i != n; i = s.next[i], ++j) {
          const int bank = (in[l].pos[i] >> 6) % L;
          if (sel_idx == -1) {
            sel_idx = j;
            sel_at = i;
            continue;
          }
          if (sel_idx >= L) return false;
          if (bank_flag[sel_idx] > bank_flag[bank]) {
            sel_idx = j;
            sel_at = i;
          }
        }
        if (sel_at < 0) return false;  // cannot happen: a lane emits exactly `longest` items
        bank_flag[(in[l].pos[sel_at] >> 6) % L] += 1;
        take(l, sel_at);
      }
    }
  }
  return true;
}

// ---- output-channel regrouping (REORDER_OUT_CHANNEL) -------------------------------------------
void regroup_channels(const float* filter, int C, int K, int ks, int T, std::vector<int32_t>& perm) {
  const int S = (C - 1) / T + 1, kk = ks * ks;
  std::vector<int> cnt((size_t)K * S, 0);
  std::vector<std::vector<int32_t>> taps((size_t)K * S);  // position words with the absolute channel
  for (int o = 0; o < K; ++o)
    for (int j = 0; j < C; ++j)
      for (int r = 0; r < ks; ++r)
        for (int s = 0; s < ks; ++s)
          if (filter[((size_t)o * C + j) * kk + r * ks + s] != 0.f) {
            cnt[(size_t)o * S + j / T] += 1;
            taps[(size_t)o * S + j / T].push_back(pos_word(s, r, j));
          }

  typedef std::pair<int, int> Key;  // (-cost, first channel): ascending = highest cost first, then lowest l
  std::set<Key> waiting;
  std::vector<int> sub_end(K, 0);
  for (int l = 0; l < K; l += 8) {
    const int r = std::min(K, l + 8);
    int cost = 0;
    for (int st = 0; st < S; ++st) {
      int m = 0;
      for (int o = l; o < r; ++o) m = std::max(m, cnt[(size_t)o * S + st]);
      cost += m;
    }
    sub_end[l] = r;
    waiting.insert(Key(-cost, l));
  }

  perm.clear();
  std::vector<char> seen((size_t)C << 6, 0);
  std::vector<int32_t> seen_list;
  std::vector<int> cur_mx(S), cur_bank((size_t)S * L);
  while (!waiting.empty()) {
    std::fill(cur_mx.begin(), cur_mx.end(), 0);
    std::fill(cur_bank.begin(), cur_bank.end(), 0);
    for (int32_t p : seen_list) seen[p] = 0;
    seen_list.clear();
    size_t group_size = 0;

    auto absorb = [&](int l, int r) {  // UpdateBankCount + UpdateStageMX + append
      for (int o = l; o < r; ++o)
        for (int st = 0; st < S; ++st) {
          for (int32_t p : taps[(size_t)o * S + st])
            if (!seen[p]) {
              seen[p] = 1;
              seen_list.push_back(p);
              cur_bank[(size_t)st * L + (p >> 6) % L] += 1;
            }
          cur_mx[st] = std::max(cur_mx[st], cnt[(size_t)o * S + st]);
        }
      for (int o = l; o < r; ++o) perm.push_back(o);
      group_size += r - l;
    };
    auto cost_of = [&](int l, int r) -> float {
      float total = 0;
      for (int st = 0; st < S; ++st) {
        int bank[L];
        for (int b = 0; b < L; ++b) bank[b] = cur_bank[(size_t)st * L + b];
        int mx = 0;
        for (int o = l; o < r; ++o) {
          mx = std::max(mx, cnt[(size_t)o * S + st]);
          for (int32_t p : taps[(size_t)o * S + st])
            if (!seen[p]) bank[(p >> 6) % L] += 1;
        }
        const int mx_bank = *std::max_element(bank, bank + L);
        const int padding = std::abs(mx - cur_mx[st]);
        total += std::max(mx_bank - std::max(mx, cur_mx[st]), padding);
      }
      return total;
    };

    const int seed = waiting.begin()->second;
    waiting.erase(waiting.begin());
    absorb(seed, sub_end[seed]);
    while (!waiting.empty() && group_size < (size_t)L) {
      float best_cost = 1e18;
      Key best(0, -1);
      for (const Key& c : waiting) {
        const float v = cost_of(c.second, sub_end[c.second]);
        if (v < best_cost) {
          best_cost = v;
          best = c;
        }
      }
      waiting.erase(best);
      absorb(best.second, sub_end[best.second]);
    }
  }
}

}  // namespace

int spf_pack_host(const float* filter, int C, int K, int ks, int T, bool apply_reorder, bool apply_vectorize,
                  unsigned flags, tetris_spf* out) {
  if (!filter || !out) return fail(TETRIS_EINVAL, "null argument");
  if (C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs || T <= 0)
    return fail(TETRIS_EINVAL, "bad filter shape C=%d K=%d ks=%d tile_ic=%d (ks <= %d)", C, K, ks, T, kMaxKs);
  const int S = (C - 1) / T + 1, kk = ks * ks;
  out->C = C; out->K = K; out->ks = ks; out->tile_ic = T;
  out->nnz = 0;
  out->offsets.assign(1, 0);
  out->stage_len.clear();
  out->position.clear();
  out->values.clear();
  out->oc_permutation.resize(K);
  for (int o = 0; o < K; ++o) out->oc_permutation[o] = o;

  if (!apply_reorder) {  // rows kept as they are: one run per (channel, stage)
    out->offsets.reserve((size_t)K * S + 1);
    for (int o = 0; o < K; ++o)
      for (int st = 0; st < S; ++st) {
        Lane run;
        scan_lane(filter, C, ks, T, o, st * T, run);
        out->position.insert(out->position.end(), run.pos.begin(), run.pos.end());
        out->values.insert(out->values.end(), run.val.begin(), run.val.end());
        out->offsets.push_back((int32_t)out->position.size());
      }
    out->nnz = (int64_t)out->position.size();
    return TETRIS_OK;
  }

  if (flags & TETRIS_REORDER_OUT_CHANNEL) regroup_channels(filter, C, K, ks, T, out->oc_permutation);
  const int groups = (K - 1) / L + 1;
  const int vec = apply_vectorize ? 4 : 1;
  out->offsets.assign((size_t)groups * S + 1, 0);
  out->stage_len.assign((size_t)groups * L * S, 0);
  (void)kk;

  for (int g = 0; g < groups; ++g)
    for (int st = 0; st < S; ++st) {
      Lane scan[L], ordered[L];
      for (int l = 0; l < L && g * L + l < K; ++l)
        scan_lane(filter, C, ks, T, out->oc_permutation[g * L + l], st * T, scan[l]);
      const Lane* lanes = scan;
      if (flags & TETRIS_BANK_OPTIMIZE) {
        if (!bank_sr(scan, ordered))
          return fail(TETRIS_EUNSUPPORTED,
                      "Bank-SR reads its bank flags out of range for this filter (group %d, stage %d): the "
                      "reference's result is undefined",
                      g, st);
        lanes = ordered;
      }
      int longest = 0;
      for (int l = 0; l < L && g * L + l < K; ++l) {
        const int n = (int)lanes[l].pos.size();
        longest = std::max(longest, (n + vec - 1) / vec * vec);
        out->stage_len[((size_t)g * S + st) * L + l] = n;
      }
      const size_t oid = (size_t)g * S + st;
      out->offsets[oid + 1] = out->offsets[oid] + longest;
      const size_t base = out->position.size();
      out->position.resize(base + (size_t)longest * L, 0);
      out->values.resize(base + (size_t)longest * L, 0.0f);
      for (int l = 0; l < L; ++l) {
        const int n = (int)lanes[l].pos.size();
        for (int e = 0; e < n; ++e) {
          const size_t at = base + (size_t)(e / vec) * L * vec + (size_t)l * vec + e % vec;
          out->position[at] = lanes[l].pos[e];
          out->values[at] = lanes[l].val[e];
        }
      }
    }
  return TETRIS_OK;
}

// What the device code that reads a SparseFilter's arrays relies on: offsets_ starts at 0 and never decreases
// (spconv2d_utils.h:45-47, :213-216), every step of the interleaved layout is a multiple of the vector width (:209-212),
// and the entries the offsets span -- `lanes` per unit of offset -- fit the arrays (`capacity` entries; 0: not known).
int check_spf_offsets(const int32_t* offsets, int n_off, int lanes, int vec, long long capacity) {
  if (!offsets || n_off < 1) return fail(TETRIS_EINVAL, "no offsets");
  if (offsets[0] != 0) return fail(TETRIS_EINVAL, "offsets[0] is %d, not 0: not a packed filter", offsets[0]);
  for (int i = 1; i < n_off; ++i) {
    if (offsets[i] < offsets[i - 1])
      return fail(TETRIS_EINVAL, "offsets decrease at %d (%d after %d): wrong out_channel, tile_ic or vector width?", i,
                  offsets[i], offsets[i - 1]);
    if (vec > 1 && (offsets[i] - offsets[i - 1]) % vec != 0)
      return fail(TETRIS_EINVAL, "stream %d holds %d steps, not a multiple of the vector width %d", i - 1,
                  offsets[i] - offsets[i - 1], vec);
  }
  const long long n_ent = (long long)lanes * offsets[n_off - 1];
  if (n_ent > (1ll << 31)) return fail(TETRIS_EINVAL, "offsets end at %lld entries: not a packed filter", n_ent);
  if (capacity > 0 && n_ent > capacity)
    return fail(TETRIS_EINVAL, "offsets span %lld entries, the arrays hold %lld: wrong out_channel, tile_ic or vector width?",
                n_ent, capacity);
  return TETRIS_OK;
}

}  // namespace tetris

extern "C" int tetris_spf_check_offsets(const int32_t* h_offsets, int64_t n_offsets, int vec_width, int64_t n_entries) {
  if (n_offsets < 1 || n_offsets > (1ll << 28) || (vec_width != 0 && vec_width != 1 && vec_width != 4) || n_entries < 0)
    return tetris::fail(TETRIS_EINVAL, "bad argument");
  return tetris::check_spf_offsets(h_offsets, (int)n_offsets, vec_width == 0 ? 1 : tetris::kRefLanes, vec_width, n_entries);
}
