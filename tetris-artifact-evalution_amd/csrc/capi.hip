// extern "C" layer of libtetris_spconv2d.so: handles, launch, the reference-shaped host entry points
// (CudaSparseConv2d, Tetris/spconv2d.cc:332-367; SparseConv2d_SPF, Tetris/spf.cc:22-93) and the path's
// small utilities (Tetris/tensor_utils.cc:17-34, :55-82).
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>

#include <algorithm>
#include <atomic>

#include "common.h"

namespace tetris {

namespace {
thread_local std::string g_error;

std::mutex g_registry_mu;
std::map<const void*, tetris_spf*> g_registry;  // d_values of every live tetris_spf -> its handle
}  // namespace

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return code;
}

namespace {

template <typename T>
int upload(const std::vector<T>& v, T** d) {
  *d = nullptr;
  const size_t bytes = std::max<size_t>(v.size(), 1) * sizeof(T);
  TETRIS_HIP(hipMalloc(d, bytes));
  if (!v.empty()) TETRIS_HIP(hipMemcpy(*d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return TETRIS_OK;
}

// The launch plan of (input shape, tile) for pack `p`: looked up, or -- when `create` allows it -- made (geometry,
// bound entries: one device allocation and one small kernel on `stream`) and remembered.
int find_plan(tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile* tile, hipStream_t stream,
              bool create, Plan* out) {
  const bool given = tile && tile->lanes_w > 0;
  // a NULL tile is remembered under a key of zeros, so that the library's own choice is made once per shape
  const tetris_tile none{};
  const tetris_tile& kt = given ? *tile : none;
  const int key[11] = {N, H, W, stride, pad, kt.lanes_w, kt.quads, kt.oc_per_wave, kt.waves, kt.tile_ic, kt.csplit};
  {
    std::lock_guard<std::mutex> lock(p->mu);
    for (size_t i = p->plans.size(); i-- > 0;)
      if (memcmp(p->plans[i].key, key, sizeof key) == 0) {
        *out = p->plans[i];
        return TETRIS_OK;
      }
  }
  if (!create)
    return fail(TETRIS_ENOTFOUND, "no launch plan for N=%d H=%d W=%d stride=%d pad=%d with this tile: call "
                "tetris_g950_prepare first", N, H, W, stride, pad);
  tetris_tile t{};
  if (given) {
    t = *tile;
  } else {
    int rc = choose_tile(N, H, W, p->C, p->K, p->ks, stride, pad, &t);
    if (rc) return rc;
  }
  if (t.tile_ic != p->tile_ic || t.oc_per_wave != p->g)
    return fail(TETRIS_EINVAL, "tile (tile_ic=%d, oc_per_wave=%d) does not match the pack (tile_ic=%d, oc_per_wave=%d)",
                t.tile_ic, t.oc_per_wave, p->tile_ic, p->g);
  Plan plan;
  int rc = make_geom(p, N, H, W, stride, pad, t, &plan.geom);
  if (rc) return rc;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
    return fail(TETRIS_EINVAL, "the first launch of a shape allocates: call tetris_g950_prepare before capturing");
  rc = g950_bind(p, plan.geom, geom_walks_pairs(plan.geom), stream, &plan.entries, &plan.grp_off, &plan.grp_pair,
                 &plan.geom.heads_off);
  if (rc) return rc;
  memcpy(plan.key, key, sizeof key);
  std::lock_guard<std::mutex> lock(p->mu);
  if (p->plans.size() >= 64) p->plans.erase(p->plans.begin());
  p->plans.push_back(plan);
  *out = plan;
  return TETRIS_OK;
}

// scratch of a split layer: the tickets, then csplit copies of the output
size_t partial_bytes_of(const Geom& g) {
  return g.csplit > 1 ? (size_t)kTicketBytes + sizeof(float) * (size_t)g.csplit * g.N * g.K * g.OH * g.OW : 0;
}

// Partial-sum buffer of a split layer: one per (pack, stream), so that launches of one pack on different streams do
// not share it.  A buffer that has to grow is replaced, and the old one is kept until the pack is destroyed: a HIP
// graph captured earlier may still hold its address.
int partial_buffer(tetris_g950* p, hipStream_t stream, size_t need, bool grow, float** out) {
  std::lock_guard<std::mutex> lock(p->mu);
  tetris_g950::Partial& b = p->partial[stream];
  if (b.bytes < need) {
    if (!grow)
      return fail(TETRIS_ENOTFOUND, "no partial-sum buffer of %zu bytes on this stream: call tetris_g950_prepare first",
                  need);
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return fail(TETRIS_EINVAL, "this launch would allocate its partial-sum buffer: call tetris_g950_prepare before "
                  "capturing");
    bool same_xcd = false;  // asked here, where allocating and synchronising is allowed, so that launches find the answer
    int rc = same_xcd_by_residue(&same_xcd);
    if (rc) return rc;
    float* d = nullptr;
    TETRIS_HIP(hipMalloc(&d, need));
    // the tickets start at zero; the kernels leave them at zero (this is not under capture: see above)
    hipError_t e = hipMemsetAsync(d, 0, kTicketBytes, stream);
    if (e != hipSuccess) {
      (void)hipFree(d);
      return fail(TETRIS_EHIP, "clearing the tickets failed: %s", hipGetErrorString(e));
    }
    if (b.ptr) p->retired.push_back(b.ptr);
    b.ptr = d;
    b.bytes = need;
  }
  *out = b.ptr;
  return TETRIS_OK;
}

int run_launch(tetris_g950* p, const float* d_in, float* d_out, int N, int H, int W, int stride, int pad,
               const tetris_tile* tile, hipStream_t stream, int act = 0) {
  if (!p || !d_in || !d_out) return fail(TETRIS_EINVAL, "null argument");
  Plan plan;
  int rc = find_plan(p, N, H, W, stride, pad, tile, stream, true, &plan);
  if (rc) return rc;
  float* d_partial = nullptr;
  if (plan.geom.csplit > 1) {
    rc = partial_buffer(p, stream, partial_bytes_of(plan.geom), true, &d_partial);
    if (rc) return rc;
  }
  return launch_conv(plan.geom, d_in, d_out, d_partial, plan.entries, plan.grp_off, plan.grp_pair, p->d_oc_order, act,
                     stream);
}

// ---- scratch of the entry point that allocates nothing ------------------------------------------------------------
// Tickets and partial sums of split layers for callers that cannot allocate.  One array per GPU, held until the
// process ends (zero when the code object is loaded: the tickets start at zero, and every launch leaves them so);
// every call on a GPU shares it, so calls that overlap in time on one GPU race.
constexpr size_t kStaticScratchBytes = (size_t)TETRIS_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) __attribute__((used)) float scratch[kStaticScratchBytes / sizeof(float)];

std::atomic<size_t> g_scratch_limit{kStaticScratchBytes};  // bytes of the array the entry point may use
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, looked up once per device

int static_scratch(float** out) {
  int dev = -1;
  TETRIS_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(TETRIS_EINVAL, "device %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    TETRIS_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(TETRIS_EHIP, "hipGetSymbolAddress returned a null address for the scratch array");
    bool same_xcd = false;  // the placement probe of split layers, made here so that launches find the answer ready
    const int rc = same_xcd_by_residue(&same_xcd);
    if (rc) return rc;
    g_scratch_ptr[dev] = static_cast<float*>(ptr);
  }
  *out = g_scratch_ptr[dev];
  return TETRIS_OK;
}

int time_launches(tetris_g950* p, const float* d_in, float* d_out, int N, int H, int W, int stride, int pad,
                  const tetris_tile* tile, hipStream_t stream, int warm, int repeat, float* ms_out) {
  if (repeat <= 0 || warm < 0) return fail(TETRIS_EINVAL, "bad warm/repeat");
  hipEvent_t a = nullptr, b = nullptr;
  auto done = [&](int code) {
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
    return code;
  };
#define HIPT(call)                                                                                          \
  do {                                                                                                      \
    hipError_t e_ = (call);                                                                                 \
    if (e_ != hipSuccess)                                                                                   \
      return done(fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__, hipGetErrorString(e_))); \
  } while (0)
  HIPT(hipEventCreate(&a));
  HIPT(hipEventCreate(&b));
  for (int i = 0; i < warm; ++i) {
    const int rc = run_launch(p, d_in, d_out, N, H, W, stride, pad, tile, stream);
    if (rc) return done(rc);
  }
  HIPT(hipStreamSynchronize(stream));
  float ms = 0;
  if (options() & TETRIS_OPT_COLD_TIMING) {
    // every timed launch starts with cold caches, as a layer between other layers does: the mean of `repeat` single
    // launches, each between its own pair of events, with a cache-evicting pass before it (not timed)
    for (int i = 0; i < repeat; ++i) {
      int rc = sweep_caches(stream);
      if (rc) return done(rc);
      HIPT(hipEventRecord(a, stream));
      rc = run_launch(p, d_in, d_out, N, H, W, stride, pad, tile, stream);
      if (rc) return done(rc);
      HIPT(hipEventRecord(b, stream));
      HIPT(hipEventSynchronize(b));
      float one = 0;
      HIPT(hipEventElapsedTime(&one, a, b));
      ms += one;
    }
  } else {
    HIPT(hipEventRecord(a, stream));
    for (int i = 0; i < repeat; ++i) {
      const int rc = run_launch(p, d_in, d_out, N, H, W, stride, pad, tile, stream);
      if (rc) return done(rc);
    }
    HIPT(hipEventRecord(b, stream));
    HIPT(hipEventSynchronize(b));
    HIPT(hipEventElapsedTime(&ms, a, b));
  }
#undef HIPT
  if (ms_out) *ms_out = ms / repeat;
  return done(TETRIS_OK);
}

// ---- the reference layout's device arrays as the source of a convolution ------------------------------------------
// A view remembers, for one set of array addresses, the content hash it was built from, the dense filter decoded from
// the arrays (device memory), and the kernel packs and tiles made from it.  At most kMaxViews live at a time.
struct SpfView {
  const void* ptrs[4];  // offsets, permutation, position, values
  int C, K, ks, tile_ic, vec;
  unsigned long long hash = 0;
  float* d_filter = nullptr;
  std::vector<int32_t> order;                              // oc_permutation copied to the host: the packs' slot order
  std::map<std::array<int, 2>, tetris_g950*> packs;        // by (tile_ic of the kernel, oc_per_wave)
  std::map<std::array<int, 5>, tetris_tile> tiles;         // by (N, H, W, stride, pad): the library's choice, made once
  void clear() {
    for (auto& kv : packs) tetris_g950_destroy(kv.second);
    packs.clear();
    tiles.clear();
    if (d_filter) (void)hipFree(d_filter);
    d_filter = nullptr;
  }
};
constexpr size_t kMaxViews = 16;
std::mutex g_views_mu;
std::vector<SpfView*> g_views;  // most recently used last
unsigned long long* g_hash_scratch = nullptr;

void drop_views(const void* d_values) {
  std::lock_guard<std::mutex> lock(g_views_mu);
  for (size_t i = g_views.size(); i-- > 0;)
    if (g_views[i]->ptrs[3] == d_values) {
      g_views[i]->clear();
      delete g_views[i];
      g_views.erase(g_views.begin() + (long)i);
    }
}

// The kernel pack (and tile) for a convolution whose weights are the arrays at these addresses, rebuilt when the
// arrays' content has changed since the view was made.  The caller holds g_views_mu, and keeps it until the launch
// that uses the pack has been issued: a view (and its packs) can only be evicted or dropped under that lock.
// Before any kernel touches the arrays the offsets are copied to the host and checked (non-negative, non-decreasing,
// the entries they span within `capacity` when the caller gave one), so that a wrong K, tile_ic or vector width is
// an error code and not an out-of-bounds read on the device.  Hashing reads the arrays once and synchronises `stream`;
// with TETRIS_OPT_TRUST_SPF_ARRAYS a view that exists for these addresses is used as it is (no read-back, no
// synchronisation) until tetris_spf_invalidate or tetris_spf_destroy drops it.
int view_pack(const int32_t* d_offsets, const int32_t* d_perm, const int32_t* d_position, const float* d_values, int N,
              int H, int W, int C, int K, int ks, int stride, int pad, int tile_ic, int vec, long long capacity,
              const tetris_tile* tile, hipStream_t stream, tetris_g950** pack_out, tetris_tile* tile_out) {
  if (!d_offsets || !d_position || !d_values || (vec != 0 && !d_perm)) return fail(TETRIS_EINVAL, "null argument");
  if (C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs || tile_ic <= 0 || (vec != 0 && vec != 1 && vec != 4))
    return fail(TETRIS_EINVAL, "bad filter shape C=%d K=%d ks=%d tile_ic=%d vector width=%d", C, K, ks, tile_ic, vec);
  if (capacity < 0) return fail(TETRIS_EINVAL, "negative entry capacity");
  auto find = [&]() -> SpfView* {  // the view of these addresses and this shape, if there is one
    for (SpfView* c : g_views)
      if (c->ptrs[0] == d_offsets && c->ptrs[1] == d_perm && c->ptrs[2] == d_position && c->ptrs[3] == d_values &&
          c->C == C && c->K == K && c->ks == ks && c->tile_ic == tile_ic && c->vec == vec)
        return c;
    return nullptr;
  };
  SpfView* v = find();
  const bool trusted = v && v->d_filter && (options() & TETRIS_OPT_TRUST_SPF_ARRAYS);
  unsigned long long hash = v ? v->hash : 0;
  int rc = TETRIS_OK;
  if (!trusted) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return fail(TETRIS_EINVAL, "this entry point reads the arrays back (a synchronisation): it cannot be captured; "
                  "capture tetris_spconv2d_launch on a tetris_g950 instead");
    const int stages = (C - 1) / tile_ic + 1;
    const long long n_off_ll = (long long)(vec == 0 ? K : (K + kRefLanes - 1) / kRefLanes) * stages + 1;
    if (n_off_ll > (1ll << 28)) return fail(TETRIS_EINVAL, "%lld stream offsets: not a packed filter", n_off_ll);
    const int n_off = (int)n_off_ll;
    const int lanes = vec == 0 ? 1 : kRefLanes;
    std::vector<int32_t> h_off((size_t)n_off);
    TETRIS_HIP(hipMemcpyAsync(h_off.data(), d_offsets, sizeof(int32_t) * (size_t)n_off, hipMemcpyDeviceToHost, stream));
    TETRIS_HIP(hipStreamSynchronize(stream));
    rc = check_spf_offsets(h_off.data(), n_off, lanes, vec, capacity);
    if (rc) return rc;
    const long long n_ent = (long long)lanes * h_off[n_off - 1];
    if (!g_hash_scratch) TETRIS_HIP(hipMalloc(&g_hash_scratch, 16));
    rc = spf_arrays_hash(d_offsets, n_off, d_perm, vec == 0 ? 0 : K, d_position, d_values, n_ent, g_hash_scratch, stream,
                         &hash);
    if (rc) return rc;
    hash ^= 0x5bd1e995ull * (unsigned long long)(C * 131 + ks) + (unsigned long long)tile_ic * 7919ull + (unsigned)vec;
  }
  if (v) g_views.erase(std::find(g_views.begin(), g_views.end(), v));  // moves to the most-recently-used end below
  if (!v) {
    v = new SpfView;
    v->ptrs[0] = d_offsets; v->ptrs[1] = d_perm; v->ptrs[2] = d_position; v->ptrs[3] = d_values;
    v->C = C; v->K = K; v->ks = ks; v->tile_ic = tile_ic; v->vec = vec;
    v->hash = ~hash;
  }
  g_views.push_back(v);
  while (g_views.size() > kMaxViews) {
    g_views.front()->clear();
    delete g_views.front();
    g_views.erase(g_views.begin());
  }
  if (v->hash != hash || !v->d_filter) {  // new, or rewritten in place since the view was made: decode again
    v->clear();
    TETRIS_HIP(hipMalloc(&v->d_filter, sizeof(float) * (size_t)C * K * ks * ks));
    rc = spf_arrays_decode(d_offsets, d_perm, d_position, d_values, v->d_filter, C, K, ks, tile_ic, vec, stream);
    if (rc) return rc;
    v->order.assign(K, 0);
    if (vec != 0) {
      TETRIS_HIP(hipMemcpyAsync(v->order.data(), d_perm, sizeof(int32_t) * K, hipMemcpyDeviceToHost, stream));
      TETRIS_HIP(hipStreamSynchronize(stream));
      std::vector<char> seen(K, 0);
      for (int k = 0; k < K; ++k) {
        if (v->order[k] < 0 || v->order[k] >= K || seen[v->order[k]])
          return fail(TETRIS_EINVAL, "oc_permutation is not a permutation of 0..%d", K - 1);
        seen[v->order[k]] = 1;
      }
    } else {
      for (int k = 0; k < K; ++k) v->order[k] = k;
    }
    v->hash = hash;
  }
  tetris_tile t{};
  if (tile && tile->lanes_w > 0) {
    t = *tile;
  } else {
    const std::array<int, 5> key{N, H, W, stride, pad};
    auto it = v->tiles.find(key);
    if (it == v->tiles.end()) {
      rc = choose_tile(N, H, W, C, K, ks, stride, pad, &t);
      if (rc) return rc;
      it = v->tiles.emplace(key, t).first;
    }
    t = it->second;
  }
  const std::array<int, 2> pkey{t.tile_ic, t.oc_per_wave};
  auto it = v->packs.find(pkey);
  if (it == v->packs.end()) {
    // slots in the order of the arrays' own oc_permutation: the caller's channel regrouping is kept
    tetris_g950* p = nullptr;
    rc = tetris_g950_create_device(v->d_filter, C, K, ks, t.tile_ic, t.oc_per_wave, v->order.data(), stream, &p);
    if (rc) return rc;
    it = v->packs.emplace(pkey, p).first;
  }
  *pack_out = it->second;
  *tile_out = t;
  return TETRIS_OK;
}

// Shared body of the two host-to-host entry points.
// The fixed tile of the spf entry point, the counterpart of the reference's one instantiation <3, 1, 128, 2, 4>
// (Tetris/spf.cc:59-60): four waves of eight channels, one quad, eight staged channels, lanes across a quarter of the
// output width (at most 16).  A shape it cannot run falls back to the library's choice.
tetris_tile fixed_spf_tile(int N, int H, int W, int C, int K, int ks, int stride, int pad) {
  tetris_tile t{};
  const int OW = out_extent(W, pad, ks, stride);
  t.lanes_w = std::max(1, std::min(16, ceil_div(OW, 4)));
  t.quads = 1; t.oc_per_wave = 8; t.waves = 4; t.tile_ic = std::min(8, C);
  tetris_g950 shape;
  shape.C = C; shape.K = K; shape.ks = ks; shape.tile_ic = t.tile_ic; shape.g = t.oc_per_wave;
  shape.stages = ceil_div(C, t.tile_ic);
  shape.slots = ceil_div(K, kSlotPad) * kSlotPad;
  Geom g;
  if (make_geom(&shape, N, H, W, stride, pad, t, &g) != TETRIS_OK) (void)choose_tile(N, H, W, C, K, ks, stride, pad, &t);
  return t;
}

// The Baseline rung's tile: the fixed tile with ONE output channel per wave, so that a wave walks one stream per (output
// channel, stage) in file order -- the keep-as-is runs of the CSR-like arrays, no channels grouped into a stream and
// no channel order chosen -- where the SPF rung's waves walk the merged, position-sorted stream of eight channels.
tetris_tile baseline_tile(tetris_tile t, int N, int H, int W, int C, int K, int ks, int stride, int pad) {
  tetris_tile b = t;
  b.oc_per_wave = 1;
  tetris_g950 shape;
  shape.C = C; shape.K = K; shape.ks = ks; shape.tile_ic = b.tile_ic; shape.g = b.oc_per_wave;
  shape.stages = ceil_div(C, b.tile_ic);
  shape.slots = ceil_div(K, kSlotPad) * kSlotPad;
  Geom g;
  return make_geom(&shape, N, H, W, stride, pad, b, &g) == TETRIS_OK ? b : t;
}

// Shared body of the two host-to-host entry points.  spf_path: the reference's SparseConv2d_SPF (Tetris/spf.cc:22-93):
// SparseFilter with TILE_IC = 128 and apply_reorder = true whatever the caller passed (:43-44), its device arrays handed
// to the launcher, one fixed tile.
// baseline: the reference's SparseConv2d_Baseline (Tetris/baseline.cc:22-93): SparseFilter with TILE_IC = 128 and
// apply_reorder = false (the keep-as-is, CSR-like arrays of spconv2d_utils.h:38-61) handed to the launcher, the same
// fixed tile with one output channel per wave (baseline_tile): one stream per (output channel, stage), as the
// reference's baseline kernel walks one run per (thread = output channel, stage) (ablation_kernel.cu:76-98).
int conv_host(const float* h_in, const float* h_filter, float* h_out, int N, int H, int W, int C, int K, int ks,
              int stride, int pad, hipStream_t stream, bool apply_reorder, bool spf_path, unsigned spf_flags,
              float* ms_out, bool baseline = false) {
  if (!h_in || !h_filter || !h_out) return fail(TETRIS_EINVAL, "null argument");
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs || stride <= 0 || pad < 0)
    return fail(TETRIS_EINVAL, "bad conv shape");
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
  if (OH <= 0 || OW <= 0) return fail(TETRIS_EINVAL, "empty output");
  tetris_tile tile{};
  tetris_g950* pack = nullptr;   // owned here (the normal path)
  tetris_spf* spf = nullptr;     // owned here (the spf path; its view owns the pack)
  float *d_in = nullptr, *d_out = nullptr;
  const size_t in_bytes = sizeof(float) * (size_t)N * C * H * W, out_bytes = sizeof(float) * (size_t)N * K * OH * OW;
  std::unique_lock<std::mutex>* held = nullptr;
  auto done = [&](int code) {
    if (held && held->owns_lock()) held->unlock();  // tetris_spf_destroy drops the views under the same lock
    if (d_in) (void)hipFree(d_in);
    if (d_out) (void)hipFree(d_out);
    tetris_g950_destroy(pack);
    tetris_spf_destroy(spf);
    return code;
  };
  int rc;
  tetris_g950* run = nullptr;
  // the spf path runs on a pack its view owns: the views' lock is held until the launches have been issued
  std::unique_lock<std::mutex> views_lock(g_views_mu, std::defer_lock);
  held = &views_lock;
  if (spf_path) {
    rc = tetris_spf_create(h_filter, C, K, ks, 128, baseline ? 0 : 1, 1, spf_flags, &spf);
    if (rc) return done(rc);
    tetris_spf_arrays a{};
    rc = tetris_spf_device_arrays(spf, &a);
    if (rc) return done(rc);
    tetris_tile fixed = fixed_spf_tile(N, H, W, C, K, ks, stride, pad);
    if (baseline) fixed = baseline_tile(fixed, N, H, W, C, K, ks, stride, pad);
    views_lock.lock();
    rc = view_pack(a.offsets, baseline ? nullptr : a.oc_permutation, a.position, a.values, N, H, W, C, K, ks, stride, pad,
                   128, baseline ? 0 : 4, a.n_values, &fixed, stream, &run, &tile);
    if (rc) return done(rc);
  } else {
    rc = choose_tile(N, H, W, C, K, ks, stride, pad, &tile);
    if (rc) return done(rc);
    // apply_reorder: the reference regroups output channels for its warps (ReorderOutChannel); the kernel here
    // gets the order that balances its own waves instead.  The results do not depend on the order.
    std::vector<int32_t> order;
    if (apply_reorder) {
      order.resize(K);
      rc = balance_oc_order(h_filter, C, K, ks, tile, order.data());
      if (rc) return done(rc);
    }
    rc = tetris_g950_create(h_filter, C, K, ks, tile.tile_ic, tile.oc_per_wave, apply_reorder ? order.data() : nullptr,
                            stream, &pack);
    if (rc) return done(rc);
    run = pack;
  }
#define HIPD(call)                                                                                          \
  do {                                                                                                      \
    hipError_t e_ = (call);                                                                                 \
    if (e_ != hipSuccess)                                                                                   \
      return done(fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__, hipGetErrorString(e_))); \
  } while (0)
  HIPD(hipMalloc(&d_in, in_bytes));
  HIPD(hipMalloc(&d_out, out_bytes));
  HIPD(hipMemcpyAsync(d_in, h_in, in_bytes, hipMemcpyHostToDevice, stream));
  float ms = 0;
  rc = time_launches(run, d_in, d_out, N, H, W, stride, pad, &tile, stream, 30, 100, &ms);
  if (views_lock.owns_lock()) views_lock.unlock();
  if (rc) return done(rc);
  HIPD(hipMemcpyAsync(h_out, d_out, out_bytes, hipMemcpyDeviceToHost, stream));
  HIPD(hipStreamSynchronize(stream));
#undef HIPD
  if (ms_out) *ms_out = ms;
  return done(TETRIS_OK);
}

}  // namespace
}  // namespace tetris

using namespace tetris;

extern "C" {

const char* tetris_last_error(void) { return g_error.c_str(); }
const char* tetris_version(void) { return "tetris-spconv2d gfx950 0.1"; }

// Device copies of the five arrays are made on first use, so that packing alone needs no GPU.
static int spf_ensure_device(tetris_spf* f) {
  std::lock_guard<std::mutex> lock(f->mu);
  if (f->d_values) return TETRIS_OK;
  int rc = upload(f->offsets, &f->d_offsets);
  if (rc == TETRIS_OK) rc = upload(f->stage_len, &f->d_stage_len);
  if (rc == TETRIS_OK) rc = upload(f->position, &f->d_position);
  if (rc == TETRIS_OK) rc = upload(f->oc_permutation, &f->d_oc_permutation);
  float* d_values = nullptr;
  if (rc == TETRIS_OK) rc = upload(f->values, &d_values);
  if (rc != TETRIS_OK) {
    if (f->d_offsets) (void)hipFree(f->d_offsets);
    if (f->d_stage_len) (void)hipFree(f->d_stage_len);
    if (f->d_position) (void)hipFree(f->d_position);
    if (f->d_oc_permutation) (void)hipFree(f->d_oc_permutation);
    f->d_offsets = f->d_stage_len = f->d_position = f->d_oc_permutation = nullptr;
    return rc;
  }
  f->d_values = d_values;
  std::lock_guard<std::mutex> rlock(g_registry_mu);
  g_registry[f->d_values] = f;
  return TETRIS_OK;
}

int tetris_spf_create(const float* h_filter, int C, int K, int ks, int tile_ic, int apply_reorder, int apply_vectorize,
                      unsigned flags, tetris_spf** out) {
  if (!out) return fail(TETRIS_EINVAL, "null argument");
  tetris_spf* f = new tetris_spf;
  int rc = spf_pack_host(h_filter, C, K, ks, tile_ic, apply_reorder != 0, apply_vectorize != 0, flags, f);
  if (rc != TETRIS_OK) {
    delete f;
    return rc;
  }
  f->vec = apply_reorder ? (apply_vectorize ? 4 : 1) : 0;
  *out = f;
  return TETRIS_OK;
}

void tetris_spf_destroy(tetris_spf* f) {
  if (!f) return;
  if (f->d_values) {
    std::lock_guard<std::mutex> lock(g_registry_mu);
    auto it = g_registry.find(f->d_values);
    if (it != g_registry.end() && it->second == f) g_registry.erase(it);
  }
  drop_views(f->d_values);
  if (f->d_offsets) (void)hipFree(f->d_offsets);
  if (f->d_stage_len) (void)hipFree(f->d_stage_len);
  if (f->d_position) (void)hipFree(f->d_position);
  if (f->d_values) (void)hipFree(f->d_values);
  if (f->d_oc_permutation) (void)hipFree(f->d_oc_permutation);
  delete f;
}

int tetris_spf_host_arrays(const tetris_spf* f, tetris_spf_arrays* o) {
  if (!f || !o) return fail(TETRIS_EINVAL, "null argument");
  o->offsets = f->offsets.data();               o->n_offsets = (int64_t)f->offsets.size();
  o->stage_len = f->stage_len.data();           o->n_stage_len = (int64_t)f->stage_len.size();
  o->position = f->position.data();             o->n_position = (int64_t)f->position.size();
  o->values = f->values.data();                 o->n_values = (int64_t)f->values.size();
  o->oc_permutation = f->oc_permutation.data(); o->n_oc_permutation = (int64_t)f->oc_permutation.size();
  o->nnz = f->nnz;
  o->tile_ic = f->tile_ic;
  return TETRIS_OK;
}

int tetris_spf_device_arrays(tetris_spf* f, tetris_spf_arrays* o) {
  int rc = tetris_spf_host_arrays(f, o);
  if (rc) return rc;
  rc = spf_ensure_device(f);
  if (rc) return rc;
  o->offsets = f->d_offsets;
  o->stage_len = f->d_stage_len;
  o->position = f->d_position;
  o->values = f->d_values;
  o->oc_permutation = f->d_oc_permutation;
  return TETRIS_OK;
}

int tetris_options_set(unsigned flags) {
  if (flags & ~(TETRIS_OPT_PAIRS | TETRIS_OPT_NO_BANK_RULE | TETRIS_OPT_COLD_TIMING | TETRIS_OPT_TRUST_SPF_ARRAYS |
                TETRIS_OPT_ADD_IN_KERNEL))
    return fail(TETRIS_EINVAL, "unknown option bits 0x%x", flags);
  set_options(flags);
  return TETRIS_OK;
}
unsigned tetris_options_get(void) { return options(); }

int tetris_tile_select(int N, int H, int W, int C, int K, int ks, int stride, int pad, tetris_tile* out) {
  if (!out) return fail(TETRIS_EINVAL, "null argument");
  return choose_tile(N, H, W, C, K, ks, stride, pad, out);
}

int tetris_tile_table_load(const char* path, int* rows_out) {
  if (!path) return fail(TETRIS_EINVAL, "null argument");
  return load_tile_table(path, rows_out);
}

int tetris_oc_order_balanced(const float* h_filter, int C, int K, int ks, const tetris_tile* tile, int32_t* order_out) {
  if (!h_filter || !tile || !order_out) return fail(TETRIS_EINVAL, "null argument");
  if (C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs) return fail(TETRIS_EINVAL, "bad filter shape");
  return balance_oc_order(h_filter, C, K, ks, *tile, order_out);
}

int tetris_tile_autotune_list(const float* h_filter, int N, int H, int W, int C, int K, int ks, int stride, int pad,
                              int max_candidates, void* stream_, tetris_tile* out, float* ms_out, int max_out,
                              int* n_out) {
  if (!h_filter || !out || max_out < 1) return fail(TETRIS_EINVAL, "null argument");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs) return fail(TETRIS_EINVAL, "bad layer shape");
  size_t nnz = 0;
  const size_t n_w = (size_t)C * K * ks * ks;
  for (size_t i = 0; i < n_w; ++i) nnz += h_filter[i] != 0.f;
  std::vector<tetris_tile> ranked;
  int rc = rank_tiles(N, H, W, C, K, ks, stride, pad, &ranked, (double)nnz / (double)n_w);
  if (rc) return rc;
  if (max_candidates == 0) max_candidates = 24;
  if (max_candidates < 0) max_candidates = (int)ranked.size();  // exhaustive, like the reference's table walk
  const int OH = out_extent(H, pad, ks, stride), OW = out_extent(W, pad, ks, stride);
  const size_t in_bytes = sizeof(float) * (size_t)N * C * H * W, out_bytes = sizeof(float) * (size_t)N * K * OH * OW;
  const size_t f_bytes = sizeof(float) * (size_t)C * K * ks * ks;
  float *d_in = nullptr, *d_out = nullptr, *d_f = nullptr;
  std::map<std::array<int, 3>, tetris_g950*> packs;  // by (tile_ic, oc_per_wave, waves): what the pack and its order depend on
  std::vector<int32_t> order(K);
  auto done = [&](int code) {
    for (auto& kv : packs) tetris_g950_destroy(kv.second);
    if (d_in) (void)hipFree(d_in);
    if (d_out) (void)hipFree(d_out);
    if (d_f) (void)hipFree(d_f);
    return code;
  };
#define HIPA(call)                                                                                          \
  do {                                                                                                      \
    hipError_t e_ = (call);                                                                                 \
    if (e_ != hipSuccess)                                                                                   \
      return done(fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__, hipGetErrorString(e_))); \
  } while (0)
  HIPA(hipMalloc(&d_in, in_bytes));
  HIPA(hipMalloc(&d_out, out_bytes));
  HIPA(hipMalloc(&d_f, f_bytes));
  HIPA(hipMemsetAsync(d_in, 0, in_bytes, stream));  // timing does not depend on the values
  HIPA(hipMemcpyAsync(d_f, h_filter, f_bytes, hipMemcpyHostToDevice, stream));
#undef HIPA
  // first pass: a quick look at every candidate; second pass: the four fastest again, with more launches
  std::vector<std::pair<float, tetris_tile>> timed;
  for (const tetris_tile& t : ranked) {
    if ((int)timed.size() >= max_candidates) break;
    const std::array<int, 3> key{t.tile_ic, t.oc_per_wave, t.waves};
    auto it = packs.find(key);
    if (it == packs.end()) {
      tetris_g950* p = nullptr;
      rc = balance_oc_order(h_filter, C, K, ks, t, order.data());
      if (rc == TETRIS_OK) rc = tetris_g950_create_device(d_f, C, K, ks, t.tile_ic, t.oc_per_wave, order.data(), stream, &p);
      if (rc) return done(rc);
      it = packs.emplace(key, p).first;
    }
    float ms = 0;
    rc = time_launches(it->second, d_in, d_out, N, H, W, stride, pad, &t, stream, timed.empty() ? 8 : 1, 3, &ms);
    if (rc == TETRIS_EINVAL) continue;  // the model ranks shapes make_geom may still refuse
    if (rc) return done(rc);
    if (timed.empty() && ms > 0) {
      // The first candidate also settles the shader clock: it idles near 2.1 GHz and needs 10-25 ms of unbroken work to
      // reach the 2.3-2.4 GHz it holds under load, a tenth in time that would otherwise count against the candidates
      // the model ranks first.  Some 30 ms of launches, then the candidate's time again.
      const int settle = (int)std::min(3000.0f, 30.0f / ms);
      rc = time_launches(it->second, d_in, d_out, N, H, W, stride, pad, &t, stream, settle, 3, &ms);
      if (rc) return done(rc);
    }
    timed.emplace_back(ms, t);
  }
  if (timed.empty()) return done(fail(TETRIS_EINVAL, "no tile shape could be launched for this layer"));
  auto by_time = [](const std::pair<float, tetris_tile>& a, const std::pair<float, tetris_tile>& b) { return a.first < b.first; };
  std::stable_sort(timed.begin(), timed.end(), by_time);
  // The candidates so far leave the split of the channel reduction to the rule.  For the fastest of them, where the
  // layer has few enough pixels for a split to be legal, time the other slice counts too (1 = none, 2, 4, 8): fewer
  // slices move fewer partial sums, more slices fill more of the GPU.
  {
    const size_t top = std::min<size_t>(timed.size(), 6);
    std::vector<std::pair<float, tetris_tile>> extra;
    for (size_t i = 0; i < top; ++i) {
      const tetris_tile base = timed[i].second;
      tetris_g950* pk = packs[{base.tile_ic, base.oc_per_wave, base.waves}];
      Geom g0;
      if (make_geom(pk, N, H, W, stride, pad, base, &g0) != TETRIS_OK) continue;
      for (int cs : {1, 2, 4, 8}) {
        if (cs == g0.csplit) continue;
        tetris_tile v = base;
        v.csplit = cs;
        Geom gv;
        if (make_geom(pk, N, H, W, stride, pad, v, &gv) != TETRIS_OK) continue;
        // more slices than wave slots to run them at once only add partial sums
        if (cs > g0.csplit && (long long)gv.ugroups * gv.kblocks * cs * v.waves > 16ll * 256 * 2) continue;
        float ms = 0;
        rc = time_launches(pk, d_in, d_out, N, H, W, stride, pad, &v, stream, 1, 3, &ms);
        if (rc == TETRIS_EINVAL) continue;
        if (rc) return done(rc);
        extra.emplace_back(ms, v);
      }
    }
    timed.insert(timed.end(), extra.begin(), extra.end());
    std::stable_sort(timed.begin(), timed.end(), by_time);
  }
  const size_t again = std::min<size_t>(timed.size(), std::max(4, max_out));
  for (size_t i = 0; i < again; ++i) {
    const tetris_tile& t = timed[i].second;
    float ms = 0;
    rc = time_launches(packs[{t.tile_ic, t.oc_per_wave, t.waves}], d_in, d_out, N, H, W, stride, pad, &t, stream, 2, 10,
                       &ms);
    if (rc) return done(rc);
    timed[i].first = ms;
  }
  std::stable_sort(timed.begin(), timed.begin() + again, by_time);
  const int n = (int)std::min<size_t>(again, (size_t)max_out);
  for (int i = 0; i < n; ++i) {
    out[i] = timed[i].second;
    if (ms_out) ms_out[i] = timed[i].first;
  }
  if (n_out) *n_out = n;
  return done(TETRIS_OK);
}

int tetris_tile_autotune(const float* h_filter, int N, int H, int W, int C, int K, int ks, int stride, int pad,
                         int max_candidates, void* stream, tetris_tile* out, float* ms_out) {
  return tetris_tile_autotune_list(h_filter, N, H, W, C, K, ks, stride, pad, max_candidates, stream, out, ms_out, 1,
                                   nullptr);
}

int tetris_spconv2d_launch(tetris_g950* p, const float* d_in, float* d_out, int N, int H, int W, int stride, int pad,
                           const tetris_tile* tile, void* stream) {
  return run_launch(p, d_in, d_out, N, H, W, stride, pad, tile, static_cast<hipStream_t>(stream));
}

int tetris_spconv2d_launch_act(tetris_g950* p, const float* d_in, float* d_out, int N, int H, int W, int stride,
                               int pad, const tetris_tile* tile, int activation, void* stream) {
  if (activation < TETRIS_ACT_NONE || activation > TETRIS_ACT_RELU_POOL2)
    return fail(TETRIS_EINVAL, "unknown activation %d", activation);
  return run_launch(p, d_in, d_out, N, H, W, stride, pad, tile, static_cast<hipStream_t>(stream), activation);
}

int tetris_spconv2d_act_supported(tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile* tile,
                                  int activation, int* supported) {
  if (!p || !tile || !supported) return fail(TETRIS_EINVAL, "null argument");
  if (activation < TETRIS_ACT_NONE || activation > TETRIS_ACT_RELU_POOL2)
    return fail(TETRIS_EINVAL, "unknown activation %d", activation);
  Geom g;
  const int rc = make_geom(p, N, H, W, stride, pad, *tile, &g);
  if (rc) return rc;
  *supported = activation != TETRIS_ACT_RELU_POOL2 ||
               (g.OH >= 2 && g.OW >= 2 && (g.csplit > 1 || geom_pools_in_kernel(g)));
  return TETRIS_OK;
}

int tetris_launch_shape_of(tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile* tile,
                           tetris_launch_shape* out) {
  if (!p || !tile || !out) return fail(TETRIS_EINVAL, "null argument");
  Geom g;
  const int rc = make_geom(p, N, H, W, stride, pad, *tile, &g);
  if (rc) return rc;
  out->unit_groups = g.ugroups;
  out->channel_blocks = g.kblocks;
  out->csplit = g.csplit;
  out->workgroups = g.ugroups * g.kblocks * g.csplit;
  out->stages = g.stages;
  out->lanes_used = g.ver == 4 ? 64 : g.lw * std::min(g.lh, g.thi * g.nb);
  out->kernel = g.ver;
  out->lds_bytes = g.ver == 4 ? 2 * g.buf_bytes : g.ver == 3 ? kBufs * g.buf_bytes : kTileBytes;
  out->scratch_bytes = (int64_t)partial_bytes_of(g);
  return TETRIS_OK;
}

int tetris_g950_prepare(tetris_g950* p, int N, int H, int W, int stride, int pad, const tetris_tile* tile, void* stream_) {
  if (!p) return fail(TETRIS_EINVAL, "null argument");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Plan plan;
  int rc = find_plan(p, N, H, W, stride, pad, tile, stream, true, &plan);
  if (rc) return rc;
  if (plan.geom.csplit > 1) {
    float* d_partial = nullptr;
    rc = partial_buffer(p, stream, partial_bytes_of(plan.geom), true, &d_partial);
    if (rc) return rc;
  }
  float* s = nullptr;
  return static_scratch(&s);  // looks the static scratch array of this GPU up, for tetris_spconv2d_launch_noalloc
}

int tetris_split_layers_add_in_kernel(int* yes) {
  if (!yes) return fail(TETRIS_EINVAL, "null argument");
  bool ok = false;
  const int rc = same_xcd_by_residue(&ok);
  if (rc) return rc;
  *yes = ok && (options() & TETRIS_OPT_ADD_IN_KERNEL);
  return TETRIS_OK;
}

size_t tetris_noalloc_scratch_bytes(void) { return g_scratch_limit.load(); }

size_t tetris_noalloc_scratch_limit(size_t bytes) {
  if (bytes == 0 || bytes > kStaticScratchBytes) bytes = kStaticScratchBytes;
  g_scratch_limit.store(bytes);
  return bytes;
}

int tetris_spconv2d_launch_noalloc(tetris_g950* p, const float* d_in, float* d_out, int N, int H, int W, int stride,
                                   int pad, const tetris_tile* tile, void* stream_) {
  if (!p || !d_in || !d_out) return fail(TETRIS_EINVAL, "null argument");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  Plan plan;
  int rc = find_plan(p, N, H, W, stride, pad, tile, stream, false, &plan);
  if (rc) return rc;
  float* d_partial = nullptr;
  if (plan.geom.csplit > 1) {
    const size_t need = partial_bytes_of(plan.geom);
    const size_t limit = g_scratch_limit.load();
    if (need > limit)
      return fail(TETRIS_EINVAL, "this layer needs %zu bytes of tickets and partial sums, the static scratch holds %zu: "
                  "use tetris_spconv2d_launch", need, limit);
    rc = static_scratch(&d_partial);
    if (rc) return rc;
  }
  // Every element of the partial sums that reduce_kernel reads is written by this launch's conv kernel first, so
  // what an earlier call left in the array needs no clearing.
  return launch_conv(plan.geom, d_in, d_out, d_partial, plan.entries, plan.grp_off, plan.grp_pair, p->d_oc_order, 0,
                     stream);
}

int tetris_spconv2d_launch_spf_arrays(const float* d_in, const int32_t* d_offsets, const int32_t* d_stage_len,
                                      const int32_t* d_perm, const int32_t* d_position, const float* d_values,
                                      float* d_out, int N, int H, int W, int C, int K, int ks, int stride, int pad,
                                      int tile_ic, int vec_width, int64_t n_entries, const tetris_tile* tile,
                                      void* stream_) {
  (void)d_stage_len;  // the reference's kernel does not read it either (Tetris/spconv2d_kernel.cu:13-160)
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  tetris_g950* pack = nullptr;
  tetris_tile t{};
  // held until the launch is issued: the pack belongs to a view that another thread's call may evict or drop
  std::lock_guard<std::mutex> lock(g_views_mu);
  int rc = view_pack(d_offsets, d_perm, d_position, d_values, N, H, W, C, K, ks, stride, pad, tile_ic, vec_width,
                     (long long)n_entries, tile, stream, &pack, &t);
  if (rc) return rc;
  return run_launch(pack, d_in, d_out, N, H, W, stride, pad, &t, stream);
}

void tetris_spf_invalidate(const float* d_values) { drop_views(d_values); }

int tetris_spconv2d_launch_spf(const float* d_in, const int32_t* d_offsets, const int32_t* d_stage_len,
                               const int32_t* d_perm, const int32_t* d_position, const float* d_values, float* d_out,
                               int N, int H, int W, int C, int K, int ks, int stride, int pad, void* stream) {
  // the call shape of the reference launcher carries neither TILE_IC (a template argument there) nor the vector
  // width: they are taken from the live tetris_spf that owns `d_values`; the CONTENT comes from the arrays
  int tile_ic = 0, vec = 0;
  int64_t n_entries = 0;
  {
    std::lock_guard<std::mutex> lock(g_registry_mu);
    auto it = g_registry.find(d_values);
    if (it == g_registry.end())
      return fail(TETRIS_ENOTFOUND, "device arrays do not belong to a live tetris_spf handle (use "
                  "tetris_spconv2d_launch_spf_arrays for arrays of your own)");
    const tetris_spf* f = it->second;
    if (f->C != C || f->K != K || f->ks != ks)
      return fail(TETRIS_EINVAL, "shape C=%d K=%d ks=%d does not match the packed filter (%d, %d, %d)", C, K, ks, f->C,
                  f->K, f->ks);
    tile_ic = f->tile_ic;
    vec = f->vec;
    n_entries = (int64_t)f->values.size();
  }
  return tetris_spconv2d_launch_spf_arrays(d_in, d_offsets, d_stage_len, d_perm, d_position, d_values, d_out, N, H, W, C,
                                           K, ks, stride, pad, tile_ic, vec, n_entries, nullptr, stream);
}

int tetris_spconv2d_time(tetris_g950* p, const float* d_in, float* d_out, int N, int H, int W, int stride, int pad,
                         const tetris_tile* tile, void* stream, int warm, int repeat, float* ms_out) {
  return time_launches(p, d_in, d_out, N, H, W, stride, pad, tile, static_cast<hipStream_t>(stream), warm, repeat,
                       ms_out);
}

int tetris_spconv2d_host(const float* h_in, const float* h_filter, float* h_out, int N, int H, int W, int C, int K,
                         int ks, int stride, int pad, void* stream, const char* layout, int apply_reorder,
                         float* ms_out) {
  (void)layout;
  return conv_host(h_in, h_filter, h_out, N, H, W, C, K, ks, stride, pad, static_cast<hipStream_t>(stream),
                   apply_reorder != 0, false, 0u, ms_out);
}

int tetris_spconv2d_spf_host(const float* h_in, const float* h_filter, float* h_out, int N, int H, int W, int C, int K,
                             int ks, int stride, int pad, void* stream, const char* layout, int apply_reorder,
                             unsigned flags, float* ms_out) {
  (void)layout;
  (void)apply_reorder;  // the reference ignores it here too: its SparseFilter is always built reordered (spf.cc:43-44)
  if (flags & ~(TETRIS_BANK_OPTIMIZE | TETRIS_REORDER_OUT_CHANNEL)) return fail(TETRIS_EINVAL, "unknown flags 0x%x", flags);
  return conv_host(h_in, h_filter, h_out, N, H, W, C, K, ks, stride, pad, static_cast<hipStream_t>(stream), true, true,
                   flags, ms_out);
}

int tetris_spconv2d_baseline_host(const float* h_in, const float* h_filter, float* h_out, int N, int H, int W, int C,
                                  int K, int ks, int stride, int pad, void* stream, const char* layout, float* ms_out) {
  (void)layout;
  return conv_host(h_in, h_filter, h_out, N, H, W, C, K, ks, stride, pad, static_cast<hipStream_t>(stream), false, true,
                   0u, ms_out, true);
}

int tetris_read_weight_file(const char* path, int32_t header[8], float** h_filter_out, int64_t* nnz_out) {
  if (!path || !header || !h_filter_out) return fail(TETRIS_EINVAL, "null argument");
  FILE* fp = fopen(path, "r");
  if (!fp) return fail(TETRIS_EIO, "Open file error: %s", path);
  for (int i = 0; i < 8; ++i)
    if (fscanf(fp, "%d", &header[i]) != 1) {
      fclose(fp);
      return fail(TETRIS_EIO, "truncated header in %s", path);
    }
  const int64_t n = (int64_t)header[3] * header[2] * header[4] * header[4];
  if (n <= 0 || header[4] > kMaxKs) {
    fclose(fp);
    return fail(TETRIS_EINVAL, "bad header in %s", path);
  }
  float* f = static_cast<float*>(malloc(sizeof(float) * (size_t)n));
  if (!f) {
    fclose(fp);
    return fail(TETRIS_EINVAL, "out of memory for %lld weights", (long long)n);
  }
  int64_t nnz = 0;
  for (int64_t i = 0; i < n; ++i) {
    if (fscanf(fp, "%f", &f[i]) != 1) {
      free(f);
      fclose(fp);
      return fail(TETRIS_EIO, "truncated weights in %s (%lld of %lld)", path, (long long)i, (long long)n);
    }
    nnz += f[i] != 0;
  }
  fclose(fp);
  *h_filter_out = f;
  if (nnz_out) *nnz_out = nnz;
  return TETRIS_OK;
}

void tetris_free(void* p) { free(p); }

int tetris_float_equal(float x, float y) { return std::fabs(x - y) <= 1e-5 * (std::fabs(x) + std::fabs(y)) + 1e-5; }

int64_t tetris_tensor_first_mismatch(const float* x, const float* y, int64_t len) {
  for (int64_t i = 0; i < len; ++i)
    if (!tetris_float_equal(x[i], y[i])) return i;
  return -1;
}

}  // extern "C"
