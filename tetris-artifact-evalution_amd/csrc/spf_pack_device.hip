// gfx950 weight-preprocessing pass: dense OIHW fp32 filter -> one stream of non-zero (position, value)
// entries per (wave group of G output-channel slots, input-channel stage), built on the device in three
// deterministic kernels (count, scan, scatter).
//
// Takes the place of the reference's host-side SparseFilter constructor (Tetris/spconv2d_utils.h:62-98,
// :206-244) for the HIP kernel.  The position word keeps the reference encoding
// s | r << 3 | (ic % tile_ic) << 6 (spconv2d_utils.h:91) in its low 24 bits, and the zero test keeps
// `value != 0.f`, so -0.0 is dropped like the reference drops it.  What differs is the arrangement: the
// reference interleaves 32 lanes x 4 entries because its lanes are output channels; here every entry is
// wave-uniform.  A stream lists the non-zeros of the group's G channels position by position (channel,
// row, column ascending; within a position by slot), carries the slot's index inside the group in bits
// 24..31, and is padded with zero entries to a multiple of 8 (one 64-byte scalar fetch).
#include "common.h"

namespace tetris {
namespace {

// one wave per (group, stage); element i of the stage is (position i / G, slot i % G)
__global__ __launch_bounds__(256) void count_kernel(const float* __restrict__ filter, const int32_t* __restrict__ oc_order,
                                                    int32_t* __restrict__ grp_nnz, int32_t* __restrict__ grp_pad, int C,
                                                    int ks, int tile_ic, int stages, int G, int nstream) {
  const int sid = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (sid >= nstream) return;
  const int grp = sid / stages, st = sid - grp * stages;
  const int kk = ks * ks;
  const int c0 = st * tile_ic;
  const int n = min(tile_ic, C - c0) * kk * G;
  int cnt = 0;
  for (int i = lane; i < n; i += 64) {
    const int p = i / G, l = i - p * G;
    const int oc = oc_order[grp * G + l];
    if (oc >= 0) cnt += (filter[((size_t)oc * C + c0) * kk + p] != 0.f) ? 1 : 0;
  }
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_xor(cnt, off);
  if (lane == 0) {
    grp_nnz[sid] = cnt;
    grp_pad[sid] = (cnt + kBatch - 1) / kBatch * kBatch;
  }
}

// exclusive scan of grp_pad into grp_off[0..n], single workgroup
__global__ __launch_bounds__(1024) void scan_kernel(const int32_t* __restrict__ grp_pad, int32_t* __restrict__ grp_off,
                                                    int n) {
  __shared__ int part[1024];
  const int tid = threadIdx.x;
  const int chunk = (n + 1023) / 1024;
  const int b = min(n, tid * chunk), e = min(n, b + chunk);
  int s = 0;
  for (int i = b; i < e; ++i) s += grp_pad[i];
  part[tid] = s;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const int v = tid >= off ? part[tid - off] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  int run = tid ? part[tid - 1] : 0;
  for (int i = b; i < e; ++i) {
    grp_off[i] = run;
    run += grp_pad[i];
  }
  if (tid == 1023) grp_off[n] = part[1023];
}

__global__ __launch_bounds__(256) void scatter_kernel(const float* __restrict__ filter,
                                                      const int32_t* __restrict__ oc_order,
                                                      const int32_t* __restrict__ grp_off, int32_t* __restrict__ position,
                                                      float* __restrict__ values, int C, int ks, int tile_ic, int stages,
                                                      int G, int nstream) {
  const int sid = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (sid >= nstream) return;
  const int grp = sid / stages, st = sid - grp * stages;
  const int beg = grp_off[sid], end = grp_off[sid + 1];
  const int kk = ks * ks;
  const int c0 = st * tile_ic;
  const int n = min(tile_ic, C - c0) * kk * G;
  int written = 0;
  for (int i0 = 0; i0 < n; i0 += 64) {
    const int i = i0 + lane;
    const int p = i / G, l = i - p * G;
    float v = 0.f;
    if (i < n) {
      const int oc = oc_order[grp * G + l];
      if (oc >= 0) v = filter[((size_t)oc * C + c0) * kk + p];
    }
    const bool nz = v != 0.f;
    const unsigned long long m = __ballot(nz);
    if (nz) {
      const int rank = __popcll(m & ((1ull << lane) - 1ull));
      const int ic = p / kk, rs = p - ic * kk;
      const int r = rs / ks, s = rs - r * ks;
      position[beg + written + rank] = s + (r << 3) + (ic << 6) + (l << 24);
      values[beg + written + rank] = v;
    }
    written += __popcll(m);
  }
  for (int i = beg + written + lane; i < end; i += 64) {  // padding entries
    position[i] = 0;
    values[i] = 0.f;
  }
}

// position word -> the kernel's entry code for one tile geometry
__global__ __launch_bounds__(256) void bind_kernel(const int32_t* __restrict__ position, const float* __restrict__ values,
                                                   int2* __restrict__ out, long long n, int plane, int pitch, int par,
                                                   int stride, int nq) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int pos = position[i];
  const int s = pos & 7, r = (pos >> 3) & 7, ic = (pos >> 6) & 0x3ffff, l = (pos >> 24) & 0xff;
  int2 e;
  // [15:0] LDS byte offset, [23:16] first accumulator of the slot, [31:28] VGPR-index enables (see gen_walk_asm.py)
  e.x = 4 * (ic * plane + r * pitch + (s % stride) * par + (s / stride) * 4) | ((l * 4 * nq) << 16) | (int)0xC0000000u;
  e.y = __float_as_int(values[i]);
  out[i] = e;
}

int pack_device(const float* d_filter, int C, int K, int ks, int tile_ic, int G, const int32_t* oc_order,
                hipStream_t stream, tetris_g950** out) {
  if (!d_filter || !out) return fail(TETRIS_EINVAL, "null argument");
  if (C <= 0 || K <= 0 || ks <= 0 || ks > kMaxKs || tile_ic <= 0)
    return fail(TETRIS_EINVAL, "bad filter shape C=%d K=%d ks=%d tile_ic=%d (ks <= %d)", C, K, ks, tile_ic, kMaxKs);
  if (G != 1 && G != 2 && G != 4 && G != 8 && G != 16 && G != 32)
    return fail(TETRIS_EINVAL, "oc_per_wave must be 1, 2, 4, 8, 16 or 32 (got %d)", G);
  if ((long long)tile_ic * 64 >= (1 << 24))
    return fail(TETRIS_EINVAL, "tile_ic %d does not fit the position word", tile_ic);
  tetris_g950* p = new tetris_g950;
  p->C = C; p->K = K; p->ks = ks; p->tile_ic = tile_ic; p->g = G;
  p->stages = (C - 1) / tile_ic + 1;
  p->slots = (K + kSlotPad - 1) / kSlotPad * kSlotPad;
  p->groups = p->slots / G;
  const int nseg = p->groups * p->stages;

  std::vector<int32_t> order(p->slots, -1);
  std::vector<char> seen(K, 0);
  for (int i = 0; i < K; ++i) {
    const int oc = oc_order ? oc_order[i] : i;
    if (oc < 0 || oc >= K || seen[oc]) {
      delete p;
      return fail(TETRIS_EINVAL, "oc_order is not a permutation of 0..%d", K - 1);
    }
    seen[oc] = 1;
    order[i] = oc;
  }
  int32_t* d_pad = nullptr;
  auto cleanup = [&](int rc) {
    if (d_pad) (void)hipFree(d_pad);
    if (rc != TETRIS_OK) tetris_g950_destroy(p);
    return rc;
  };
#define HIPC(call)                                                                                              \
  do {                                                                                                          \
    hipError_t e_ = (call);                                                                                     \
    if (e_ != hipSuccess)                                                                                       \
      return cleanup(fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__, hipGetErrorString(e_))); \
  } while (0)
  HIPC(hipMalloc(&p->d_oc_order, sizeof(int32_t) * p->slots));
  HIPC(hipMalloc(&p->d_grp_off, sizeof(int32_t) * (nseg + 1)));
  HIPC(hipMalloc(&p->d_grp_nnz, sizeof(int32_t) * nseg));
  HIPC(hipMalloc(&d_pad, sizeof(int32_t) * nseg));
  HIPC(hipMemcpyAsync(p->d_oc_order, order.data(), sizeof(int32_t) * p->slots, hipMemcpyHostToDevice, stream));
  const int blocks = (nseg + 3) / 4;
  hipLaunchKernelGGL(count_kernel, dim3(blocks), dim3(256), 0, stream, d_filter, p->d_oc_order, p->d_grp_nnz, d_pad, C,
                     ks, tile_ic, p->stages, G, nseg);
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, stream, d_pad, p->d_grp_off, nseg);
  HIPC(hipGetLastError());
  int32_t total = 0;
  HIPC(hipMemcpyAsync(&total, p->d_grp_off + nseg, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
  HIPC(hipStreamSynchronize(stream));
  p->n_entries = total;
  // one spare batch so that a kernel may prefetch the batch after the last one
  HIPC(hipMalloc(&p->d_position, sizeof(int32_t) * (size_t)(total + kBatch)));
  HIPC(hipMalloc(&p->d_values, sizeof(float) * (size_t)(total + kBatch)));
  HIPC(hipMemsetAsync(p->d_position + total, 0, sizeof(int32_t) * kBatch, stream));
  HIPC(hipMemsetAsync(p->d_values + total, 0, sizeof(float) * kBatch, stream));
  hipLaunchKernelGGL(scatter_kernel, dim3(blocks), dim3(256), 0, stream, d_filter, p->d_oc_order, p->d_grp_off,
                     p->d_position, p->d_values, C, ks, tile_ic, p->stages, G, nseg);
  HIPC(hipGetLastError());
  // nnz = sum of seg_nnz, summed on the host (small)
  std::vector<int32_t> nz(nseg);
  HIPC(hipMemcpyAsync(nz.data(), p->d_grp_nnz, sizeof(int32_t) * nseg, hipMemcpyDeviceToHost, stream));
  HIPC(hipStreamSynchronize(stream));
  p->nnz = 0;
  for (int v : nz) p->nnz += v;
#undef HIPC
  *out = p;
  return cleanup(TETRIS_OK);
}

}  // namespace

namespace {

// Which entries of a stream become pair members.  The stream lists its entries position by position (slots ascending
// inside a position); of a run of k entries with one position the first 2 * (k / 2) form k / 2 pairs, and the last
// one of an odd run stays single.  Entry i is therefore single exactly when it is the last of its run and its index
// inside the run is even.  One wave per stream; returns, per lane, the classification of entry base + lane.
struct PairScan {
  int carry_start;  // first entry index of the run that the previous chunk ended in
  int carry_pos;    // position of the previous chunk's last entry
};

__device__ __forceinline__ bool entry_is_single(const int32_t* __restrict__ position, int beg, int nnz, int i, int lane,
                                                PairScan& c) {
  const int pos = i < nnz ? (position[beg + i] & 0xffffff) : -1;
  int prev = __shfl_up(pos, 1);
  if (lane == 0) prev = c.carry_pos;
  const bool start = i < nnz && (i == 0 || pos != prev);
  int run_start = start ? i : -1;  // inclusive max-scan over the lanes
  for (int off = 1; off < 64; off <<= 1) {
    const int o = __shfl_up(run_start, off);
    if (lane >= off) run_start = max(run_start, o);
  }
  run_start = max(run_start, c.carry_start);
  const int next = i + 1 < nnz ? (position[beg + i + 1] & 0xffffff) : -2;
  const bool last = i < nnz && next != pos;
  const bool single = last && (((i - run_start) & 1) == 0);
  c.carry_start = __shfl(run_start, 63);
  c.carry_pos = __shfl(pos, 63);
  return single;
}

__global__ __launch_bounds__(256) void pair_count_kernel(const int32_t* __restrict__ position,
                                                         const int32_t* __restrict__ grp_off,
                                                         const int32_t* __restrict__ grp_nnz,
                                                         int32_t* __restrict__ seg_len, int32_t* __restrict__ seg_pair,
                                                         int nstream) {
  const int sid = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (sid >= nstream) return;
  const int beg = grp_off[sid], nnz = grp_nnz[sid];
  PairScan c{-1, -3};
  int singles = 0;
  for (int i0 = 0; i0 < nnz; i0 += 64) singles += __popcll(__ballot(entry_is_single(position, beg, nnz, i0 + lane, lane, c)));
  if (lane == 0) {
    const int pairs = (nnz - singles + kBatch - 1) / kBatch * kBatch;
    seg_pair[sid] = pairs;
    seg_len[sid] = pairs + (singles + kBatch - 1) / kBatch * kBatch;
  }
}

__global__ __launch_bounds__(256) void bind_pairs_kernel(const int32_t* __restrict__ position,
                                                         const float* __restrict__ values,
                                                         const int32_t* __restrict__ grp_off,
                                                         const int32_t* __restrict__ grp_nnz,
                                                         const int32_t* __restrict__ pgrp_off,
                                                         const int32_t* __restrict__ pgrp_pair, int2* __restrict__ out,
                                                         int nstream, int plane, int pitch, int par, int stride, int nq) {
  const int sid = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (sid >= nstream) return;
  const int beg = grp_off[sid], nnz = grp_nnz[sid];
  const int obeg = pgrp_off[sid], oend = pgrp_off[sid + 1], opair = pgrp_pair[sid];
  const int2 pad = make_int2((int)0xC0000000u, 0);
  PairScan c{-1, -3};
  int np = 0, ns = 0;  // pair members and singles written so far
  for (int i0 = 0; i0 < nnz; i0 += 64) {
    const int i = i0 + lane;
    const bool single = entry_is_single(position, beg, nnz, i, lane, c);
    const bool live = i < nnz;
    const unsigned long long ms = __ballot(single), mp = __ballot(live && !single);
    const unsigned long long below = (1ull << lane) - 1ull;
    if (live) {
      const int pos = position[beg + i];
      const int s = pos & 7, r = (pos >> 3) & 7, ic = (pos >> 6) & 0x3ffff, l = (pos >> 24) & 0xff;
      int2 e;
      e.x = 4 * (ic * plane + r * pitch + (s % stride) * par + (s / stride) * 4) | ((l * 4 * nq) << 16) | (int)0xC0000000u;
      e.y = __float_as_int(values[beg + i]);
      out[single ? obeg + opair + ns + __popcll(ms & below) : obeg + np + __popcll(mp & below)] = e;
    }
    np += __popcll(mp);
    ns += __popcll(ms);
  }
  for (int i = obeg + np + lane; i < obeg + opair; i += 64) out[i] = pad;
  for (int i = obeg + opair + ns + lane; i < oend; i += 64) out[i] = pad;
}

__global__ void fill_pad_kernel(int2* __restrict__ out, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = make_int2((int)0xC0000000u, 0);
}

// heads[seg][0..7] = the eight entries at the start of stream `seg` (for an empty stream: of the stream that follows)
__global__ __launch_bounds__(256) void heads_kernel(const int2* __restrict__ entries, const int32_t* __restrict__ grp_off,
                                                    int2* __restrict__ heads, int nseg) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < nseg * kBatch) heads[i] = entries[grp_off[i / kBatch] + i % kBatch];
}

}  // namespace

int g950_bind(tetris_g950* p, const Geom& g, bool paired, hipStream_t stream, const int2** entries_out,
              const int32_t** grp_off_out, const int32_t** grp_pair_out, int* heads_off_out) {
  const BoundKey key{g.plane, g.pitch, g.par, g.stride, g.nq, paired ? 1 : 0};
  const int nseg = p->groups * p->stages;
  std::lock_guard<std::mutex> lock(p->mu);
  if (!p->d_zero_pair) {
    TETRIS_HIP(hipMalloc(&p->d_zero_pair, sizeof(int32_t) * std::max(nseg, 1)));
    TETRIS_HIP(hipMemsetAsync(p->d_zero_pair, 0, sizeof(int32_t) * std::max(nseg, 1), stream));
  }
  const int blocks = (nseg + 3) / 4;
  if (paired && !p->d_pgrp_off) {  // the paired arrangement's stream offsets, once per pack
    int32_t *d_len = nullptr, *d_off = nullptr, *d_pair = nullptr;
    auto drop = [&](int rc) {
      if (d_len) (void)hipFree(d_len);
      if (rc != TETRIS_OK) {
        if (d_off) (void)hipFree(d_off);
        if (d_pair) (void)hipFree(d_pair);
      }
      return rc;
    };
#define HIPB(call)                                                                                              \
  do {                                                                                                          \
    hipError_t e_ = (call);                                                                                     \
    if (e_ != hipSuccess)                                                                                       \
      return drop(fail(TETRIS_EHIP, "%s failed at %s:%d: %s", #call, __FILE__, __LINE__, hipGetErrorString(e_))); \
  } while (0)
    HIPB(hipMalloc(&d_len, sizeof(int32_t) * nseg));
    HIPB(hipMalloc(&d_off, sizeof(int32_t) * (nseg + 1)));
    HIPB(hipMalloc(&d_pair, sizeof(int32_t) * nseg));
    hipLaunchKernelGGL(pair_count_kernel, dim3(blocks), dim3(256), 0, stream, p->d_position, p->d_grp_off, p->d_grp_nnz,
                       d_len, d_pair, nseg);
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, stream, d_len, d_off, nseg);
    HIPB(hipGetLastError());
    int32_t total = 0;
    HIPB(hipMemcpyAsync(&total, d_off + nseg, sizeof(int32_t), hipMemcpyDeviceToHost, stream));
    HIPB(hipStreamSynchronize(stream));
#undef HIPB
    p->n_paired_entries = total;
    p->d_pgrp_off = d_off;
    p->d_pgrp_pair = d_pair;
    drop(TETRIS_OK);
  }
  auto it = p->bound.find(key);
  if (it == p->bound.end()) {
    int2* d = nullptr;
    const long long n = (paired ? p->n_paired_entries : p->n_entries) + kBatch;  // a spare batch for the look-ahead fetch
    if (n + (long long)nseg * kBatch > 0x7fffffffll) return fail(TETRIS_EINVAL, "pack too large to bind");
    TETRIS_HIP(hipMalloc(&d, sizeof(int2) * (size_t)(n + (long long)nseg * kBatch)));  // entries, then the streams' heads
    if (paired) {
      hipLaunchKernelGGL(bind_pairs_kernel, dim3(blocks), dim3(256), 0, stream, p->d_position, p->d_values, p->d_grp_off,
                         p->d_grp_nnz, p->d_pgrp_off, p->d_pgrp_pair, d, nseg, g.plane, g.pitch, g.par, g.stride, g.nq);
      hipLaunchKernelGGL(fill_pad_kernel, dim3(1), dim3(64), 0, stream, d + p->n_paired_entries, kBatch);
    } else {
      hipLaunchKernelGGL(bind_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p->d_position, p->d_values,
                         d, n, g.plane, g.pitch, g.par, g.stride, g.nq);
    }
    if (nseg > 0)
      hipLaunchKernelGGL(heads_kernel, dim3((unsigned)((nseg * kBatch + 255) / 256)), dim3(256), 0, stream, d,
                         paired ? p->d_pgrp_off : p->d_grp_off, d + n, nseg);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      (void)hipFree(d);
      return fail(TETRIS_EHIP, "bind kernel launch failed: %s", hipGetErrorString(e));
    }
    it = p->bound.emplace(key, d).first;
  }
  *entries_out = it->second;
  *grp_off_out = paired ? p->d_pgrp_off : p->d_grp_off;
  *grp_pair_out = paired ? p->d_pgrp_pair : p->d_zero_pair;
  *heads_off_out = (int)((paired ? p->n_paired_entries : p->n_entries) + kBatch);
  return TETRIS_OK;
}

// ---- the reference layout's device arrays as the source of a convolution ------------------------------------------
// SparseConv2d<...> of the reference computes from offsets_/position_/values_/oc_permutation_ on the device
// (Tetris/spconv2d_kernel.cu:91-156).  Here those arrays are decoded, on the device, back into a dense OIHW filter
// from which the kernel's own pack is made; a content hash tells when a caller has rewritten them in place.
namespace {

__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// out[0] += order-independent hash of (array id, index, word) over the four arrays, n_ent entries of the last two
__global__ __launch_bounds__(256) void spf_hash_kernel(const int32_t* __restrict__ offsets, int n_off,
                                                       const int32_t* __restrict__ perm, int K,
                                                       const int32_t* __restrict__ position,
                                                       const float* __restrict__ values, long long n_ent,
                                                       unsigned long long* __restrict__ out) {
  const long long total = n_off + K + 2 * n_ent;
  unsigned long long h = 0;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
    unsigned word;
    if (i < n_off) word = (unsigned)offsets[i];
    else if (i < n_off + K) word = (unsigned)perm[i - n_off];
    else if (i < n_off + K + n_ent) word = (unsigned)position[i - n_off - K];
    else word = __float_as_uint(values[i - n_off - K - n_ent]);
    h += mix64(((unsigned long long)i << 32) ^ word ^ 0x9E3779B97F4A7C15ull);
  }
  for (int off = 32; off > 0; off >>= 1) h += __shfl_xor(h, off);
  if ((threadIdx.x & 63) == 0) atomicAdd(out, h);
}

// vec > 0: the reorder path's layout (Tetris/spconv2d_utils.h:206-244): one workgroup per (32-lane group, stage);
// entry e of lane l sits at 32 * offsets[seg] + (e / vec) * 32 * vec + l * vec + e % vec and belongs to output channel
// perm[group * 32 + l], input channel (position >> 6) + stage * tile_ic.  vec == 0: the keep-as-is layout (:38-61),
// one run of entries per (output channel, stage).  Zero values (padding of either kind) are skipped.
__global__ __launch_bounds__(256) void spf_decode_kernel(const int32_t* __restrict__ offsets,
                                                         const int32_t* __restrict__ perm,
                                                         const int32_t* __restrict__ position,
                                                         const float* __restrict__ values, float* __restrict__ filter,
                                                         int C, int K, int ks, int tile_ic, int stages, int vec) {
  const int seg = blockIdx.x;
  const int stage = seg % stages, row = seg / stages;  // row: 32-lane group, or output channel when vec == 0
  const int beg = offsets[seg], len = max(offsets[seg + 1] - beg, 0);
  const int kk = ks * ks;
  if (vec == 0) {
    for (int e = threadIdx.x; e < len; e += blockDim.x) {
      const float v = values[beg + e];
      const int pos = position[beg + e];
      const int c = (pos >> 6) + stage * tile_ic, r = (pos >> 3) & 7, s_ = pos & 7;
      if (v != 0.f && c < C && r < ks && s_ < ks) filter[((size_t)row * C + c) * kk + r * ks + s_] = v;
    }
    return;
  }
  const long long base = 32ll * beg;
  for (int j = threadIdx.x; j < 32 * len; j += blockDim.x) {
    const int lane = (j % (32 * vec)) / vec;
    const int slot = row * 32 + lane;
    const float v = values[base + j];
    if (slot >= K || v == 0.f) continue;
    const int pos = position[base + j];
    const int c = (pos >> 6) + stage * tile_ic, r = (pos >> 3) & 7, s_ = pos & 7;
    const int k = perm[slot];
    if (k >= 0 && k < K && c < C && r < ks && s_ < ks) filter[((size_t)k * C + c) * kk + r * ks + s_] = v;
  }
}

__global__ void fill_zero_kernel(float* __restrict__ p, long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) p[i] = 0.f;
}

}  // namespace

int spf_arrays_hash(const int32_t* d_offsets, int n_off, const int32_t* d_perm, int K, const int32_t* d_position,
                    const float* d_values, long long n_ent, unsigned long long* d_scratch2, hipStream_t stream,
                    unsigned long long* hash_out) {
  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, stream, reinterpret_cast<float*>(d_scratch2), 4ll);
  hipLaunchKernelGGL(spf_hash_kernel, dim3(256), dim3(256), 0, stream, d_offsets, n_off, d_perm, K, d_position, d_values,
                     n_ent, d_scratch2);
  TETRIS_HIP(hipGetLastError());
  unsigned long long h[2] = {0, 0};
  TETRIS_HIP(hipMemcpyAsync(h, d_scratch2, sizeof h, hipMemcpyDeviceToHost, stream));
  TETRIS_HIP(hipStreamSynchronize(stream));
  *hash_out = h[0];
  return TETRIS_OK;
}

int spf_arrays_decode(const int32_t* d_offsets, const int32_t* d_perm, const int32_t* d_position, const float* d_values,
                      float* d_filter, int C, int K, int ks, int tile_ic, int vec, hipStream_t stream) {
  const int stages = (C - 1) / tile_ic + 1;
  const int rows = vec == 0 ? K : (K + 31) / 32;
  const long long n = (long long)C * K * ks * ks;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)std::min<long long>((n + 255) / 256, 4096)), dim3(256), 0, stream,
                     d_filter, n);
  hipLaunchKernelGGL(spf_decode_kernel, dim3(rows * stages), dim3(256), 0, stream, d_offsets, d_perm, d_position, d_values,
                     d_filter, C, K, ks, tile_ic, stages, vec);
  TETRIS_HIP(hipGetLastError());
  return TETRIS_OK;
}

}  // namespace tetris

extern "C" {

int tetris_g950_create_device(const float* d_filter, int C, int K, int ks, int tile_ic, int oc_per_wave,
                              const int32_t* oc_order, void* stream, tetris_g950** out) {
  return tetris::pack_device(d_filter, C, K, ks, tile_ic, oc_per_wave, oc_order, static_cast<hipStream_t>(stream), out);
}

int tetris_g950_create(const float* h_filter, int C, int K, int ks, int tile_ic, int oc_per_wave,
                       const int32_t* oc_order, void* stream, tetris_g950** out) {
  if (!h_filter) return tetris::fail(TETRIS_EINVAL, "null filter");
  if (C <= 0 || K <= 0 || ks <= 0) return tetris::fail(TETRIS_EINVAL, "bad filter shape C=%d K=%d ks=%d", C, K, ks);
  float* d = nullptr;
  const size_t bytes = sizeof(float) * (size_t)C * K * ks * ks;
  TETRIS_HIP(hipMalloc(&d, bytes));
  hipError_t e = hipMemcpyAsync(d, h_filter, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream));
  int rc = e == hipSuccess ? TETRIS_OK : tetris::fail(TETRIS_EHIP, "filter upload failed: %s", hipGetErrorString(e));
  if (rc == TETRIS_OK)
    rc = tetris::pack_device(d, C, K, ks, tile_ic, oc_per_wave, oc_order, static_cast<hipStream_t>(stream), out);
  (void)hipStreamSynchronize(static_cast<hipStream_t>(stream));
  (void)hipFree(d);
  return rc;
}

void tetris_g950_destroy(tetris_g950* p) {
  if (!p) return;
  for (auto& kv : p->bound) (void)hipFree(kv.second);
  (void)hipFree(p->d_grp_off);
  (void)hipFree(p->d_grp_nnz);
  (void)hipFree(p->d_position);
  (void)hipFree(p->d_values);
  (void)hipFree(p->d_oc_order);
  (void)hipFree(p->d_pgrp_off);
  (void)hipFree(p->d_pgrp_pair);
  (void)hipFree(p->d_zero_pair);
  for (auto& kv : p->partial) (void)hipFree(kv.second.ptr);
  for (float* d : p->retired) (void)hipFree(d);
  delete p;
}

int tetris_g950_host_arrays(tetris_g950* p, tetris_g950_arrays* out) {
  if (!p || !out) return tetris::fail(TETRIS_EINVAL, "null argument");
  const int nseg = p->groups * p->stages;
  std::lock_guard<std::mutex> lock(p->mu);
  if (p->h_grp_off.empty()) {
    p->h_grp_off.resize(nseg + 1);
    p->h_grp_nnz.resize(nseg);
    p->h_position.resize(p->n_entries);
    p->h_values.resize(p->n_entries);
    p->h_oc_order.resize(p->slots);
    TETRIS_HIP(hipMemcpy(p->h_grp_off.data(), p->d_grp_off, sizeof(int32_t) * (nseg + 1), hipMemcpyDeviceToHost));
    TETRIS_HIP(hipMemcpy(p->h_grp_nnz.data(), p->d_grp_nnz, sizeof(int32_t) * nseg, hipMemcpyDeviceToHost));
    if (p->n_entries) {
      TETRIS_HIP(hipMemcpy(p->h_position.data(), p->d_position, sizeof(int32_t) * p->n_entries, hipMemcpyDeviceToHost));
      TETRIS_HIP(hipMemcpy(p->h_values.data(), p->d_values, sizeof(float) * p->n_entries, hipMemcpyDeviceToHost));
    }
    TETRIS_HIP(hipMemcpy(p->h_oc_order.data(), p->d_oc_order, sizeof(int32_t) * p->slots, hipMemcpyDeviceToHost));
  }
  out->grp_offsets = p->h_grp_off.data(); out->n_grp_offsets = nseg + 1;
  out->grp_nnz = p->h_grp_nnz.data();     out->n_grp_nnz = nseg;
  out->position = p->h_position.data();   out->n_entries = p->n_entries;
  out->values = p->h_values.data();
  out->oc_order = p->h_oc_order.data();   out->n_slots = p->slots;
  out->stages = p->stages; out->tile_ic = p->tile_ic; out->oc_per_wave = p->g; out->nnz = p->nnz;
  return TETRIS_OK;
}

}  // extern "C"
