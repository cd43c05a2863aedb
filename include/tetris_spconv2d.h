/* C ABI of the MI355X (gfx950) filter-sparse conv2d engine.
 *
 * Every entry point replaces one interface of the reference's spconv2d / spf path (file:line are
 * relative to the reference checkout).  Pointers named h_* are host memory, d_* device memory of the
 * current HIP device.  All tensors are fp32; indices are int32.  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  Every function returns 0 on success or a TETRIS_E* code;
 * tetris_last_error() gives the message of the calling thread's last failure.  Nothing here exits
 * the process (the reference's checkCudaErrors prints and calls exit, Tetris/cuda_utils.h:9-16).
 */
#ifndef TETRIS_SPCONV2D_H_
#define TETRIS_SPCONV2D_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  TETRIS_OK = 0,
  TETRIS_EINVAL = 1,      /* bad argument (shape, NULL, ks > 7, ...) */
  TETRIS_EHIP = 2,        /* a HIP call failed */
  TETRIS_EUNSUPPORTED = 3,/* reference behaviour undefined for this input (see tetris_spf_create) */
  TETRIS_ENOTFOUND = 4,   /* raw device arrays not produced by a live tetris_spf handle; or no launch plan prepared */
  TETRIS_EIO = 5          /* weight file cannot be opened or is truncated */
};

/* The reference's two compile-time packer macros (Tetris/spconv2d_utils.h:66, :80), as run-time flags. */
#define TETRIS_BANK_OPTIMIZE 1u
#define TETRIS_REORDER_OUT_CHANNEL 2u

const char* tetris_last_error(void);
const char* tetris_version(void);

/* ------------------------------------------------------------------------------------------------
 * Weight preprocessing, reference layout ("SPF").
 * Replaces: struct SparseFilter<float,int,int> -- constructor Tetris/spconv2d_utils.h:25-265,
 * destructor :267-273, getters :495-500, public vectors :505-509.
 * The five arrays are byte-identical to the reference's for the same arguments and macro set.
 * TETRIS_EUNSUPPORTED is returned when Bank-SR would read its 32 bank flags out of range
 * (spconv2d_utils.h:184 indexes them by an entry index), where the reference's result is undefined.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tetris_spf tetris_spf;

int tetris_spf_create(const float* h_filter_oihw, int in_channel, int out_channel, int kernel_size, int tile_ic,
                      int apply_reorder, int apply_vectorize, unsigned flags, tetris_spf** out);
void tetris_spf_destroy(tetris_spf* f);

typedef struct tetris_spf_arrays {
  const int32_t* offsets;        int64_t n_offsets;         /* offsets_         */
  const int32_t* stage_len;      int64_t n_stage_len;       /* stage_len_       */
  const int32_t* position;       int64_t n_position;        /* position_        */
  const float*   values;         int64_t n_values;          /* values_          */
  const int32_t* oc_permutation; int64_t n_oc_permutation;  /* oc_permutation_  */
  int64_t nnz;                   /* nnz_ (counted on the apply_reorder == 0 path only, like the reference) */
  int32_t tile_ic;               /* GetTileIC() */
} tetris_spf_arrays;

int tetris_spf_host_arrays(const tetris_spf* f, tetris_spf_arrays* out);   /* the public vectors */
/* GetDevice*(): the device copies are made on the first call (the reference uploads in its constructor). */
int tetris_spf_device_arrays(tetris_spf* f, tetris_spf_arrays* out);

/* ------------------------------------------------------------------------------------------------
 * Weight preprocessing, gfx950 layout: a device pass (count, scan, scatter) over the dense OIHW
 * filter.  Output-channel slots are taken `oc_per_wave` at a time (one group per wave of the conv
 * kernel); per (group, input-channel stage) it writes ONE stream with the group's non-zero entries,
 * position by position (channel, row, column ascending; slots ascending inside a position), padded
 * with zero entries to a multiple of 8 so that a wave fetches eight (position, value) pairs with one
 * 64-byte scalar load.  The position word is the reference's s | r<<3 | (ic % tile_ic)<<6
 * (Tetris/spconv2d_utils.h:91) with the slot's index inside its group in bits 24..31.
 * No reference counterpart for the layout; it plays the role of the SparseFilter constructor for the
 * HIP kernel.  `oc_order` (may be NULL = identity) lists, slot by slot, which output channel a slot
 * computes -- pass a tetris_spf's oc_permutation to keep the reference's channel regrouping.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tetris_g950 tetris_g950;

int tetris_g950_create(const float* h_filter_oihw, int in_channel, int out_channel, int kernel_size, int tile_ic,
                       int oc_per_wave, const int32_t* oc_order, void* stream, tetris_g950** out);
/* Same, from a filter already resident in device memory. */
int tetris_g950_create_device(const float* d_filter_oihw, int in_channel, int out_channel, int kernel_size,
                              int tile_ic, int oc_per_wave, const int32_t* oc_order, void* stream,
                              tetris_g950** out);
void tetris_g950_destroy(tetris_g950* p);

typedef struct tetris_g950_arrays {
  const int32_t* grp_offsets; int64_t n_grp_offsets; /* [groups*stages+1], entry index, multiples of 8  */
  const int32_t* grp_nnz;     int64_t n_grp_nnz;     /* [groups*stages], real entries in the stream     */
  const int32_t* position;    int64_t n_entries;     /* s | r<<3 | (ic % tile_ic)<<6 | slot-in-group<<24 */
  const float*   values;                             /* 0.0f for padding                                */
  const int32_t* oc_order;    int64_t n_slots;       /* output channel of each slot, -1 for padding     */
  int32_t stages, tile_ic, oc_per_wave;
  int64_t nnz;
} tetris_g950_arrays;

/* Copies the packed arrays to host memory owned by the handle (valid until it is destroyed). */
int tetris_g950_host_arrays(tetris_g950* p, tetris_g950_arrays* out);

/* ------------------------------------------------------------------------------------------------
 * Tile shape of the conv kernel.  Replaces the template arguments <TILE_IC, TILE_H, TILE_W> of the
 * reference launcher and its exhaustive table (Tetris/spconv2d.cc:90-329).  On launch, tile_ic and
 * oc_per_wave must be the ones the pack was created with; a NULL tile means "choose for me" and needs
 * a pack created with the tile_ic and oc_per_wave that tetris_tile_select returns for the shape.
 * ---------------------------------------------------------------------------------------------- */
typedef struct tetris_tile {
  int32_t lanes_w;     /* active lanes across a tile row (1..62); the tile is 4*lanes_w columns wide.  A tile at
                          least twice (four times) as wide as the output puts 2 (4) images side by side.
                          64 = the flat tile of 1x1 layers without padding (any stride): a lane owns four
                          consecutive pixels of the image (of the sub-grid a strided layer reads), 64 lanes a run of
                          256; takes waves = 8 or 16 */
  int32_t quads;       /* 4-pixel groups per lane (1, 2 or 4)                                      */
  int32_t oc_per_wave; /* output channels a wave accumulates at once; oc_per_wave*4*quads <= 128 (64 when waves = 16) */
  int32_t waves;       /* waves per workgroup (1, 2, 4, 8 or 16); it computes waves*oc_per_wave channels */
  int32_t tile_ic;     /* input channels staged in LDS at a time                                   */
  int32_t csplit;      /* workgroups that share an output tile, each reducing a slice of the input-channel stages
                          into partial sums that are added afterwards (for layers with too few pixels to fill the
                          GPU): 1 = none, 2..8 (each slice needs at least two stages), 0 = the library's rule --
                          split while fewer than half of the GPU's wave slots would be used */
} tetris_tile;

/* Unmeasured selection: a built-in table of tiles measured on MI355X for the layer shapes of the benchmark
 * suites (csrc/tuned_tiles.inc, made by tetris_amd/tune.py); for other shapes the tile of the most similar
 * measured layer of the same kernel size and stride, refitted to the image width; else the first choice of a
 * cycle model. */
int tetris_tile_select(int batch, int img_h, int img_w, int in_channel, int out_channel, int kernel_size, int stride,
                       int padding, tetris_tile* out);

/* Persisted tile selection: reads rows `{N, H, W, C, K, ks, stride, pad, {lanes_w, quads, oc_per_wave, waves,
 * tile_ic}},` (the format of csrc/tuned_tiles.inc, which `python -m tetris_amd.tune --out FILE` writes from
 * tetris_tile_autotune runs; other lines are skipped) and makes tetris_tile_select, and every entry point that
 * chooses the tile itself, answer from them before the built-in table.  Plays the part of the reference's static
 * per-layer cache of the exhaustive search (Tetris/spconv2d.cc:90, 285-329), kept across processes.  A row whose
 * tile the kernel's checks refuse is ignored at look-up.  *rows_out (may be NULL) receives the rows read.
 * Process-wide; may be called several times (later files win). */
int tetris_tile_table_load(const char* path, int* rows_out);

/* Switches for ablation runs, the counterpart of the reference's build variants (-DBANK_OPTIMIZE / -DREORDER_OUT_CHANNEL
 * and its ablation binaries, evalution/script/build_ablation.sh:12-18, Tetris/ablation_kernel.cu).  Process-wide; they
 * act on launch plans made afterwards (a pack keeps the plans it already has).  The initial value is taken from the
 * environment variable TETRIS_OPTIONS (a number) when it is set, else 0. */
#define TETRIS_OPT_PAIRS 1u        /* halo'd kernels walk streams rearranged into pairs of entries that share one LDS read, then singles */
#define TETRIS_OPT_NO_BANK_RULE 2u /* LDS rows packed densely: the lane-row pitch rule that keeps 16-byte LDS reads conflict-free is off */
/* tetris_spconv2d_time and tetris_tile_autotune evict the caches (a pass over a 512 MiB buffer the library keeps until
 * the process ends) before every timed launch and time the launches one by one.  A layer in the middle of a network
 * finds its input, its weights and its code in HBM, and the tile that wins from warm caches, as back-to-back launches
 * of one layer measure it (the reference's protocol, Tetris/spconv2d.cc:44-68), is not always the one that wins there. */
#define TETRIS_OPT_COLD_TIMING 4u
/* tetris_spconv2d_launch_spf / _spf_arrays take a set of device arrays they have already decoded once as unchanged:
 * no read-back, no hash, no synchronisation -- the launch is then as asynchronous as tetris_spconv2d_launch.  A caller
 * that rewrites the arrays in place says so with tetris_spf_invalidate. */
#define TETRIS_OPT_TRUST_SPF_ARRAYS 8u
/* Layers whose channel reduction is split over workgroups add their partial sums inside the conv kernel -- the last
 * wave of every (output tile, wave) pair to finish reads the slices back through L2 and adds them -- instead of in a
 * second kernel.  Same bits either way.  Measured slower on every suite (the adding wave's loads are a chain of L2
 * round trips at the end of the kernel, where nothing hides them), so it is a switch for comparing the two, off by
 * default. */
#define TETRIS_OPT_ADD_IN_KERNEL 16u
/* Whether split layers add their slices inside the conv kernel on the current GPU: TETRIS_OPT_ADD_IN_KERNEL is on and
 * the workgroups whose ids are equal modulo 8 run on one XCD (they then share an L2), which a probe kernel checks once
 * per device.  No reference counterpart.  Synchronises the device the first time. */
int tetris_split_layers_add_in_kernel(int* yes);
int tetris_options_set(unsigned flags);
unsigned tetris_options_get(void);

/* What this GPU delivers to a plain device copy (GB/s, read + write bytes of a 256 MiB buffer) and to a loop of
 * independent fp32 FMAs (TFLOP/s, non-packed), for reading roofline fractions against measured ceilings as well
 * as nominal ones.  No reference counterpart (the reference prints milliseconds and "T" per layer only,
 * Tetris/spconv2d.cc:357-358).  Allocates 512 MiB for its duration; synchronises `stream`.  Either output may
 * be NULL. */
int tetris_measure_peaks(void* stream, float* copy_gbs_out, float* fma_tflops_out);

/* Output-channel order for tetris_g950_create that evens out the work of the waves of a workgroup of `tile`
 * (uses tile->oc_per_wave, waves and tile_ic).  Plays the part of SparseFilter::ReorderOutChannel
 * (Tetris/spconv2d_utils.h:275-420) for the HIP kernel: channels sorted by their non-zero count are dealt to the
 * workgroups' blocks of waves*oc_per_wave slots in serpentine order, then inside a block each goes to the wave
 * where it adds least to the sum over input-channel stages of the busiest SIMD's entries (waves w, w+4, ... share
 * a SIMD), then of the busiest wave's.  On pruned networks,
 * whose channels differ widely in density, the busiest wave of a stage holds 1.2-1.5x the mean in file order.
 * `order_out` receives a permutation of 0..out_channel-1.  Pure host code. */
int tetris_oc_order_balanced(const float* h_filter_oihw, int in_channel, int out_channel, int kernel_size,
                             const tetris_tile* tile, int32_t* order_out);

/* Measured selection, the counterpart of GetTetrisSparseConv2dTime (Tetris/spconv2d.cc:72-329): packs the filter
 * for the `max_candidates` (0 = 24) tile shapes the model of tetris_tile_select ranks best (each in the
 * output-channel order of tetris_oc_order_balanced for that tile), times each on the device with the real
 * weights (1 warm-up + 3 launches on zero-filled input), times the four fastest again (2 + 10 launches) and
 * returns the fastest and its milliseconds per launch.  Allocates and frees its own device buffers;
 * synchronises `stream`. */
int tetris_tile_autotune(const float* h_filter_oihw, int batch, int img_h, int img_w, int in_channel, int out_channel,
                         int kernel_size, int stride, int padding, int max_candidates, void* stream,
                         tetris_tile* out, float* ms_out);
/* The same search, returning the `max_out` fastest candidates (all of them timed again with 2 + 10 launches), fastest
 * first, with their milliseconds: what a tuner needs that wants to break near ties by something other than time --
 * tetris_amd/tune.py takes, among the tiles within two per cent of the fastest, the one that moves the fewest HBM
 * bytes by the FETCH_SIZE / WRITE_SIZE counters of rocprofv3.  out and ms_out (may be NULL) have room for max_out
 * entries; *n_out (may be NULL) receives how many were written. */
int tetris_tile_autotune_list(const float* h_filter_oihw, int batch, int img_h, int img_w, int in_channel,
                              int out_channel, int kernel_size, int stride, int padding, int max_candidates,
                              void* stream, tetris_tile* out, float* ms_out, int max_out, int* n_out);

/* ------------------------------------------------------------------------------------------------
 * Conv launch on device tensors.  Replaces: SparseConv2d<float,int,int,KS,STRIDE,TILE_IC,TILE_H,TILE_W>
 * (Tetris/spconv2d_kernel.cuh:14-21, Tetris/spconv2d_kernel.cu:163-188).  Asynchronous on `stream`.
 * d_input is NCHW [batch][in_channel][img_h][img_w], d_output NCHW [batch][out_channel][oh][ow] with
 * oh = (img_h + 2*padding - kernel_size)/stride + 1 (the reference keeps NHWC on the device; its host
 * entry points below take and return NCHW, as here).  A layer with very few pixels per image is computed
 * by several workgroups per output tile: each writes partial sums to a scratch buffer owned by `p` and a second
 * kernel of the same launch adds them, in a fixed order, into d_output.  `p` keeps one such buffer per stream it is
 * launched on (made by tetris_g950_prepare or by the first such launch on that stream, freed with `p`), so launches
 * of one pack on different streams do not disturb each other; two launches on ONE stream are ordered by the stream.
 * The first launch of an (input shape, tile) pair also makes its launch plan (a device allocation and a small
 * kernel); it is refused with TETRIS_EINVAL while `stream` is being captured -- call tetris_g950_prepare before.
 * ---------------------------------------------------------------------------------------------- */
int tetris_spconv2d_launch(tetris_g950* p, const float* d_input, float* d_output, int batch, int img_h, int img_w,
                           int stride, int padding, const tetris_tile* tile, void* stream);

/* tetris_spconv2d_launch with the activation that follows the layer done on the way out, instead of by a second pass
 * over the tensor (tetris_relu_maxpool): the sums never reach memory.  No counterpart in the reference, whose layers
 * are timed one by one without activations.  TETRIS_ACT_RELU: d_output = max(conv, 0), same shape, every tile.
 * TETRIS_ACT_RELU_POOL2: ReLU then 2x2 max-pooling of stride 2, d_output is [batch][out_channel][oh/2][ow/2] (an odd
 * last row or column is dropped); a split layer pools in its adding kernel, any other layer inside the conv kernel,
 * which needs a halo'd tile (not the flat tile of pointwise layers) with an even number of lanes per row and of rows
 * per unit -- otherwise TETRIS_EUNSUPPORTED and nothing is launched (tetris_spconv2d_act_supported tells beforehand,
 * in *supported; launch with TETRIS_ACT_RELU and pool with tetris_relu_maxpool then).  Results are
 * bit-identical to tetris_spconv2d_launch followed by tetris_relu_maxpool.  Plans, scratch and graph capture as for
 * tetris_spconv2d_launch. */
/* How a layer is cut into workgroups for a tile, without launching anything: what the launcher derives from
 * (input shape, tile) before it launches.  No reference counterpart (the reference's grid follows from its template
 * arguments, Tetris/spconv2d_kernel.cu:163-188). */
typedef struct tetris_launch_shape {
  int32_t workgroups;     /* unit_groups * channel_blocks * csplit */
  int32_t unit_groups;    /* workgroups along the output pixels (each `quads` units of up to 256 pixels) */
  int32_t channel_blocks; /* workgroups along the output channels (each waves * oc_per_wave channels) */
  int32_t csplit;         /* workgroups that share an output tile (the tile's value, or the rule's when that is 0) */
  int32_t stages;         /* input-channel stages of the whole reduction: ceil(in_channel / tile_ic) */
  int32_t lanes_used;     /* lanes of a wave that own pixels, out of 64 */
  int32_t kernel;         /* 2 single LDS tile, 3 three LDS buffers, 4 flat tile of pointwise layers */
  int32_t lds_bytes;      /* dynamic LDS of a workgroup */
  int64_t scratch_bytes;  /* tickets + partial sums a split layer needs (0 when csplit is 1) */
} tetris_launch_shape;
int tetris_launch_shape_of(tetris_g950* p, int batch, int img_h, int img_w, int stride, int padding,
                           const tetris_tile* tile, tetris_launch_shape* out);

#define TETRIS_ACT_NONE 0
#define TETRIS_ACT_RELU 1
#define TETRIS_ACT_RELU_POOL2 2
int tetris_spconv2d_launch_act(tetris_g950* p, const float* d_input, float* d_output, int batch, int img_h, int img_w,
                               int stride, int padding, const tetris_tile* tile, int activation, void* stream);
int tetris_spconv2d_act_supported(tetris_g950* p, int batch, int img_h, int img_w, int stride, int padding,
                                  const tetris_tile* tile, int activation, int* supported);

/* Makes everything tetris_spconv2d_launch would otherwise make on its first call for (input shape, tile) on
 * `stream`: the launch plan, the entries bound to the tile geometry and, for a split layer, the partial-sum buffer of
 * that stream.  After it returns, launches with the same arguments allocate nothing and can be captured into a HIP
 * graph.  Counterpart of the reference doing all its allocation in the SparseFilter constructor
 * (Tetris/spconv2d_utils.h:248-264) before the launcher runs. */
int tetris_g950_prepare(tetris_g950* p, int batch, int img_h, int img_w, int stride, int padding,
                        const tetris_tile* tile, void* stream);

/* tetris_spconv2d_launch for callers that cannot allocate device memory (code under HIP graph capture, serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  It allocates nothing: the launch plan
 * must exist already (tetris_g950_prepare or an earlier tetris_spconv2d_launch with the same shape and tile, else
 * TETRIS_ENOTFOUND), and the partial sums of a split layer go to a static device array of
 * TETRIS_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends (64 KiB of it are the
 * split layers' tickets).  A layer whose partial sums need more is refused with TETRIS_EINVAL.  All calls on one GPU share that array: calls that overlap in
 * time on one GPU (different streams or threads) race; calls on one stream are ordered by the stream.  Results are
 * bit-identical to tetris_spconv2d_launch's. */
#define TETRIS_NOALLOC_SCRATCH_BYTES (64u << 20)
int tetris_spconv2d_launch_noalloc(tetris_g950* p, const float* d_input, float* d_output, int batch, int img_h,
                                   int img_w, int stride, int padding, const tetris_tile* tile, void* stream);
size_t tetris_noalloc_scratch_bytes(void); /* bytes of the array the entry point may use right now */
/* Lets the entry point use only the first `bytes` of the array (0 or more than TETRIS_NOALLOC_SCRATCH_BYTES = all of
 * it); returns the limit now in force.  For harnesses that want a larger layer refused rather than run. */
size_t tetris_noalloc_scratch_limit(size_t bytes);

/* The reference launcher on the five device arrays of a SparseFilter (Tetris/spconv2d_kernel.cuh:14-21,
 * Tetris/spconv2d_kernel.cu:91-156): the convolution is computed FROM THE ARRAYS PASSED -- offsets, positions, values
 * and the output-channel permutation -- not from anything a handle remembers.  The arrays are hashed on the device at
 * every call (one pass over them and a stream synchronisation); the first call, and any call after their content has
 * changed (a caller that rewrites d_values in place), decodes them on the device into the kernel's own pack, whose
 * slots follow d_oc_permutation.  Decoded packs are cached per set of addresses (16 sets, least recently used first
 * out).  d_stage_len is accepted and not read, as in the reference's kernel.  tile_ic and vec_width are the
 * SparseFilter's TILE_IC (a template argument of the reference launcher) and entries per lane and step: 4
 * (apply_vectorize), 1, or 0 for the keep-as-is layout of apply_reorder = false (spconv2d_utils.h:38-61; then
 * d_oc_permutation may be NULL) -- the format of the reference's CSR-like baseline variant.  n_entries: how many
 * entries d_position and d_values hold (0: not known).  Before any kernel reads the arrays the offsets are copied to
 * the host and checked -- they start at 0, never decrease, step by multiples of vec_width and span at most n_entries
 * entries -- so a wrong out_channel, tile_ic or vec_width is TETRIS_EINVAL, not an out-of-range read on the device.
 * tile: NULL = the library chooses.  Not capturable into a HIP graph (it synchronises); capture
 * tetris_spconv2d_launch instead.  With TETRIS_OPT_TRUST_SPF_ARRAYS a set of arrays seen before is neither read back
 * nor hashed (see there). */
int tetris_spconv2d_launch_spf_arrays(const float* d_input, const int32_t* d_offsets, const int32_t* d_stage_len,
                                      const int32_t* d_oc_permutation, const int32_t* d_position, const float* d_values,
                                      float* d_output, int batch, int img_h, int img_w, int in_channel, int out_channel,
                                      int kernel_size, int stride, int padding, int tile_ic, int vec_width,
                                      int64_t n_entries, const tetris_tile* tile, void* stream);
/* Forgets what the two launchers above remember about the arrays whose values live at d_values: the next call decodes
 * them again.  For callers that rewrite the arrays in place under TETRIS_OPT_TRUST_SPF_ARRAYS. */
void tetris_spf_invalidate(const float* d_values);
/* The host-side check the launchers apply to a copy of d_offsets, usable on its own: n_offsets =
 * ceil(out_channel / 32) * stages + 1 (out_channel * stages + 1 for vec_width 0).  TETRIS_OK or TETRIS_EINVAL. */
int tetris_spf_check_offsets(const int32_t* h_offsets, int64_t n_offsets, int vec_width, int64_t n_entries);

/* Same, in the exact call shape of the reference launcher, which carries neither TILE_IC nor the vector width:
 * those two are taken from the live tetris_spf whose device arrays these are (found through d_values;
 * TETRIS_ENOTFOUND otherwise).  The content still comes from the arrays. */
int tetris_spconv2d_launch_spf(const float* d_input, const int32_t* d_offsets, const int32_t* d_stage_len,
                               const int32_t* d_oc_permutation, const int32_t* d_position, const float* d_values,
                               float* d_output, int batch, int img_h, int img_w, int in_channel, int out_channel,
                               int kernel_size, int stride, int padding, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Host-to-host entry points.
 * tetris_spconv2d_host  replaces CudaSparseConv2d<float,int,int>  (Tetris/spconv2d.cc:332-367)
 * tetris_spconv2d_spf_host replaces SparseConv2d_SPF<float,int,int> (Tetris/spf.cc:22-93)
 * h_input NCHW, h_filter OIHW, h_output NCHW.  Both upload, pack, time the launch with the reference's
 * protocol (30 warm-up + 100 timed launches between two events, Tetris/tensor_utils.h:10-11), and
 * download.  *ms_out (may be NULL) receives the mean milliseconds per launch.  `layout` is accepted
 * for source compatibility ("NHWC" in the reference's mains) and does not change the host layout.
 * tetris_spconv2d_host lets the library choose the tile and, with apply_reorder, packs in the balanced channel order.
 * tetris_spconv2d_spf_host follows the reference's fixed configuration instead: a SparseFilter with TILE_IC = 128,
 * always reordered (spf.cc:43-44; apply_reorder is ignored there as here) and built with `flags` (the reference's
 * -DBANK_OPTIMIZE / -DREORDER_OUT_CHANNEL), whose DEVICE ARRAYS feed the convolution (as
 * tetris_spconv2d_launch_spf_arrays does), run with one fixed tile -- lanes over a quarter of the output width (at
 * most 16), one quad, eight channels per wave, four waves, eight staged channels -- in place of <3, 1, 128, 2, 4>
 * (spf.cc:59-60); a shape that tile cannot run gets the library's choice.
 * ---------------------------------------------------------------------------------------------- */
int tetris_spconv2d_host(const float* h_input, const float* h_filter, float* h_output, int batch, int img_h,
                         int img_w, int in_channel, int out_channel, int kernel_size, int stride, int padding,
                         void* stream, const char* layout, int apply_reorder, float* ms_out);
int tetris_spconv2d_spf_host(const float* h_input, const float* h_filter, float* h_output, int batch, int img_h,
                             int img_w, int in_channel, int out_channel, int kernel_size, int stride, int padding,
                             void* stream, const char* layout, int apply_reorder, unsigned flags, float* ms_out);
/* Replaces SparseConv2d_Baseline<float,int,int> (Tetris/baseline.cc:22-93), the first rung of the reference's
 * ablation ladder: as tetris_spconv2d_spf_host, but the SparseFilter is built with apply_reorder = false (baseline.cc:44:
 * the keep-as-is, CSR-like arrays of spconv2d_utils.h:38-61, no channel permutation) and those arrays feed the
 * convolution (tetris_spconv2d_launch_spf_arrays with vec_width 0), run with the same fixed tile at ONE output
 * channel per wave: every wave walks one stream per (output channel, stage) in file order, as a thread of the
 * reference's baseline kernel walks one run per (output channel, stage) (Tetris/ablation_kernel.cu:76-98); no
 * channels are merged into a stream and no channel order is chosen.  That is the step "Baseline -> SPF" measures. */
int tetris_spconv2d_baseline_host(const float* h_input, const float* h_filter, float* h_output, int batch, int img_h,
                                  int img_w, int in_channel, int out_channel, int kernel_size, int stride, int padding,
                                  void* stream, const char* layout, float* ms_out);

/* Times `repeat` back-to-back launches after `warm` untimed ones (TimingTetrisSparseConv2d,
 * Tetris/spconv2d.cc:29-69); mean milliseconds per launch in *ms_out. */
int tetris_spconv2d_time(tetris_g950* p, const float* d_input, float* d_output, int batch, int img_h, int img_w,
                         int stride, int padding, const tetris_tile* tile, void* stream, int warm, int repeat,
                         float* ms_out);

/* ------------------------------------------------------------------------------------------------
 * Glue for running a stack of layers as a whole network: d_output = max(d_input, 0) (pool = 1), or that followed by
 * 2x2 max-pooling of stride 2 (pool = 2; output img_h/2 x img_w/2 per plane, an odd last row or column is dropped).
 * NCHW fp32 on the device, asynchronous on `stream`; pool = 1 may run in place.  No counterpart in the reference,
 * whose mains time single layers on random inputs (Tetris/spconv2d.cc:369-450); it plays the part of the
 * activation and pooling layers that sit between the convolutions of the networks its weight files come from.
 * ---------------------------------------------------------------------------------------------- */
int tetris_relu_maxpool(const float* d_input, float* d_output, int batch, int channels, int img_h, int img_w, int pool,
                        void* stream);

/* ------------------------------------------------------------------------------------------------
 * Utilities of the path.
 * tetris_read_weight_file replaces ReadConfigAndDataFromFile (Tetris/tensor_utils.cc:55-82); header
 * order H W IC OC KS PAD STRIDE GROUPS; *h_filter_out is malloc'ed, release with tetris_free.
 * tetris_float_equal / tetris_tensor_equal replace FloatEqual / TensorEqual (:17-34).
 * ---------------------------------------------------------------------------------------------- */
int tetris_read_weight_file(const char* path, int32_t header[8], float** h_filter_out, int64_t* nnz_out);
void tetris_free(void* p);
int tetris_float_equal(float x, float y);
int64_t tetris_tensor_first_mismatch(const float* x, const float* y, int64_t len); /* -1 when equal */

#ifdef __cplusplus
}
#endif
#endif /* TETRIS_SPCONV2D_H_ */
