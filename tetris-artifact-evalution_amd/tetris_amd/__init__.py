"""Python face of libtetris_spconv2d.so (ctypes over the C ABI in include/tetris_spconv2d.h).

The names mirror the reference's C++ interface for this path so that tests read like its mains:
SparseFilter (Tetris/spconv2d_utils.h:23-515), SparseConv2d (Tetris/spconv2d_kernel.cuh:14-21),
CudaSparseConv2d (Tetris/spconv2d.cc:332-367), SparseConv2d_SPF (Tetris/spf.cc:22-93).
PyTorch, where used by callers, only provides device memory and streams; nothing here imports it.
There is no CPU fallback: if the library is missing, importing this module fails.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# TETRIS_SPCONV2D_LIB: another build of the same library (the sanitizer build of `make asan`)
LIB_PATH = os.environ.get("TETRIS_SPCONV2D_LIB") or os.path.join(os.path.dirname(_HERE), "libtetris_spconv2d.so")
if not os.path.exists(LIB_PATH):
    raise ImportError("libtetris_spconv2d.so is not built: run `make -C tetris-artifact-evalution_amd` "
                      "(or __graft_entry__.build())")


def _share_hip_runtime_with_torch():
    """A process can hold one HIP runtime.  PyTorch-ROCm wheels bundle their own libamdhip64 (same soname as
    the system one); if this library were loaded first it would bind the system copy and a later
    `import torch` would bring in a second runtime that finds no device.  So when torch is installed and not
    yet loaded, its copy is loaded first and both sides resolve to it."""
    import importlib.util
    import sys

    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.submodule_search_locations:
        return
    bundled = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
    if os.path.exists(bundled):
        C.CDLL(bundled, mode=C.RTLD_GLOBAL)


_share_hip_runtime_with_torch()
_lib = C.CDLL(LIB_PATH)

BANK_OPTIMIZE = 1
REORDER_OUT_CHANNEL = 2

OK, EINVAL, EHIP, EUNSUPPORTED, ENOTFOUND, EIO = range(6)
OPT_PAIRS, OPT_NO_BANK_RULE, OPT_COLD_TIMING, OPT_TRUST_SPF_ARRAYS, OPT_ADD_IN_KERNEL = 1, 2, 4, 8, 16  # tetris_options_set
ACT_NONE, ACT_RELU, ACT_RELU_POOL2 = 0, 1, 2  # tetris_spconv2d_launch_act


class TetrisError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("tetris error %d: %s" % (code, msg))
        self.code = code


class _SpfArrays(C.Structure):
    _fields_ = [("offsets", C.c_void_p), ("n_offsets", C.c_int64), ("stage_len", C.c_void_p), ("n_stage_len", C.c_int64),
                ("position", C.c_void_p), ("n_position", C.c_int64), ("values", C.c_void_p), ("n_values", C.c_int64),
                ("oc_permutation", C.c_void_p), ("n_oc_permutation", C.c_int64), ("nnz", C.c_int64),
                ("tile_ic", C.c_int32)]


class _G950Arrays(C.Structure):
    _fields_ = [("grp_offsets", C.c_void_p), ("n_grp_offsets", C.c_int64), ("grp_nnz", C.c_void_p),
                ("n_grp_nnz", C.c_int64), ("position", C.c_void_p), ("n_entries", C.c_int64), ("values", C.c_void_p),
                ("oc_order", C.c_void_p), ("n_slots", C.c_int64), ("stages", C.c_int32), ("tile_ic", C.c_int32),
                ("oc_per_wave", C.c_int32), ("nnz", C.c_int64)]


class Tile(C.Structure):
    """tetris_tile: lanes_w, quads, oc_per_wave, waves, tile_ic (all zero = let the library choose) and csplit
    (slices of the channel reduction: 0 = the library's rule, 1 = none, 2..8)."""
    _fields_ = [("lanes_w", C.c_int32), ("quads", C.c_int32), ("oc_per_wave", C.c_int32), ("waves", C.c_int32),
                ("tile_ic", C.c_int32), ("csplit", C.c_int32)]

    def as_list(self):
        """[lanes_w, quads, oc_per_wave, waves, tile_ic], plus csplit when the tile fixes it."""
        five = [self.lanes_w, self.quads, self.oc_per_wave, self.waves, self.tile_ic]
        return five + [self.csplit] if self.csplit else five

    def __repr__(self):
        return "Tile(lanes_w=%d, quads=%d, oc_per_wave=%d, waves=%d, tile_ic=%d%s)" % (
            self.lanes_w, self.quads, self.oc_per_wave, self.waves, self.tile_ic,
            ", csplit=%d" % self.csplit if self.csplit else "")


class LaunchShape(C.Structure):
    """tetris_launch_shape: how a layer is cut into workgroups for a tile."""
    _fields_ = [("workgroups", C.c_int32), ("unit_groups", C.c_int32), ("channel_blocks", C.c_int32),
                ("csplit", C.c_int32), ("stages", C.c_int32), ("lanes_used", C.c_int32), ("kernel", C.c_int32),
                ("lds_bytes", C.c_int32), ("scratch_bytes", C.c_int64)]


_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i32p_opt = C.c_void_p

_lib.tetris_last_error.restype = C.c_char_p
_lib.tetris_version.restype = C.c_char_p
_lib.tetris_spf_create.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_uint,
                                   C.POINTER(C.c_void_p)]
_lib.tetris_spf_destroy.argtypes = [C.c_void_p]
_lib.tetris_spf_destroy.restype = None
_lib.tetris_spf_host_arrays.argtypes = [C.c_void_p, C.POINTER(_SpfArrays)]
_lib.tetris_spf_device_arrays.argtypes = [C.c_void_p, C.POINTER(_SpfArrays)]
_lib.tetris_g950_create.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i32p_opt, C.c_void_p,
                                    C.POINTER(C.c_void_p)]
_lib.tetris_g950_create_device.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _i32p_opt,
                                           C.c_void_p, C.POINTER(C.c_void_p)]
_lib.tetris_g950_destroy.argtypes = [C.c_void_p]
_lib.tetris_g950_destroy.restype = None
_lib.tetris_g950_host_arrays.argtypes = [C.c_void_p, C.POINTER(_G950Arrays)]
_lib.tetris_options_set.argtypes = [C.c_uint]
_lib.tetris_options_get.restype = C.c_uint
_lib.tetris_tile_select.argtypes = [C.c_int] * 8 + [C.POINTER(Tile)]
_lib.tetris_tile_table_load.argtypes = [C.c_char_p, C.POINTER(C.c_int)]
_lib.tetris_measure_peaks.argtypes = [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]
_lib.tetris_relu_maxpool.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_void_p]
_lib.tetris_spconv2d_launch_act.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [
    C.POINTER(Tile), C.c_int, C.c_void_p]
_lib.tetris_spconv2d_act_supported.argtypes = [C.c_void_p] + [C.c_int] * 5 + [C.POINTER(Tile), C.c_int,
                                               C.POINTER(C.c_int)]
_lib.tetris_oc_order_balanced.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.POINTER(Tile),
                                          np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")]
_lib.tetris_tile_autotune.argtypes = [_f32p] + [C.c_int] * 9 + [C.c_void_p, C.POINTER(Tile), C.POINTER(C.c_float)]
_lib.tetris_tile_autotune_list.argtypes = [_f32p] + [C.c_int] * 9 + [C.c_void_p, C.POINTER(Tile), C.POINTER(C.c_float),
                                           C.c_int, C.POINTER(C.c_int)]
_lib.tetris_spconv2d_launch.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.POINTER(Tile),
                                                                                                C.c_void_p]
_lib.tetris_g950_prepare.argtypes = [C.c_void_p] + [C.c_int] * 5 + [C.POINTER(Tile), C.c_void_p]
_lib.tetris_spconv2d_launch_noalloc.argtypes = _lib.tetris_spconv2d_launch.argtypes
_lib.tetris_launch_shape_of.argtypes = [C.c_void_p] + [C.c_int] * 5 + [C.POINTER(Tile), C.POINTER(LaunchShape)]
_lib.tetris_noalloc_scratch_bytes.restype = C.c_size_t
_lib.tetris_noalloc_scratch_limit.argtypes = [C.c_size_t]
_lib.tetris_noalloc_scratch_limit.restype = C.c_size_t
_lib.tetris_spconv2d_launch_spf.argtypes = [C.c_void_p] * 7 + [C.c_int] * 8 + [C.c_void_p]
_lib.tetris_spconv2d_time.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [
    C.POINTER(Tile), C.c_void_p, C.c_int, C.c_int, C.POINTER(C.c_float)]
_lib.tetris_spconv2d_launch_spf_arrays.argtypes = [C.c_void_p] * 7 + [C.c_int] * 10 + [C.c_int64, C.POINTER(Tile),
                                                                                    C.c_void_p]
_lib.tetris_spf_invalidate.argtypes = [C.c_void_p]
_lib.tetris_spf_invalidate.restype = None
_lib.tetris_spf_check_offsets.argtypes = [np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS"), C.c_int64, C.c_int,
                                          C.c_int64]
_lib.tetris_spconv2d_host.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 8 + [C.c_void_p, C.c_char_p, C.c_int,
                                                                            C.POINTER(C.c_float)]
_lib.tetris_spconv2d_spf_host.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 8 + [C.c_void_p, C.c_char_p, C.c_int, C.c_uint,
                                                                                C.POINTER(C.c_float)]
_lib.tetris_read_weight_file.argtypes = [C.c_char_p, C.POINTER(C.c_int32), C.POINTER(C.POINTER(C.c_float)),
                                         C.POINTER(C.c_int64)]
_lib.tetris_free.argtypes = [C.c_void_p]
_lib.tetris_free.restype = None
_lib.tetris_float_equal.argtypes = [C.c_float, C.c_float]
_lib.tetris_tensor_first_mismatch.argtypes = [_f32p, _f32p, C.c_int64]
_lib.tetris_tensor_first_mismatch.restype = C.c_int64


def _check(rc):
    if rc != 0:
        raise TetrisError(rc, _lib.tetris_last_error().decode())


def version():
    return _lib.tetris_version().decode()


def out_extent(size, pad, ks, stride):
    return (size + 2 * pad - ks) // stride + 1


def _np_view(ptr, n, dtype):
    if not ptr or n == 0:
        return np.zeros(0, dtype)
    ct = C.c_float if dtype == np.float32 else C.c_int32
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(ct)), shape=(int(n),)).copy()


class SparseFilter:
    """SparseFilter<float,int,int>(filter, in_channel, out_channel, kernel_size, TILE_IC=32,
    apply_reorder=False, apply_vectorize=True); `flags` carries the reference's build macros."""

    def __init__(self, filter, in_channel, out_channel, kernel_size, TILE_IC=32, apply_reorder=False,
                 apply_vectorize=True, flags=0):
        w = np.ascontiguousarray(filter, np.float32).reshape(out_channel, in_channel, kernel_size, kernel_size)
        self._h = C.c_void_p()
        _check(_lib.tetris_spf_create(w, in_channel, out_channel, kernel_size, TILE_IC, int(apply_reorder),
                                      int(apply_vectorize), flags, C.byref(self._h)))
        a = _SpfArrays()
        _check(_lib.tetris_spf_host_arrays(self._h, C.byref(a)))
        self.in_channel_, self.out_channel_, self.kernel_size_ = in_channel, out_channel, kernel_size
        self.TILE_IC_ = int(a.tile_ic)
        self.nnz_ = int(a.nnz)
        self.offsets_ = _np_view(a.offsets, a.n_offsets, np.int32)
        self.stage_len_ = _np_view(a.stage_len, a.n_stage_len, np.int32)
        self.position_ = _np_view(a.position, a.n_position, np.int32)
        self.values_ = _np_view(a.values, a.n_values, np.float32)
        self.oc_permutation_ = _np_view(a.oc_permutation, a.n_oc_permutation, np.int32)
        self._dev = None

    def _device(self):
        if self._dev is None:
            a = _SpfArrays()
            _check(_lib.tetris_spf_device_arrays(self._h, C.byref(a)))
            self._dev = a
        return self._dev

    def GetDeviceOffsets(self):
        return self._device().offsets

    def GetDeviceStageLen(self):
        return self._device().stage_len

    def GetDeviceValues(self):
        return self._device().values

    def GetDevicePosition(self):
        return self._device().position

    def GetDeviceOCPermutation(self):
        return self._device().oc_permutation

    def GetTileIC(self):
        return self.TILE_IC_

    def arrays(self):
        return (self.offsets_, self.stage_len_, self.position_, self.values_, self.oc_permutation_)

    def close(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.tetris_spf_destroy(self._h)
            self._h = None

    __del__ = close


class G950Filter:
    """The gfx950 pack the HIP kernel consumes (tetris_g950_create / _create_device).

    `G950Filter.for_tile(filter, tile)` makes the pack that a Tile from tile_select() needs."""

    @classmethod
    def for_tile(cls, filter, tile, oc_order=None, stream=0):
        """oc_order: None or "file" (file order), an int32 permutation, "balanced" (oc_order_balanced for this tile) or
        "reference" (the order the reference's ReorderOutChannel pass gives, spconv2d_utils.h:249-289)."""
        if isinstance(oc_order, str):
            if oc_order == "balanced":
                oc_order = oc_order_balanced(filter, tile)
            elif oc_order == "reference":
                oc_order = oc_order_reference(filter, tile.tile_ic)
            elif oc_order == "file":
                oc_order = None
            else:
                raise ValueError("oc_order: None, 'file', 'balanced', 'reference' or a permutation")
        return cls(filter, tile.tile_ic, tile.oc_per_wave, oc_order, stream)

    def __init__(self, filter, tile_ic, oc_per_wave, oc_order=None, stream=0, device_ptr=None, shape=None):
        if device_ptr is None:
            w = np.ascontiguousarray(filter, np.float32)
            K, Cc, ks, _ = w.shape
        else:
            K, Cc, ks, _ = shape
        order = None if oc_order is None else np.ascontiguousarray(oc_order, np.int32)
        optr = None if order is None else order.ctypes.data_as(C.c_void_p)
        self._h = C.c_void_p()
        if device_ptr is None:
            _check(_lib.tetris_g950_create(w, Cc, K, ks, tile_ic, oc_per_wave, optr, C.c_void_p(stream),
                                           C.byref(self._h)))
        else:
            _check(_lib.tetris_g950_create_device(C.c_void_p(device_ptr), Cc, K, ks, tile_ic, oc_per_wave, optr,
                                                  C.c_void_p(stream), C.byref(self._h)))
        self.K, self.C, self.ks, self.tile_ic, self.oc_per_wave = K, Cc, ks, tile_ic, oc_per_wave

    def host_arrays(self):
        a = _G950Arrays()
        _check(_lib.tetris_g950_host_arrays(self._h, C.byref(a)))
        return dict(grp_offsets=_np_view(a.grp_offsets, a.n_grp_offsets, np.int32),
                    grp_nnz=_np_view(a.grp_nnz, a.n_grp_nnz, np.int32),
                    position=_np_view(a.position, a.n_entries, np.int32),
                    values=_np_view(a.values, a.n_entries, np.float32),
                    oc_order=_np_view(a.oc_order, a.n_slots, np.int32), stages=int(a.stages), tile_ic=int(a.tile_ic),
                    oc_per_wave=int(a.oc_per_wave), nnz=int(a.nnz))

    def launch(self, d_input, d_output, batch, img_h, img_w, stride, padding, tile=None, stream=0):
        """Asynchronous conv on raw device pointers (NCHW in, NCHW out)."""
        _check(_lib.tetris_spconv2d_launch(self._h, C.c_void_p(d_input), C.c_void_p(d_output), batch, img_h, img_w,
                                           stride, padding, C.byref(tile) if tile is not None else None,
                                           C.c_void_p(stream)))

    def launch_act(self, d_input, d_output, batch, img_h, img_w, stride, padding, tile, activation, stream=0):
        """launch() with ReLU (ACT_RELU) or ReLU + 2x2 max-pooling (ACT_RELU_POOL2, output N x K x OH/2 x OW/2) done as
        the sums are written (tetris_spconv2d_launch_act)."""
        _check(_lib.tetris_spconv2d_launch_act(self._h, C.c_void_p(d_input), C.c_void_p(d_output), batch, img_h, img_w,
                                               stride, padding, C.byref(tile) if tile is not None else None,
                                               activation, C.c_void_p(stream)))

    def act_supported(self, batch, img_h, img_w, stride, padding, tile, activation):
        """Whether launch_act can do `activation` for this shape and tile (tetris_spconv2d_act_supported)."""
        yes = C.c_int()
        _check(_lib.tetris_spconv2d_act_supported(self._h, batch, img_h, img_w, stride, padding, C.byref(tile),
                                                  activation, C.byref(yes)))
        return bool(yes.value)

    def prepare(self, batch, img_h, img_w, stride, padding, tile=None, stream=0):
        """Makes the launch plan (and a split layer's partial-sum buffer on `stream`) ahead of the first launch."""
        _check(_lib.tetris_g950_prepare(self._h, batch, img_h, img_w, stride, padding,
                                        C.byref(tile) if tile is not None else None, C.c_void_p(stream)))

    def launch_shape(self, batch, img_h, img_w, stride, padding, tile):
        """How the layer is cut into workgroups for `tile` (tetris_launch_shape_of); nothing is launched."""
        out = LaunchShape()
        _check(_lib.tetris_launch_shape_of(self._h, batch, img_h, img_w, stride, padding, C.byref(tile), C.byref(out)))
        return out

    def launch_noalloc(self, d_input, d_output, batch, img_h, img_w, stride, padding, tile=None, stream=0):
        """launch() for callers that cannot allocate: needs prepare() first, uses the library's static scratch array."""
        _check(_lib.tetris_spconv2d_launch_noalloc(self._h, C.c_void_p(d_input), C.c_void_p(d_output), batch, img_h,
                                                   img_w, stride, padding, C.byref(tile) if tile is not None else None,
                                                   C.c_void_p(stream)))

    def time(self, d_input, d_output, batch, img_h, img_w, stride, padding, tile=None, stream=0, warm=30, repeat=100):
        ms = C.c_float()
        _check(_lib.tetris_spconv2d_time(self._h, C.c_void_p(d_input), C.c_void_p(d_output), batch, img_h, img_w,
                                         stride, padding, C.byref(tile) if tile is not None else None,
                                         C.c_void_p(stream), warm, repeat, C.byref(ms)))
        return float(ms.value)

    def close(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.tetris_g950_destroy(self._h)
            self._h = None

    __del__ = close


def options_set(flags):
    """Ablation switches (OPT_PAIRS, OPT_NO_BANK_RULE) for launch plans made from now on."""
    _check(_lib.tetris_options_set(flags))


def options_get():
    return int(_lib.tetris_options_get())


def tile_select(batch, img_h, img_w, in_channel, out_channel, kernel_size, stride, padding):
    t = Tile()
    _check(_lib.tetris_tile_select(batch, img_h, img_w, in_channel, out_channel, kernel_size, stride, padding,
                                   C.byref(t)))
    return t


def noalloc_scratch_bytes():
    """Size of the static device array launch_noalloc keeps the partial sums of split layers in."""
    return int(_lib.tetris_noalloc_scratch_bytes())


def noalloc_scratch_limit(nbytes):
    """Restricts launch_noalloc to the first `nbytes` of its array (0 = all of it); -> the limit in force."""
    return int(_lib.tetris_noalloc_scratch_limit(nbytes))


def tile_table_load(path):
    """Makes tile_select answer from the rows of `path` (format of csrc/tuned_tiles.inc, written by tetris_amd.tune)
    before the built-in table; -> number of rows read."""
    n = C.c_int()
    _check(_lib.tetris_tile_table_load(os.fsencode(path), C.byref(n)))
    return int(n.value)


def measure_peaks(stream=0):
    """-> (device copy GB/s, non-packed fp32 FMA TFLOP/s) measured on this GPU (tetris_measure_peaks)."""
    c, f = C.c_float(), C.c_float()
    _check(_lib.tetris_measure_peaks(C.c_void_p(stream), C.byref(c), C.byref(f)))
    return float(c.value), float(f.value)


def relu_maxpool(d_input, d_output, batch, channels, img_h, img_w, pool=1, stream=0):
    """d_output = max(d_input, 0), followed by 2x2 max-pooling of stride 2 when pool == 2 (tetris_relu_maxpool);
    device pointers to NCHW fp32, asynchronous on `stream`."""
    _check(_lib.tetris_relu_maxpool(C.c_void_p(d_input), C.c_void_p(d_output), batch, channels, img_h, img_w, pool,
                                    C.c_void_p(stream)))


def oc_order_balanced(filter, tile):
    """Output-channel order that evens out the waves of a workgroup of `tile` (tetris_oc_order_balanced)."""
    w = np.ascontiguousarray(filter, np.float32)
    K, Cc, ks, _ = w.shape
    order = np.empty(K, np.int32)
    _check(_lib.tetris_oc_order_balanced(w, Cc, K, ks, C.byref(tile), order))
    return order


def oc_order_reference(filter, tile_ic=32):
    """Output-channel order of the reference's ReorderOutChannel pass (spconv2d_utils.h:249-289) for this filter."""
    w = np.ascontiguousarray(filter, np.float32)
    K, Cc, ks, _ = w.shape
    f = SparseFilter(w, Cc, K, ks, TILE_IC=tile_ic, apply_reorder=True, flags=REORDER_OUT_CHANNEL)
    order = np.array(f.oc_permutation_, np.int32)
    f.close()
    return order


def tile_autotune(filter, batch, img_h, img_w, stride, padding, max_candidates=0, stream=0):
    """-> (Tile, ms per launch) of the fastest measured tile shape for this filter and input shape."""
    w = np.ascontiguousarray(filter, np.float32)
    K, Cc, ks, _ = w.shape
    t, ms = Tile(), C.c_float()
    _check(_lib.tetris_tile_autotune(w, batch, img_h, img_w, Cc, K, ks, stride, padding, max_candidates,
                                     C.c_void_p(stream), C.byref(t), C.byref(ms)))
    return t, float(ms.value)


def tile_autotune_list(filter, batch, img_h, img_w, stride, padding, max_candidates=0, max_out=4, stream=0):
    """-> [(Tile, ms per launch), ...]: the `max_out` fastest measured tile shapes, fastest first
    (tetris_tile_autotune_list)."""
    w = np.ascontiguousarray(filter, np.float32)
    K, Cc, ks, _ = w.shape
    tiles, ms, n = (Tile * max_out)(), (C.c_float * max_out)(), C.c_int()
    _check(_lib.tetris_tile_autotune_list(w, batch, img_h, img_w, Cc, K, ks, stride, padding, max_candidates,
                                          C.c_void_p(stream), tiles, ms, max_out, C.byref(n)))
    return [(Tile(tiles[i].lanes_w, tiles[i].quads, tiles[i].oc_per_wave, tiles[i].waves, tiles[i].tile_ic,
                  tiles[i].csplit), float(ms[i]))
            for i in range(n.value)]


def SparseConv2d(input, offsets, stage_len, oc_permutation, position, values, output, batch_size, img_h, img_w,
                 in_channel, out_channel, kernel_size, stride, padding, stream=0, TILE_IC=0, vec_width=4, tile=None,
                 n_entries=0):
    """The reference launcher's call shape on raw device pointers: computes from the arrays passed.  TILE_IC = 0: the
    arrays belong to a live SparseFilter, whose TILE_IC is looked up; else any arrays in that layout
    (vec_width 4, 1, or 0 for the keep-as-is layout of apply_reorder=False; n_entries: how many entries `position`
    and `values` hold, 0 if not known)."""
    if TILE_IC:
        _check(_lib.tetris_spconv2d_launch_spf_arrays(
            C.c_void_p(input), C.c_void_p(offsets), C.c_void_p(stage_len), C.c_void_p(oc_permutation), C.c_void_p(position),
            C.c_void_p(values), C.c_void_p(output), batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride,
            padding, TILE_IC, vec_width, n_entries, C.byref(tile) if tile is not None else None, C.c_void_p(stream)))
    else:
        _check(_lib.tetris_spconv2d_launch_spf(C.c_void_p(input), C.c_void_p(offsets), C.c_void_p(stage_len),
                                               C.c_void_p(oc_permutation), C.c_void_p(position), C.c_void_p(values),
                                               C.c_void_p(output), batch_size, img_h, img_w, in_channel, out_channel,
                                               kernel_size, stride, padding, C.c_void_p(stream)))


def split_layers_add_in_kernel():
    """Whether layers whose channel reduction is split add their slices inside the conv kernel on this GPU."""
    yes = C.c_int(0)
    _check(_lib.tetris_split_layers_add_in_kernel(C.byref(yes)))
    return bool(yes.value)


def spf_invalidate(values):
    """Forget what the raw launchers remember about the arrays whose values live at device address `values`."""
    _lib.tetris_spf_invalidate(C.c_void_p(values))


def spf_check_offsets(offsets, vec_width, n_entries=0):
    """The host-side check of a SparseFilter's offsets the raw launchers apply; raises TetrisError(EINVAL)."""
    o = np.ascontiguousarray(offsets, np.int32)
    _check(_lib.tetris_spf_check_offsets(o, len(o), vec_width, n_entries))


def _host_entry(fn, h_input, h_filter, batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride, padding,
                stream, layout, apply_reorder, *extra):
    x = np.ascontiguousarray(h_input, np.float32)
    w = np.ascontiguousarray(h_filter, np.float32)
    out = np.empty((batch_size, out_channel, out_extent(img_h, padding, kernel_size, stride),
                    out_extent(img_w, padding, kernel_size, stride)), np.float32)
    ms = C.c_float()
    _check(fn(x, w, out, batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride, padding,
              C.c_void_p(stream), layout.encode(), int(apply_reorder), *extra, C.byref(ms)))
    return out, float(ms.value)


def CudaSparseConv2d(h_input, h_filter, batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride,
                     padding, stream=0, layout="NHWC", apply_reorder=True):
    """-> (h_output NCHW, mean ms per launch)."""
    return _host_entry(_lib.tetris_spconv2d_host, h_input, h_filter, batch_size, img_h, img_w, in_channel,
                       out_channel, kernel_size, stride, padding, stream, layout, apply_reorder)


def SparseConv2d_SPF(h_input, h_filter, batch_size, img_h, img_w, in_channel, out_channel, kernel_size, stride,
                     padding, stream=0, layout="NHWC", apply_reorder=True, flags=BANK_OPTIMIZE | REORDER_OUT_CHANNEL):
    """The reference's fixed configuration (spf.cc): SparseFilter(TILE_IC=128, reordered, `flags`), its device arrays
    fed to the launcher, one fixed tile."""
    return _host_entry(_lib.tetris_spconv2d_spf_host, h_input, h_filter, batch_size, img_h, img_w, in_channel,
                       out_channel, kernel_size, stride, padding, stream, layout, apply_reorder, flags)


def ReadConfigAndDataFromFile(weight_file):
    """-> (dict H W IC OC KS PAD STRIDE GROUPS, filter OIHW, nnz); raises TetrisError(EIO) if unreadable."""
    hdr = (C.c_int32 * 8)()
    ptr = C.POINTER(C.c_float)()
    nnz = C.c_int64()
    _check(_lib.tetris_read_weight_file(weight_file.encode(), hdr, C.byref(ptr), C.byref(nnz)))
    h = dict(zip(("H", "W", "IC", "OC", "KS", "PAD", "STRIDE", "GROUPS"), [int(v) for v in hdr]))
    n = h["OC"] * h["IC"] * h["KS"] * h["KS"]
    w = np.ctypeslib.as_array(ptr, shape=(n,)).copy().reshape(h["OC"], h["IC"], h["KS"], h["KS"])
    _lib.tetris_free(ptr)
    return h, w, int(nnz.value)


def FloatEqual(x, y):
    return bool(_lib.tetris_float_equal(x, y))


def TensorEqual(x, y):
    x = np.ascontiguousarray(x, np.float32).ravel()
    y = np.ascontiguousarray(y, np.float32).ravel()
    return int(_lib.tetris_tensor_first_mismatch(x, y, x.size)) == -1
