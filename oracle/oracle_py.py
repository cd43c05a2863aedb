"""ctypes access to the CPU oracle (oracle/libtetris_oracle.so) and, when built, to the reference's own
tensor_utils.cc (oracle/_ref/libtetris_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg -- never by the shipped package.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
# The known-answer table recorded from the compiled reference used 1469598103934665603 as offset basis (the
# standard FNV-1a-64 basis 14695981039346656037 minus its last digit); inverting the recorded hashes of the
# identity permutation for K = 64, 128, 256 and 512 gives this one value each time.
FNV_BASIS = 1469598103934665603


def _load(path):
    if not os.path.exists(path):
        return None
    return C.CDLL(path)


# TETRIS_ORACLE_LIB: another build of the oracle (the sanitizer build of `make asan`)
_lib = _load(os.environ.get("TETRIS_ORACLE_LIB") or os.path.join(_HERE, "libtetris_oracle.so"))
_ref = _load(os.path.join(_HERE, "_ref", "libtetris_ref.so"))


def available():
    return _lib is not None


def ref_available():
    return _ref is not None


if _lib is not None:
    _lib.orc_host_conv2d.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 9
    _lib.orc_host_conv2d.restype = None
    _lib.orc_float_equal.argtypes = [C.c_float, C.c_float]
    _lib.orc_float_equal.restype = C.c_int
    _lib.orc_tensor_first_mismatch.argtypes = [_f32p, _f32p, C.c_int64]
    _lib.orc_tensor_first_mismatch.restype = C.c_int64
    _lib.orc_read_weight_file.argtypes = [C.c_char_p, C.POINTER(C.c_int32), C.POINTER(C.POINTER(C.c_float)),
                                          C.POINTER(C.c_int64)]
    _lib.orc_read_weight_file.restype = C.c_int
    _lib.orc_free.argtypes = [C.c_void_p]
    _lib.orc_nchw_to_nhwc.argtypes = [_f32p, _f32p] + [C.c_int] * 4
    _lib.orc_nhwc_to_nchw.argtypes = [_f32p, _f32p] + [C.c_int] * 4
    _lib.orc_spf_pack.argtypes = [_f32p] + [C.c_int] * 8
    _lib.orc_spf_pack.restype = C.c_void_p
    _lib.orc_pack_free.argtypes = [C.c_void_p]
    _lib.orc_pack_sizes.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
    for _n, _t in (("offsets", C.c_int32), ("stage_len", C.c_int32), ("position", C.c_int32), ("values", C.c_float),
                   ("perm", C.c_int32)):
        getattr(_lib, "orc_pack_" + _n).argtypes = [C.c_void_p]
        getattr(_lib, "orc_pack_" + _n).restype = C.POINTER(_t)
    _lib.orc_host_spconv2d.argtypes = [C.c_void_p, _f32p, _f32p] + [C.c_int] * 6
    _lib.orc_host_reorder_spconv2d.argtypes = [C.c_void_p, _f32p, _f32p] + [C.c_int] * 6
    _lib.orc_g950_pack.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    _lib.orc_g950_pack.restype = C.c_void_p
    _lib.orc_g950_free.argtypes = [C.c_void_p]
    _lib.orc_g950_sizes.argtypes = [C.c_void_p, C.POINTER(C.c_int64)]
    for _n, _t in (("grp_off", C.c_int32), ("grp_nnz", C.c_int32), ("position", C.c_int32), ("values", C.c_float),
                   ("order", C.c_int32)):
        getattr(_lib, "orc_g950_" + _n).argtypes = [C.c_void_p]
        getattr(_lib, "orc_g950_" + _n).restype = C.POINTER(_t)
    _lib.orc_g950_conv.argtypes = [C.c_void_p, _f32p, _f32p] + [C.c_int] * 6
    _lib.orc_fnv1a.argtypes = [C.c_void_p, C.c_int64, C.c_uint64]
    _lib.orc_fnv1a.restype = C.c_uint64
    _lib.orc_max_threads.restype = C.c_int

if _ref is not None:
    _ref.ref_host_conv2d.argtypes = [_f32p, _f32p, _f32p] + [C.c_int] * 8
    _ref.ref_float_equal.argtypes = [C.c_float, C.c_float]
    _ref.ref_float_equal.restype = C.c_int
    _ref.ref_read_weight_file.argtypes = [C.c_char_p, C.c_int, C.POINTER(C.c_int32)]
    _ref.ref_read_weight_file.restype = C.POINTER(C.c_float)
    _ref.ref_free.argtypes = [C.c_void_p]
    _ref.ref_nchw2nhwc.argtypes = [_f32p] + [C.c_int] * 4
    _ref.ref_nhwc2nchw.argtypes = [_f32p] + [C.c_int] * 4


def out_extent(size, pad, ks, stride):
    return (size + 2 * pad - ks) // stride + 1


def max_threads():
    return int(_lib.orc_max_threads())


def host_conv2d(x, w, stride, pad, threads=1):
    """Dense direct convolution, NCHW x OIHW -> NCHW (orc_host_conv2d)."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    n, c, h, wd = x.shape
    k, c2, ks, _ = w.shape
    assert c == c2
    out = np.empty((n, k, out_extent(h, pad, ks, stride), out_extent(wd, pad, ks, stride)), np.float32)
    _lib.orc_host_conv2d(x, w, out, n, h, wd, c, k, ks, stride, pad, threads)
    return out


def ref_host_conv2d(x, w, stride, pad):
    """The reference's own HostConv2d, compiled from its source."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    n, c, h, wd = x.shape
    k, _, ks, _ = w.shape
    out = np.empty((n, k, out_extent(h, pad, ks, stride), out_extent(wd, pad, ks, stride)), np.float32)
    _ref.ref_host_conv2d(x, w, out, n, h, wd, c, k, ks, stride, pad)
    return out


def nchw_to_nhwc(x):
    x = np.ascontiguousarray(x, np.float32)
    n, c, h, w = x.shape
    out = np.empty((n, h, w, c), np.float32)
    _lib.orc_nchw_to_nhwc(x, out, n, c, h, w)
    return out


def nhwc_to_nchw(x):
    x = np.ascontiguousarray(x, np.float32)
    n, h, w, c = x.shape
    out = np.empty((n, c, h, w), np.float32)
    _lib.orc_nhwc_to_nchw(x, out, n, c, h, w)
    return out


def ref_nchw_to_nhwc(x):
    """The reference's in-place NCHW2NHWC (tensor_utils.cc:85-108) on a copy."""
    x = np.array(x, np.float32, order="C")
    n, c, h, w = x.shape
    _ref.ref_nchw2nhwc(x, n, c, h, w)
    return x.reshape(n, h, w, c)


def ref_nhwc_to_nchw(x):
    """The reference's in-place NHWC2NCHW (tensor_utils.cc:110-134) on a copy."""
    x = np.array(x, np.float32, order="C")
    n, h, w, c = x.shape
    _ref.ref_nhwc2nchw(x, n, c, h, w)
    return x.reshape(n, c, h, w)


def float_equal(a, b):
    return bool(_lib.orc_float_equal(a, b))


def ref_float_equal(a, b):
    return bool(_ref.ref_float_equal(a, b))


def tensor_first_mismatch(a, b):
    a = np.ascontiguousarray(a, np.float32).ravel()
    b = np.ascontiguousarray(b, np.float32).ravel()
    return int(_lib.orc_tensor_first_mismatch(a, b, a.size))


def read_weight_file(path):
    """-> (header dict, filter OIHW float32, nnz) or raises FileNotFoundError."""
    hdr = (C.c_int32 * 8)()
    ptr = C.POINTER(C.c_float)()
    nnz = C.c_int64()
    rc = _lib.orc_read_weight_file(path.encode(), hdr, C.byref(ptr), C.byref(nnz))
    if rc != 0:
        raise FileNotFoundError(path)
    h = dict(zip(("H", "W", "IC", "OC", "KS", "PAD", "STRIDE", "GROUPS"), list(hdr)))
    n = h["OC"] * h["IC"] * h["KS"] * h["KS"]
    arr = np.ctypeslib.as_array(ptr, shape=(n,)).copy().reshape(h["OC"], h["IC"], h["KS"], h["KS"])
    _lib.orc_free(ptr)
    return h, arr, int(nnz.value)


def ref_read_weight_file(path, batch=1):
    hdr = (C.c_int32 * 8)()
    ptr = _ref.ref_read_weight_file(path.encode(), batch, hdr)
    h = dict(zip(("H", "W", "IC", "OC", "KS", "PAD", "STRIDE", "GROUPS"), list(hdr)))
    n = h["OC"] * h["IC"] * h["KS"] * h["KS"]
    arr = np.ctypeslib.as_array(ptr, shape=(n,)).copy().reshape(h["OC"], h["IC"], h["KS"], h["KS"])
    _ref.ref_free(ptr)
    return h, arr


class SpfPack:
    """Result of orc_spf_pack: the reference SparseFilter's five host arrays."""

    def __init__(self, w, tile_ic=32, apply_reorder=False, apply_vectorize=True, bank_optimize=False,
                 reorder_out_channel=False):
        w = np.ascontiguousarray(w, np.float32)
        self.K, self.C, self.ks, _ = w.shape
        self.tile_ic = tile_ic
        self.apply_reorder = apply_reorder
        self._h = _lib.orc_spf_pack(w, self.C, self.K, self.ks, tile_ic, int(apply_reorder), int(apply_vectorize),
                                    int(bank_optimize), int(reorder_out_channel))
        n = (C.c_int64 * 8)()
        _lib.orc_pack_sizes(self._h, n)
        self.nnz_counted, self.bank_oob, self.stages = int(n[5]), int(n[6]), int(n[7])

        def grab(name, cnt, dt):
            if cnt == 0:
                return np.zeros(0, dt)
            return np.ctypeslib.as_array(getattr(_lib, "orc_pack_" + name)(self._h), shape=(cnt,)).copy()

        self.offsets = grab("offsets", n[0], np.int32)
        self.stage_len = grab("stage_len", n[1], np.int32)
        self.position = grab("position", n[2], np.int32)
        self.values = grab("values", n[3], np.float32)
        self.perm = grab("perm", n[4], np.int32)

    def arrays(self):
        return (self.offsets, self.stage_len, self.position, self.values, self.perm)

    def conv(self, x, stride, pad, threads=1):
        """HostSpconv2d (keep-as-is format) or HostReorderSpconv2d (SPF) on NCHW input."""
        x = np.ascontiguousarray(x, np.float32)
        n, c, h, wd = x.shape
        assert c == self.C
        out = np.empty((n, self.K, out_extent(h, pad, self.ks, stride), out_extent(wd, pad, self.ks, stride)),
                       np.float32)
        fn = _lib.orc_host_reorder_spconv2d if self.apply_reorder else _lib.orc_host_spconv2d
        fn(self._h, x, out, n, h, wd, pad, stride, threads)
        return out

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.orc_pack_free(self._h)
            self._h = None


class G950Pack:
    """Result of orc_g950_pack: the layout the HIP kernel consumes, built on the CPU."""

    def __init__(self, w, tile_ic, oc_per_wave, order=None):
        w = np.ascontiguousarray(w, np.float32)
        self.K, self.C, self.ks, _ = w.shape
        self.tile_ic, self.oc_per_wave = tile_ic, oc_per_wave
        o = None if order is None else np.ascontiguousarray(order, np.int32)
        self._h = _lib.orc_g950_pack(w, self.C, self.K, self.ks, tile_ic, oc_per_wave,
                                     None if o is None else o.ctypes.data_as(C.c_void_p))
        n = (C.c_int64 * 5)()
        _lib.orc_g950_sizes(self._h, n)
        self.slots, self.stages = int(n[3]), int(n[4])

        def grab(name, cnt, dt):
            if cnt == 0:
                return np.zeros(0, dt)
            return np.ctypeslib.as_array(getattr(_lib, "orc_g950_" + name)(self._h), shape=(cnt,)).copy()

        self.grp_off = grab("grp_off", n[0], np.int32)
        self.grp_nnz = grab("grp_nnz", n[1], np.int32)
        self.position = grab("position", n[2], np.int32)
        self.values = grab("values", n[2], np.float32)
        self.order = grab("order", n[3], np.int32)

    def conv(self, x, stride, pad, threads=1):
        x = np.ascontiguousarray(x, np.float32)
        n, c, h, wd = x.shape
        assert c == self.C
        out = np.zeros((n, self.K, out_extent(h, pad, self.ks, stride), out_extent(wd, pad, self.ks, stride)),
                       np.float32)
        _lib.orc_g950_conv(self._h, x, out, n, h, wd, pad, stride, threads)
        return out

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:
            _lib.orc_g950_free(self._h)
            self._h = None


def fnv1a(*arrays):
    h = FNV_BASIS
    for a in arrays:
        a = np.ascontiguousarray(a)
        if a.size:
            h = int(_lib.orc_fnv1a(a.ctypes.data_as(C.c_void_p), a.nbytes, C.c_uint64(h)))
    return h
