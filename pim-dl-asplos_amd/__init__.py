"""ctypes binding of libpimdl.so (the C ABI in include/pimdl.h) for tests and benchmarks.

The product is the shared library and the C++ host layer on top of it; this module only lets
Python (numpy arrays or raw device pointers, e.g. torch tensors' data_ptr()) call the same entry
points a C++ caller would.  The directory name is not an importable identifier, so load it with
`load_package()` from the repo root's `pimdl_loader.py`, or via importlib by path.

There is no CPU fallback: if libpimdl.so is missing, or no gfx950 device is visible, calls raise.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# PIMDL_LIB_PATH: another build of the library (e.g. one compiled with other flags) instead of the in-tree one
LIB_PATH = os.environ.get("PIMDL_LIB_PATH") or os.path.join(_HERE, "libpimdl.so")
CSRC = os.path.join(_HERE, "csrc")

LUT_I8, LUT_F32 = 0, 1
BIAS_ONCE, BIAS_TIMES_CB = 0, 1
ACT_NONE, ACT_GELU_TANH = 0, 1

ERR_INVALID, ERR_UNSUPPORTED, ERR_HIP = -1, -2, -3
STATUS = {0: "PIMDL_OK", -1: "PIMDL_ERR_INVALID", -2: "PIMDL_ERR_UNSUPPORTED", -3: "PIMDL_ERR_HIP",
          -4: "PIMDL_ERR_NOMEM", -5: "PIMDL_ERR_NO_DEVICE"}

# every symbol include/pimdl.h declares
EXPORTS = ["pimdl_init", "pimdl_destroy", "pimdl_last_error", "pimdl_set_stream", "pimdl_synchronize",
           "pimdl_amm_create", "pimdl_amm_create_tuned", "pimdl_amm_destroy", "pimdl_amm_run", "pimdl_amm_run_debug",
           "pimdl_amm_profile", "pimdl_index_calculation", "pimdl_amm_index_calculation", "pimdl_lut_gather",
           "pimdl_amm_run_tiled", "pimdl_lut_gather_tiled", "pimdl_lutgen",
           "pimdl_layer_norm", "pimdl_get_device_info", "pimdl_amm_get_geometry", "pimdl_diag_bandwidth",
           "pimdl_diag_mfma_error", "pimdl_amm_group_create", "pimdl_amm_group_run", "pimdl_amm_group_destroy",
           "pimdl_attention", "pimdl_amm_group_fused_cols", "pimdl_amm_group_run_fused", "pimdl_amm_run_noalloc", "pimdl_amm_set_bias",
           "pimdl_amm_create_with", "pimdl_amm_set_tuning", "pimdl_amm_get_tuning", "pimdl_lutgen_mode",
           "pimdl_diag_mfma_error_crafted", "pimdl_amm_last_gather_kernel", "pimdl_amm_run_breakdown", "pimdl_diag_host_copy"]
NOALLOC_SCRATCH_BYTES = 8 << 20


class PimdlError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"{STATUS.get(code, code)}: {text}")
        self.code = code


class AmmDesc(ctypes.Structure):
    _fields_ = [("max_n", ctypes.c_uint32), ("input_feature_len", ctypes.c_uint32),
                ("sub_vec_len", ctypes.c_uint32), ("num_centroid", ctypes.c_uint32),
                ("output_feature_len", ctypes.c_uint32), ("lut_dtype", ctypes.c_uint32),
                ("scale_group", ctypes.c_uint32), ("bias_mode", ctypes.c_uint32),
                ("lut_bias", ctypes.c_float), ("activation", ctypes.c_uint32)]


class AmmTiming(ctypes.Structure):
    _fields_ = [("ccs_ms", ctypes.c_float), ("gather_ms", ctypes.c_float), ("total_ms", ctypes.c_float)]


class DeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("arch", ctypes.c_char * 32),
                ("compute_units", ctypes.c_uint32), ("clock_khz", ctypes.c_uint32),
                ("lds_bytes_per_cu", ctypes.c_uint32), ("hbm_bytes", ctypes.c_uint64)]


class Tiling(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in ("n_stile_size", "cb_mtile_size", "feature_stile_size",
                                               "feature_mtile_size")]


TUNING_FIELDS = ("col_block", "gather_kernel", "token_item", "cb_per_slice", "xcd_col_split", "search_kernel",
                 "search_token_tile")
GATHER_AUTO, GATHER_ROWS, GATHER_ONEHOT, GATHER_SPARSE = 0, 1, 2, 3
SEARCH_AUTO, SEARCH_SCAN, SEARCH_MFMA_F32, SEARCH_MFMA_BF16 = 0, 1, 2, 3
XCD_PLAIN = 0xFFFFFFFF


class AmmTuning(ctypes.Structure):
    """pimdl_amm_tuning: the choices a measured search may take over from the library (0 = library's choice)."""
    _fields_ = [(n, ctypes.c_uint32) for n in TUNING_FIELDS]

    def asdict(self):
        return {n: int(getattr(self, n)) for n in TUNING_FIELDS}


class AmmGeometry(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in
                ("num_codebook", "num_codebook_padded", "idx_bits", "idx_row_bytes", "col_block", "row_pitch",
                 "cb_per_slice", "lds_bytes", "tokens_per_wg", "gather_threads", "ccs_tokens_per_wg",
                 "ccs_cb_per_wg", "ccs_threads", "ccs_lds_bytes")]

    def asdict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


_lib = None


def build(verbose=False):
    """Compile libpimdl.so for gfx950 (hipcc cross-compiles without a GPU)."""
    import subprocess

    cmd = ["make", "-C", CSRC, "-j8", "-B"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode:
        print(res.stdout)
    if res.returncode:
        raise RuntimeError("building libpimdl.so failed")
    global _lib
    _lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(f"{LIB_PATH} is not built (run __graft_entry__.build() or make -C {CSRC}); "
                                "there is no CPU fallback")
    # A process may hold only one HIP runtime.  PyTorch-ROCm ships its own libamdhip64.so.7; when a
    # caller also uses torch (device tensors, streams) that copy must be the one both sides bind to,
    # so it is loaded first and libpimdl.so's NEEDED entry then resolves to it.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    vp, u32, u64 = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64
    L.pimdl_init.argtypes = [ctypes.c_int, ctypes.POINTER(vp)]
    L.pimdl_destroy.argtypes = [vp]
    L.pimdl_last_error.argtypes = [vp]
    L.pimdl_last_error.restype = ctypes.c_char_p
    L.pimdl_set_stream.argtypes = [vp, vp]
    L.pimdl_synchronize.argtypes = [vp]
    L.pimdl_amm_create.argtypes = [vp, ctypes.POINTER(AmmDesc), vp, vp, vp, vp, ctypes.POINTER(vp)]
    L.pimdl_amm_create_tuned.argtypes = [vp, ctypes.POINTER(AmmDesc), vp, vp, vp, vp, u32, ctypes.POINTER(vp)]
    L.pimdl_amm_destroy.argtypes = [vp]
    L.pimdl_amm_run.argtypes = [vp, vp, u32, vp]
    L.pimdl_amm_run_noalloc.argtypes = [vp, vp, u32, vp]
    L.pimdl_amm_run_debug.argtypes = [vp, vp, u32, vp, vp, vp]
    L.pimdl_amm_profile.argtypes = [vp, vp, u32, vp, u32, u32, ctypes.POINTER(AmmTiming)]
    L.pimdl_index_calculation.argtypes = [vp, vp, vp, u32, u32, u32, u32, vp, u32, u32]
    L.pimdl_amm_index_calculation.argtypes = [vp, vp, u32, vp, u32, u32]
    L.pimdl_amm_run_tiled.argtypes = [vp, vp, u32, vp, ctypes.POINTER(Tiling)]
    L.pimdl_lut_gather_tiled.argtypes = [vp, vp, u32, vp, ctypes.POINTER(Tiling)]
    L.pimdl_lut_gather.argtypes = [vp, vp, u32, vp]
    L.pimdl_lutgen.argtypes = [vp, vp, vp, u32, u32, u32, u32, u32, u32, vp, vp]
    L.pimdl_layer_norm.argtypes = [vp, vp, vp, vp, vp, vp, u32, u32, ctypes.c_float]
    L.pimdl_get_device_info.argtypes = [vp, ctypes.POINTER(DeviceInfo)]
    L.pimdl_amm_get_geometry.argtypes = [vp, ctypes.POINTER(AmmGeometry)]
    L.pimdl_diag_bandwidth.argtypes = [vp, u64, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
    L.pimdl_diag_mfma_error.argtypes = [vp, ctypes.c_uint32, ctypes.POINTER(ctypes.c_float)]
    L.pimdl_amm_group_create.argtypes = [vp, ctypes.POINTER(vp), u32, ctypes.POINTER(vp)]
    L.pimdl_amm_group_run.argtypes = [vp, vp, u32, ctypes.POINTER(vp)]
    L.pimdl_amm_group_destroy.argtypes = [vp]
    L.pimdl_amm_group_fused_cols.argtypes = [vp, ctypes.POINTER(u32)]
    L.pimdl_amm_group_run_fused.argtypes = [vp, vp, u32, vp]
    L.pimdl_attention.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, ctypes.c_float]
    for name in EXPORTS:
        if name != "pimdl_last_error":
            getattr(L, name).restype = ctypes.c_int
    L.pimdl_amm_last_gather_kernel.argtypes = [vp, ctypes.c_char_p, ctypes.c_size_t]
    L.pimdl_amm_set_bias.argtypes = [vp, vp]
    L.pimdl_amm_create_with.argtypes = [vp, ctypes.POINTER(AmmDesc), vp, vp, vp, vp, ctypes.POINTER(AmmTuning), ctypes.POINTER(vp)]
    L.pimdl_amm_set_tuning.argtypes = [vp, ctypes.POINTER(AmmTuning)]
    L.pimdl_amm_get_tuning.argtypes = [vp, ctypes.POINTER(AmmTuning)]
    L.pimdl_lutgen_mode.argtypes = [vp, vp, vp, u32, u32, u32, u32, u32, u32, u32, vp, vp]
    L.pimdl_diag_mfma_error_crafted.argtypes = [vp, ctypes.POINTER(ctypes.c_float)]
    _lib = L
    return L


def _ptr(a):
    """numpy array -> host pointer; int -> taken as a raw (device or host) address."""
    if a is None:
        return None
    if isinstance(a, int):
        return ctypes.c_void_p(a)
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


class Context:
    def __init__(self, device=0):
        self._h = ctypes.c_void_p()
        rc = lib().pimdl_init(device, ctypes.byref(self._h))
        if rc:
            self._h = ctypes.c_void_p()
            raise PimdlError(rc, lib().pimdl_last_error(None).decode())

    def _check(self, rc):
        if rc:
            raise PimdlError(rc, lib().pimdl_last_error(self._h).decode())

    def close(self):
        if self._h:
            lib().pimdl_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_stream(self, hip_stream):
        self._check(lib().pimdl_set_stream(self._h, ctypes.c_void_p(hip_stream) if hip_stream else None))

    def synchronize(self):
        self._check(lib().pimdl_synchronize(self._h))

    def device_info(self):
        info = DeviceInfo()
        self._check(lib().pimdl_get_device_info(self._h, ctypes.byref(info)))
        return {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
                "clock_khz": info.clock_khz, "lds_bytes_per_cu": info.lds_bytes_per_cu, "hbm_bytes": info.hbm_bytes}

    def diag_host_copy(self, nbytes=100 << 20):
        """GB/s of: pageable -> pinned and pinned -> pageable copies by the host thread pool, pinned -> device, device -> pinned."""
        r = [ctypes.c_float() for _ in range(4)]
        lib().pimdl_diag_host_copy.argtypes = [ctypes.c_void_p, ctypes.c_uint64] + [ctypes.POINTER(ctypes.c_float)] * 4
        self._check(lib().pimdl_diag_host_copy(self._h, nbytes, *[ctypes.byref(x) for x in r]))
        return dict(zip(("to_pinned_gbps", "from_pinned_gbps", "h2d_gbps", "d2h_gbps"), (x.value for x in r)))

    def diag_bandwidth(self, nbytes=1 << 30, copy=True, lds=True):
        c, l = ctypes.c_float(0), ctypes.c_float(0)
        self._check(lib().pimdl_diag_bandwidth(self._h, nbytes, ctypes.byref(c) if copy else None,
                                               ctypes.byref(l) if lds else None))
        return c.value, l.value

    def diag_mfma_error(self, trials=256):
        """Largest error of a chain of three bf16 MFMAs against the exact sum, in units of 2^-24 * sum|terms|."""
        e = ctypes.c_float(0)
        self._check(lib().pimdl_diag_mfma_error(self._h, trials, ctypes.byref(e)))
        return e.value

    def diag_mfma_error_crafted(self):
        """The same on operands built to make the accumulation lose as much as it can (see pimdl.h)."""
        e = ctypes.c_float(0)
        self._check(lib().pimdl_diag_mfma_error_crafted(self._h, ctypes.byref(e)))
        return e.value

    def index_calculation(self, x, centroids, n_stile=0, cb_mtile=0):
        """Context-level closest-centroid search: centroids are passed (and uploaded) per call."""
        x = np.ascontiguousarray(x, np.float32)
        centroids = np.ascontiguousarray(centroids, np.float32)
        n, K = x.shape
        CB, C, v = centroids.shape
        idx = np.empty(n * CB, np.uint16)
        self._check(lib().pimdl_index_calculation(self._h, _ptr(x), _ptr(centroids), n, K, v, C, _ptr(idx), n_stile,
                                                  cb_mtile))
        return idx.reshape(n, CB) if (n_stile in (0, n) and cb_mtile in (0, CB)) else idx

    def lutgen(self, centroids, weight, lut_dtype=LUT_I8, scale_group=0, ordered=False):
        """centroids f32 [CB][C][v], weight f32 [K][M] -> (lut [CB][C][M], scales or None).
        ordered: add the products of an entry in ascending order with separately rounded operations (bit for
        bit what a scalar loop gives) instead of on the matrix instruction."""
        centroids = np.ascontiguousarray(centroids, np.float32)
        weight = np.ascontiguousarray(weight, np.float32)
        CB, C, v = centroids.shape
        K, M = weight.shape
        assert K == CB * v
        if lut_dtype == LUT_F32:
            out = np.empty((CB, C, M), np.float32)
            scales = None
        else:
            out = np.empty((CB, C, M), np.int8)
            scales = np.empty(1 if scale_group == 0 else (CB + scale_group - 1) // scale_group, np.float32)
        self._check(lib().pimdl_lutgen_mode(self._h, _ptr(centroids), _ptr(weight), CB, C, v, M, lut_dtype, scale_group,
                                            1 if ordered else 0, _ptr(out), _ptr(scales)))
        return out, scales

    def layer_norm(self, x, weight, bias, residual=None, out=None, eps=1e-6):
        """norm() of the reference's layer (transformer_layer.cpp:50-90), plus the residual add when
        `residual` is given.  numpy arrays in, numpy array out; or raw addresses (ints) with n, d
        taken from `x` = (address, n, d) and `out` an address."""
        if isinstance(x, tuple):
            addr, n, d = x
            self._check(lib().pimdl_layer_norm(self._h, _ptr(addr), _ptr(weight), _ptr(bias), _ptr(residual),
                                               _ptr(out), n, d, ctypes.c_float(eps)))
            return None
        x = np.ascontiguousarray(x, np.float32)
        n, d = x.shape
        weight = np.ascontiguousarray(weight, np.float32)
        bias = np.ascontiguousarray(bias, np.float32)
        if residual is not None:
            residual = np.ascontiguousarray(residual, np.float32)
        y = np.empty_like(x)
        self._check(lib().pimdl_layer_norm(self._h, _ptr(x), _ptr(weight), _ptr(bias), _ptr(residual), _ptr(y), n, d,
                                           ctypes.c_float(eps)))
        return y

    def attention_ptr(self, q, k, v, out, batch, seq, heads, head_dim, in_stride, out_stride, scale):
        """Device addresses; out = softmax(q k^T * scale) v per (batch, head), unmasked (head_dim 64 only)."""
        self._check(lib().pimdl_attention(self._h, ctypes.c_void_p(q), ctypes.c_void_p(k), ctypes.c_void_p(v),
                                          ctypes.c_void_p(out), batch, seq, heads, head_dim, in_stride, out_stride,
                                          ctypes.c_float(scale)))

    def amm_group(self, amms):
        return AmmGroup(self, amms)

    def amm(self, centroids, lut, scales=None, bias=None, max_n=8192, lut_bias=0.0, bias_mode=BIAS_ONCE,
            scale_group=0, col_block=0, activation=ACT_NONE, tuning=None):
        """col_block: width of the gather kernel's column tile (0 = chosen by the library).
        activation: ACT_GELU_TANH applies the tanh form of GELU to the output inside the gather's epilogue.
        tuning: dict over TUNING_FIELDS (pimdl_amm_tuning), the choices a measured search takes over."""
        return Amm(self, centroids, lut, scales, bias, max_n, lut_bias, bias_mode, scale_group, col_block, activation,
                   tuning)


class AmmGroup:
    """Operators of one context that read the same input rows (separate Q/K/V projections): one search launch
    over all their codebooks, then each operator's gather.  Raises PimdlError (UNSUPPORTED / INVALID) when the
    operators cannot share a search; run them one by one then."""

    def __init__(self, ctx, amms):
        self.ctx, self.amms = ctx, list(amms)
        handles = (ctypes.c_void_p * len(self.amms))(*[a._h for a in self.amms])
        self._h = ctypes.c_void_p()
        ctx._check(lib().pimdl_amm_group_create(ctx._h, handles, len(self.amms), ctypes.byref(self._h)))
        cols = ctypes.c_uint32(0)
        ctx._check(lib().pimdl_amm_group_fused_cols(self._h, ctypes.byref(cols)))
        self.fused_cols = int(cols.value)  # > 0: run_fused writes one [n][fused_cols] buffer with one gather launch

    def close(self):
        if self._h and self.ctx._h:
            lib().pimdl_amm_group_destroy(self._h)
        self._h = ctypes.c_void_p()

    def run(self, x):
        x = np.ascontiguousarray(x, np.float32)
        n = x.shape[0]
        outs = [np.empty((n, a.M), np.float32) for a in self.amms]
        ptrs = (ctypes.c_void_p * len(outs))(*[o.ctypes.data for o in outs])
        self.ctx._check(lib().pimdl_amm_group_run(self._h, _ptr(x), n, ptrs))
        return outs

    def run_ptr(self, in_ptr, n, out_ptrs):
        """Raw addresses (device or host); asynchronous for device memory."""
        ptrs = (ctypes.c_void_p * len(out_ptrs))(*out_ptrs)
        self.ctx._check(lib().pimdl_amm_group_run(self._h, ctypes.c_void_p(in_ptr), n, ptrs))

    def run_fused(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty((x.shape[0], self.fused_cols), np.float32)
        self.ctx._check(lib().pimdl_amm_group_run_fused(self._h, _ptr(x), x.shape[0], _ptr(out)))
        return out

    def run_fused_ptr(self, in_ptr, n, out_ptr):
        self.ctx._check(lib().pimdl_amm_group_run_fused(self._h, ctypes.c_void_p(in_ptr), n, ctypes.c_void_p(out_ptr)))


class Amm:
    """One LUT-AMM operator resident in HBM."""

    def __init__(self, ctx, centroids, lut, scales, bias, max_n, lut_bias, bias_mode, scale_group, col_block=0,
                 activation=0, tuning=None):
        centroids = np.ascontiguousarray(centroids, np.float32)
        CB, C, v = centroids.shape
        lut = np.ascontiguousarray(lut)
        assert lut.dtype in (np.int8, np.float32) and lut.shape[:2] == (CB, C)
        M = lut.shape[2]
        self.ctx, self.CB, self.C, self.v, self.K, self.M = ctx, CB, C, v, CB * v, M
        self.lut_dtype = LUT_I8 if lut.dtype == np.int8 else LUT_F32
        desc = AmmDesc(max_n, CB * v, v, C, M, self.lut_dtype, scale_group, bias_mode, lut_bias, activation)
        if scales is not None:
            scales = np.ascontiguousarray(np.atleast_1d(scales), np.float32)
            want = (CB + scale_group - 1) // scale_group if (scale_group and self.lut_dtype == LUT_I8) else 1
            assert scales.size == want, f"{want} scale(s) expected, got {scales.size}"
        if bias is not None:
            bias = np.ascontiguousarray(bias, np.float32)
            assert bias.shape == (M,)
        self._h = ctypes.c_void_p()
        tune = AmmTuning(**dict(tuning or {}))
        if col_block:
            tune.col_block = col_block
        ctx._check(lib().pimdl_amm_create_with(ctx._h, ctypes.byref(desc), _ptr(centroids), _ptr(lut), _ptr(scales),
                                               _ptr(bias), ctypes.byref(tune), ctypes.byref(self._h)))

    def set_tuning(self, **fields):
        """The choices that do not touch resident data: token_item, cb_per_slice, xcd_col_split, search_kernel,
        search_token_tile (fields left out go back to the library's choice)."""
        tune = AmmTuning(**fields)
        self.ctx._check(lib().pimdl_amm_set_tuning(self._h, ctypes.byref(tune)))

    def tuning(self):
        tune = AmmTuning()
        self.ctx._check(lib().pimdl_amm_get_tuning(self._h, ctypes.byref(tune)))
        return tune.asdict()

    def close(self):
        if self._h and self.ctx._h:
            lib().pimdl_amm_destroy(self._h)
        self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def geometry(self):
        g = AmmGeometry()
        self.ctx._check(lib().pimdl_amm_get_geometry(self._h, ctypes.byref(g)))
        return g.asdict()

    def last_gather_kernel(self):
        """Name (with template arguments) of the gather kernel of the last launch, as a profile lists it."""
        buf = ctypes.create_string_buffer(96)
        self.ctx._check(lib().pimdl_amm_last_gather_kernel(self._h, buf, 96))
        return buf.value.decode()

    def run(self, x, out=None):
        """x: numpy f32 [n][K] (host) -> numpy f32 [n][M]."""
        x = np.ascontiguousarray(x, np.float32)
        n = x.shape[0]
        if out is None:
            out = np.empty((n, self.M), np.float32)
        self.ctx._check(lib().pimdl_amm_run(self._h, _ptr(x), n, _ptr(out)))
        return out

    def run_ptr(self, in_ptr, n, out_ptr):
        """Raw addresses (device or host), e.g. torch tensors' data_ptr(); asynchronous for device memory."""
        self.ctx._check(lib().pimdl_amm_run(self._h, ctypes.c_void_p(in_ptr), n, ctypes.c_void_p(out_ptr)))

    def run_noalloc_ptr(self, in_ptr, n, out_ptr):
        """Device addresses only; the call allocates nothing (fixed scratch inside the library)."""
        self.ctx._check(lib().pimdl_amm_run_noalloc(self._h, ctypes.c_void_p(in_ptr), n, ctypes.c_void_p(out_ptr)))

    def run_debug(self, x, want_acc=True):
        x = np.ascontiguousarray(x, np.float32)
        n = x.shape[0]
        out = np.empty((n, self.M), np.float32)
        idx = np.empty((n, self.CB), np.uint16)
        acc = np.empty((n, self.M), np.int32) if (want_acc and self.lut_dtype == LUT_I8) else None
        self.ctx._check(lib().pimdl_amm_run_debug(self._h, _ptr(x), n, _ptr(out), _ptr(idx), _ptr(acc)))
        return out, idx, acc

    def profile(self, in_ptr, n, out_ptr, warmup=3, iters=20):
        t = AmmTiming()
        self.ctx._check(lib().pimdl_amm_profile(self._h, ctypes.c_void_p(in_ptr), n, ctypes.c_void_p(out_ptr), warmup,
                                                iters, ctypes.byref(t)))
        return {"ccs_ms": t.ccs_ms, "gather_ms": t.gather_ms, "total_ms": t.total_ms}

    def index_calculation(self, x, n_stile=None, cb_mtile=None):
        x = np.ascontiguousarray(x, np.float32)
        n = x.shape[0]
        n_stile = n if n_stile is None else n_stile
        cb_mtile = self.CB if cb_mtile is None else cb_mtile
        idx = np.empty(n * self.CB, np.uint16)
        self.ctx._check(lib().pimdl_amm_index_calculation(self._h, _ptr(x), n, _ptr(idx), n_stile, cb_mtile))
        return idx.reshape(n, self.CB) if (n_stile == n and cb_mtile == self.CB) else idx

    def run_tiled(self, x, n_stile=0, cb_mtile=0, f_stile=0, f_mtile=0):
        """Output as a flat array in the reference's DPU order (test_amm.cpp:193-202)."""
        x = np.ascontiguousarray(x, np.float32)
        n = x.shape[0]
        out = np.empty(n * self.M, np.float32)
        til = Tiling(n_stile, cb_mtile, f_stile, f_mtile)
        self.ctx._check(lib().pimdl_amm_run_tiled(self._h, _ptr(x), n, _ptr(out), ctypes.byref(til)))
        return out

    def run_tiled_ptr(self, in_ptr, n, out_ptr, n_stile=0, cb_mtile=0, f_stile=0, f_mtile=0):
        """Raw addresses (device or host); output in the reference's DPU order."""
        til = Tiling(n_stile, cb_mtile, f_stile, f_mtile)
        self.ctx._check(lib().pimdl_amm_run_tiled(self._h, ctypes.c_void_p(in_ptr), n, ctypes.c_void_p(out_ptr),
                                                  ctypes.byref(til)))

    def lut_gather_tiled(self, idx_flat, n, n_stile=0, cb_mtile=0, f_stile=0, f_mtile=0):
        idx_flat = np.ascontiguousarray(idx_flat, np.uint16).reshape(-1)
        out = np.empty(n * self.M, np.float32)
        til = Tiling(n_stile, cb_mtile, f_stile, f_mtile)
        self.ctx._check(lib().pimdl_lut_gather_tiled(self._h, _ptr(idx_flat), n, _ptr(out), ctypes.byref(til)))
        return out

    def set_bias(self, bias):
        """Replace the operator's bias [M] (None: zeros)."""
        if bias is not None:
            bias = np.ascontiguousarray(bias, np.float32)
            assert bias.shape == (self.M,)
        self.ctx._check(lib().pimdl_amm_set_bias(self._h, _ptr(bias)))

    def lut_gather(self, idx):
        idx = np.ascontiguousarray(idx, np.uint16)
        n = idx.shape[0]
        out = np.empty((n, self.M), np.float32)
        self.ctx._check(lib().pimdl_lut_gather(self._h, _ptr(idx), n, _ptr(out)))
        return out
