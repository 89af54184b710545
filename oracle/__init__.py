"""CPU oracle for the LUT-AMM path -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package.
The shipped library never does; it has no CPU fallback.

Two layers:
  * `lib` functions: ctypes bindings of oracle/libpimdl_oracle.so (C restatement of the
    reference's host code, see pimdl_oracle.c for the file:line each function follows);
  * `np_*` functions: independent numpy statements of the same mathematics, used by the
    tests to pin the C restatement (a second derivation, not a re-typing of the C loops).
  * `ref_index_calculation`: the reference's own index_calc_host.cpp, compiled from source
    into oracle/_ref/ (present only where that library was built).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpimdl_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_index_calc.so")

_u32 = ctypes.c_uint32
_u64 = ctypes.c_uint64
_f32 = ctypes.c_float
_int = ctypes.c_int
_ptr = ctypes.c_void_p


def build(force=False):
    """Compile the C restatement (and oracle/_ref when the reference tree is present)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    sig = {
        "oracle_index_calculation": [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32, _u32, _u32, _int],
        "oracle_distances": [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32],
        "oracle_gather_i8": [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _int],
        "oracle_dequant": [_ptr, _ptr, _ptr, _u32, _u32, _u32, _f32, _f32, _int, _int],
        "oracle_amm_cpu": [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32,
                           _f32, _f32, _int],
        "oracle_gather_f32": [_ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _int],
        "oracle_gather_i8_grouped": [_ptr, _ptr, _ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _u32, _int],
        "oracle_lutgen_f32": [_ptr, _ptr, _ptr, _u32, _u32, _u32, _u32, _int],
        "oracle_lut_quant": [_ptr, _ptr, _ptr, _u64, _u64, _u64],
        "oracle_reorder_pim_lut": [_ptr, _ptr, _u32, _u32, _u32, _u32],
        "oracle_prepare_input_index": [_ptr, _u32, _u32, _u32, _u32, _u32, _int, _u32, _u32, _u32],
        "oracle_layer_norm": [_ptr, _ptr, _ptr, _ptr, _u32, _u32],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = None
    lib.oracle_output_offset.argtypes = [_u32] * 6
    lib.oracle_output_offset.restype = _u64
    lib.oracle_max_threads.argtypes = []
    lib.oracle_max_threads.restype = _int
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _p(a):
    return a.ctypes.data_as(_ptr)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def max_threads():
    return int(lib().oracle_max_threads())


# --------------------------------------------------------------------------- C restatement


def index_calculation(x, cent, v, n_stile=None, cb_mtile=None, threads=1):
    """x [N][K] f32, cent [CB][C][v] f32 -> u16 indices (flat, in the reference's tile order;
    row-major [N][CB] for the default identity tiling)."""
    x = _c(x, np.float32)
    cent = _c(cent, np.float32)
    N, K = x.shape
    CB, C, vv = cent.shape
    assert vv == v and CB * v == K
    n_stile = N if n_stile is None else n_stile
    cb_mtile = CB if cb_mtile is None else cb_mtile
    out = np.zeros(N * CB, dtype=np.uint16)
    lib().oracle_index_calculation(_p(x), _p(cent), _p(out), N, K, v, CB, C, n_stile, cb_mtile, threads)
    if n_stile == N and cb_mtile == CB:
        return out.reshape(N, CB)
    return out


def distances(x, cent, v):
    x = _c(x, np.float32)
    cent = _c(cent, np.float32)
    N, K = x.shape
    CB, C, _ = cent.shape
    out = np.zeros((N, CB, C), dtype=np.float32)
    lib().oracle_distances(_p(x), _p(cent), _p(out), N, K, v, CB, C)
    return out


def gather_i8(idx, lut, threads=1):
    """idx [N][CB] u16, lut [CB][C][M] i8 -> acc [N][M] i32."""
    idx = _c(idx, np.uint16)
    lut = _c(lut, np.int8)
    N, CB = idx.shape
    _, C, M = lut.shape
    acc = np.empty((N, M), dtype=np.int32)
    lib().oracle_gather_i8(_p(idx), _p(lut), _p(acc), N, CB, C, M, threads)
    return acc


def dequant(acc, bias_tensor, CB, scale, lut_bias=0.0, bias_mode=0, threads=1):
    acc = _c(acc, np.int32)
    bias_tensor = _c(bias_tensor, np.float32)
    N, M = acc.shape
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_dequant(_p(acc), _p(bias_tensor), _p(out), N, M, CB, scale, lut_bias, bias_mode, threads)
    return out


def amm_cpu(x, cent, lut, bias_tensor, v, scale, lut_bias=0.0, threads=1, scratch=None):
    """Whole AMM as the reference's amm_cpu.  Returns (out, idx, acc)."""
    x = _c(x, np.float32)
    cent = _c(cent, np.float32)
    lut = _c(lut, np.int8)
    bias_tensor = _c(bias_tensor, np.float32)
    N, K = x.shape
    CB, C, _ = cent.shape
    M = lut.shape[-1]
    if scratch is None:
        scratch = (np.empty((N, CB), np.uint16), np.empty((N, M), np.int32), np.empty((N, M), np.float32))
    idx, acc, out = scratch
    lib().oracle_amm_cpu(_p(x), _p(cent), _p(lut), _p(bias_tensor), _p(out), _p(idx), _p(acc),
                         N, K, v, C, M, scale, lut_bias, threads)
    return out, idx, acc


def gather_f32(idx, lut, bias_tensor, threads=1):
    idx = _c(idx, np.uint16)
    lut = _c(lut, np.float32)
    bias_tensor = _c(bias_tensor, np.float32)
    N, CB = idx.shape
    _, C, M = lut.shape
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_gather_f32(_p(idx), _p(lut), _p(bias_tensor), _p(out), N, CB, C, M, threads)
    return out


def gather_i8_grouped(idx, lut, scales, bias_tensor, group, threads=1):
    idx = _c(idx, np.uint16)
    lut = _c(lut, np.int8)
    scales = _c(scales, np.float32)
    bias_tensor = _c(bias_tensor, np.float32)
    N, CB = idx.shape
    _, C, M = lut.shape
    assert scales.size == (CB + group - 1) // group
    out = np.empty((N, M), dtype=np.float32)
    lib().oracle_gather_i8_grouped(_p(idx), _p(lut), _p(scales), _p(bias_tensor), _p(out), N, CB, C, M,
                                   group, threads)
    return out


def lutgen_f32(cent, W, threads=1):
    """cent [CB][C][v], W [K][M] -> lut [CB][C][M] f32."""
    cent = _c(cent, np.float32)
    W = _c(W, np.float32)
    CB, C, v = cent.shape
    K, M = W.shape
    assert K == CB * v
    lut = np.empty((CB, C, M), dtype=np.float32)
    lib().oracle_lutgen_f32(_p(cent), _p(W), _p(lut), CB, C, v, M, threads)
    return lut


def lut_quant(lut_f32, group_codebooks=0):
    """Per-tensor (group_codebooks=0, the reference) or per-codebook-group int8 quantisation.
    Returns (q int8 same shape, scales f32[ngroups])."""
    lut_f32 = _c(lut_f32, np.float32)
    CB, C, M = lut_f32.shape
    rows = CB * C
    group_rows = group_codebooks * C
    ng = 1 if group_rows == 0 else (rows + group_rows - 1) // group_rows
    q = np.empty(lut_f32.shape, dtype=np.int8)
    scales = np.empty(ng, dtype=np.float32)
    lib().oracle_lut_quant(_p(lut_f32), _p(q), _p(scales), rows, M, group_rows)
    return q, scales


def reorder_pim_lut(lut, ftile):
    lut = _c(lut, np.int8)
    CB, C, M = lut.shape
    out = np.empty(lut.size, dtype=np.int8)
    lib().oracle_reorder_pim_lut(_p(lut), _p(out), CB, C, M, ftile)
    return out


def output_offset(n, f, n_stile, f_stile, f_mtile, lut_parallelism):
    return int(lib().oracle_output_offset(n, f, n_stile, f_stile, f_mtile, lut_parallelism))


def prepare_input_index(idx_flat, N, CB, C, n_stile, cb_mtile, load_type, f_stile, f_load_tile, cb_load_tile):
    idx_flat = np.array(idx_flat, dtype=np.uint16, copy=True).reshape(-1)
    lib().oracle_prepare_input_index(_p(idx_flat), N, CB, C, n_stile, cb_mtile, load_type, f_stile,
                                     f_load_tile, cb_load_tile)
    return idx_flat


def layer_norm(x, gamma, beta):
    x = _c(x, np.float32)
    gamma = _c(gamma, np.float32)
    beta = _c(beta, np.float32)
    N, D = x.shape
    y = np.empty_like(x)
    lib().oracle_layer_norm(_p(x), _p(gamma), _p(beta), _p(y), N, D)
    return y


# --------------------------------------------------------------------------- reference build


def have_ref():
    return os.path.exists(_REF_PATH)


_ref = None


def ref_index_calculation(x, cent, v, n_stile=None, cb_mtile=None, threads=1):
    """The reference's own index_calculation (index_calc_host.cpp:8-53), built from source."""
    global _ref
    if _ref is None:
        _ref = ctypes.CDLL(_REF_PATH)
        _ref.ref_index_calculation.argtypes = [_ptr, _ptr, _ptr] + [_u32] * 8
        _ref.ref_index_calculation.restype = None
    x = _c(x, np.float32)
    cent = _c(cent, np.float32)
    N, K = x.shape
    CB, C, _ = cent.shape
    n_stile = N if n_stile is None else n_stile
    cb_mtile = CB if cb_mtile is None else cb_mtile
    out = np.zeros(N * CB, dtype=np.uint16)
    _ref.ref_index_calculation(_p(x), _p(cent), _p(out), N, K, v, CB, C, threads, n_stile, cb_mtile)
    if n_stile == N and cb_mtile == CB:
        return out.reshape(N, CB)
    return out


# --------------------------------------------------------------------------- numpy statements


def np_scan_argmin(dist):
    """Sequential hysteresis scan over the last axis (index_calc_host.cpp:30-39), vectorised over
    the leading axes.  The fp32 difference is compared as a double against 1e-6."""
    dist = np.asarray(dist, dtype=np.float32)
    best = dist[..., 0].copy()
    bi = np.zeros(dist.shape[:-1], dtype=np.uint16)
    for c in range(1, dist.shape[-1]):
        d = dist[..., c]
        take = (best - d).astype(np.float64) > 1e-6
        best = np.where(take, d, best)
        bi = np.where(take, np.uint16(c), bi)
    return bi


def np_distances(x, cent):
    """fp32 squared distances accumulated over t ascending with separately rounded sub, mul, add."""
    x = np.asarray(x, dtype=np.float32)
    cent = np.asarray(cent, dtype=np.float32)
    N, K = x.shape
    CB, C, v = cent.shape
    xs = x.reshape(N, CB, 1, v)
    d = np.zeros((N, CB, C), dtype=np.float32)
    for t in range(v):
        diff = (xs[..., t] - cent[None, :, :, t]).astype(np.float32)
        sq = (diff * diff).astype(np.float32)
        d = (d + sq).astype(np.float32)
    return d


def np_index_calculation(x, cent):
    return np_scan_argmin(np_distances(x, cent))


def np_gather_onehot(idx, lut):
    """acc = one_hot(idx)[N, CB*C] @ lut[CB*C, M] in integer arithmetic (a library matmul)."""
    idx = np.asarray(idx)
    lut = np.asarray(lut)
    N, CB = idx.shape
    _, C, M = lut.shape
    onehot = np.zeros((N, CB * C), dtype=np.int32)
    onehot[np.arange(N)[:, None], np.arange(CB)[None, :] * C + idx.astype(np.int64)] = 1
    return onehot @ lut.reshape(CB * C, M).astype(np.int32)


def np_lut_quant(lut_f32):
    """pim_weight_converter.py:21-35 in numpy (np.round is round-half-even, like torch.round)."""
    lut_f32 = np.asarray(lut_f32, dtype=np.float32)
    max_abs = np.maximum(np.abs(lut_f32.min()), np.abs(lut_f32.max())).astype(np.float32)
    scale = np.float32(max_abs / np.float32(127.0))
    q = np.round(np.clip((lut_f32 / scale).astype(np.float32), -128, 127)).astype(np.int8)
    return q, scale
