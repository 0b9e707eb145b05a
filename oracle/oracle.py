"""ctypes loader of the CPU oracle (oracle/libhpt_oracle.so) — TEST INFRASTRUCTURE.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
import this module; the product (hpt_amd/) never does.

All functions take and return numpy arrays. Views (permuted / sliced / stepped
numpy arrays) are passed with their element strides, so the oracle walks the
same memory layout the device kernels are given.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "libhpt_oracle.so"

BOOL, I8, I16, I32, I64, U8, U16, U32, U64, F16, BF16, F32, F64 = range(13)
SUM, PROD, MAX, MIN, MEAN, NANSUM, NANPROD, REDUCEL1, REDUCEL2, REDUCEL3, SUM_SQUARE, LOGSUMEXP, ALL, ANY = range(14)
ACC_NATIVE, ACC_F32, ACC_F64, ACC_EXACT = 0, 1, 2, 3

_NP2DT = {np.dtype(np.bool_): BOOL, np.dtype(np.int8): I8, np.dtype(np.int16): I16,
          np.dtype(np.int32): I32, np.dtype(np.int64): I64, np.dtype(np.uint8): U8,
          np.dtype(np.uint16): U16, np.dtype(np.uint32): U32, np.dtype(np.uint64): U64,
          np.dtype(np.float16): F16, np.dtype(np.float32): F32, np.dtype(np.float64): F64}
_DT2NP = {v: k for k, v in _NP2DT.items()}
_DT2NP[BF16] = np.dtype(np.uint16)


class View(C.Structure):
    _fields_ = [("data", C.c_void_p), ("shape", C.POINTER(C.c_int64)),
                ("strides", C.POINTER(C.c_int64)), ("ndim", C.c_int32), ("dtype", C.c_int32)]


def build(force: bool = False) -> Path:
    src = [HERE / "hpt_oracle.c", HERE / "hpt_oracle.h"]
    if force or not LIB_PATH.exists() or LIB_PATH.stat().st_mtime < max(s.stat().st_mtime for s in src):
        subprocess.run(["make", "-C", str(HERE), "-B", "libhpt_oracle.so"], check=True,
                       capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        l = C.CDLL(str(LIB_PATH))
        p64 = C.POINTER(C.c_int64)
        l.orc_process_axes.argtypes = [p64, C.c_int, C.c_int, p64, C.c_char_p, C.c_size_t]
        l.orc_reduce_shape.argtypes = [p64, C.c_int, p64, C.c_int, C.c_int, p64, C.POINTER(C.c_int),
                                       C.c_char_p, C.c_size_t]
        l.orc_shape_to_strides.argtypes = [p64, C.c_int, p64]
        l.orc_is_contiguous.argtypes = [p64, p64, C.c_int]
        l.orc_coalesce_dims.argtypes = [p64, p64, C.c_int, C.POINTER(C.c_int)]
        l.orc_mt_intervals.argtypes = [C.c_int64, C.c_int64, p64]
        l.orc_mt_intervals_simd.argtypes = [C.c_int64, C.c_int64, C.c_int64, p64]
        l.orc_slice_process.argtypes = [p64, p64, C.c_int, p64, C.c_int, C.c_int64, p64, p64,
                                        C.POINTER(C.c_int), p64]
        l.orc_reduce_out_dtype.argtypes = [C.c_int, C.c_int]
        l.orc_reduce.argtypes = [C.c_int, C.POINTER(View), p64, C.c_int, C.c_void_p, C.c_int, C.c_int]
        l.orc_argreduce.argtypes = [C.c_int, C.POINTER(View), C.c_int64, p64]
        l.orc_softmax.argtypes = [C.c_int, C.POINTER(View), C.c_int64, C.c_void_p, C.c_int, C.c_int]
        l.orc_layernorm.argtypes = [C.POINTER(View), C.c_int, C.c_void_p, C.c_void_p, C.c_double,
                                    C.c_void_p, C.c_int]
        pf = C.POINTER(C.c_float)
        l.orc_mt_layernorm_f32.argtypes = [pf, C.c_int64, C.c_int64, pf, pf, C.c_float, pf, C.c_int]
        l.orc_mt_softmax_f32.argtypes = [pf, C.c_int64, C.c_int64, pf, C.c_int, C.c_int]
        l.orc_mt_reduce_rows_f32.argtypes = [pf, C.c_int64, C.c_int64, pf, C.c_int, C.c_int]
        l.orc_vexpf.argtypes = [C.c_float]
        l.orc_vexpf.restype = C.c_float
        l.orc_physical_cores.restype = C.c_int
        for n in ("orc_f16_to_f32", "orc_bf16_to_f32"):
            getattr(l, n).argtypes = [C.c_uint16]
            getattr(l, n).restype = C.c_float
        for n in ("orc_f32_to_f16", "orc_f32_to_bf16"):
            getattr(l, n).argtypes = [C.c_float]
            getattr(l, n).restype = C.c_uint16
        _lib = l
    return _lib


def _i64(vals):
    vals = [int(v) for v in vals]
    return (C.c_int64 * max(1, len(vals)))(*vals)


def _view(a: np.ndarray, dtype=None):
    """orc_view of a numpy array (any strides). Returns (view, keepalive)."""
    dt = _NP2DT[a.dtype] if dtype is None else dtype
    sh = _i64(a.shape)
    st = _i64([s // a.itemsize for s in a.strides])
    v = View(C.c_void_p(a.ctypes.data), C.cast(sh, C.POINTER(C.c_int64)),
             C.cast(st, C.POINTER(C.c_int64)), a.ndim, dt)
    return v, (sh, st, a)


# ---- shape logic ---------------------------------------------------------------

def process_axes(axes, ndim):
    axes = [axes] if isinstance(axes, int) else list(axes)
    out = _i64([0] * len(axes))
    err = C.create_string_buffer(256)
    rc = lib().orc_process_axes(_i64(axes), len(axes), ndim, out, err, 256)
    if rc:
        raise ValueError(err.value.decode())
    return [out[i] for i in range(len(axes))]


def reduce_shape(shape, axes, keep_dims):
    axes = [axes] if isinstance(axes, int) else list(axes)
    out = _i64([0] * max(1, len(shape)))
    n = C.c_int()
    err = C.create_string_buffer(256)
    rc = lib().orc_reduce_shape(_i64(shape), len(shape), _i64(axes), len(axes), int(keep_dims), out,
                                C.byref(n), err, 256)
    if rc:
        raise ValueError(err.value.decode())
    return [out[i] for i in range(n.value)]


def is_contiguous(shape, strides):
    return bool(lib().orc_is_contiguous(_i64(shape), _i64(strides), len(shape)))


def coalesce_dims(shape, strides):
    g = (C.c_int * max(1, len(shape)))()
    n = lib().orc_coalesce_dims(_i64(shape), _i64(strides), len(shape), g)
    groups = [[] for _ in range(n)]
    for d in range(len(shape)):
        groups[g[d]].append(d)
    return groups


def mt_intervals(size, nthreads):
    out = _i64([0] * (2 * nthreads))
    lib().orc_mt_intervals(size, nthreads, out)
    return [(out[2 * i], out[2 * i + 1]) for i in range(nthreads)]


def mt_intervals_simd(size, nthreads, vec):
    out = _i64([0] * (2 * nthreads))
    lib().orc_mt_intervals_simd(size, nthreads, vec, out)
    return [(out[2 * i], out[2 * i + 1]) for i in range(nthreads)]


def slice_process(shape, strides, index, alpha=1):
    flat = [x for t in index for x in t]
    osh, ost = _i64([0] * len(shape)), _i64([0] * len(shape))
    n, off = C.c_int(), C.c_int64()
    rc = lib().orc_slice_process(_i64(shape), _i64(strides), len(shape), _i64(flat), len(index), alpha,
                                 osh, ost, C.byref(n), C.byref(off))
    if rc:
        raise ValueError("index length is greater than the shape length")
    return [osh[i] for i in range(n.value)], [ost[i] for i in range(n.value)], off.value


def reduce_out_dtype(op, dt):
    return lib().orc_reduce_out_dtype(op, dt)


# ---- the hot path -----------------------------------------------------------------

def reduce(op, a: np.ndarray, axes, keep_dims=False, acc=ACC_NATIVE, lanes=1, dtype=None):
    """Reduce `a` (any strides) over `axes`. dtype=BF16 reads uint16 bit patterns as bf16."""
    axes = [axes] if isinstance(axes, (int, np.integer)) else list(axes)
    dt = _NP2DT[a.dtype] if dtype is None else dtype
    odt = reduce_out_dtype(op, dt)
    flat_shape = reduce_shape(a.shape, axes, False)
    out = np.zeros(flat_shape, _DT2NP[odt])
    v, keep = _view(a, dt)
    rc = lib().orc_reduce(op, C.byref(v), _i64(axes), len(axes), C.c_void_p(out.ctypes.data), acc, lanes)
    if rc:
        raise ValueError(f"orc_reduce failed ({rc})")
    return out.reshape(reduce_shape(a.shape, axes, keep_dims))


def argreduce(is_max, a: np.ndarray, axis, keep_dims=False, dtype=None):
    dt = _NP2DT[a.dtype] if dtype is None else dtype
    out = np.zeros(reduce_shape(a.shape, [axis], False), np.int64)
    v, keep = _view(a, dt)
    rc = lib().orc_argreduce(int(is_max), C.byref(v), axis, out.ctypes.data_as(C.POINTER(C.c_int64)))
    if rc:
        raise ValueError(f"orc_argreduce failed ({rc})")
    return out.reshape(reduce_shape(a.shape, [axis], keep_dims))


def softmax(a: np.ndarray, axis, log=False, acc=ACC_NATIVE, lanes=1, dtype=None):
    dt = _NP2DT[a.dtype] if dtype is None else dtype
    out = np.zeros(a.shape, _DT2NP[dt])
    v, keep = _view(a, dt)
    rc = lib().orc_softmax(int(log), C.byref(v), axis, C.c_void_p(out.ctypes.data), acc, lanes)
    if rc:
        raise ValueError(f"orc_softmax failed ({rc})")
    return out


def layernorm(a: np.ndarray, n_norm_dims, gamma=None, beta=None, eps=1e-5, acc=ACC_NATIVE, dtype=None):
    dt = _NP2DT[a.dtype] if dtype is None else dtype
    out = np.zeros(a.shape, _DT2NP[dt])
    v, keep = _view(a, dt)
    g = np.ascontiguousarray(gamma) if gamma is not None else None
    b = np.ascontiguousarray(beta) if beta is not None else None
    rc = lib().orc_layernorm(C.byref(v), n_norm_dims,
                             C.c_void_p(g.ctypes.data) if g is not None else None,
                             C.c_void_p(b.ctypes.data) if b is not None else None,
                             float(eps), C.c_void_p(out.ctypes.data), acc)
    if rc:
        raise ValueError(f"orc_layernorm failed ({rc})")
    return out


# ---- the timed restatement --------------------------------------------------------------

def _pf(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def mt_layernorm_f32(x, gamma, beta, eps, nthreads, out=None):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x) if out is None else out
    lib().orc_mt_layernorm_f32(_pf(x), x.shape[0], x.shape[1], _pf(gamma) if gamma is not None else None,
                               _pf(beta) if beta is not None else None, eps, _pf(out), nthreads)
    return out


def mt_softmax_f32(x, log, nthreads, out=None):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty_like(x) if out is None else out
    lib().orc_mt_softmax_f32(_pf(x), x.shape[0], x.shape[1], _pf(out), int(log), nthreads)
    return out


def mt_reduce_rows_f32(x, op, nthreads, out=None):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape[0], np.float32) if out is None else out
    lib().orc_mt_reduce_rows_f32(_pf(x), x.shape[0], x.shape[1], _pf(out), op, nthreads)
    return out


def physical_cores() -> int:
    return lib().orc_physical_cores()


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(a: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round-to-nearest-even with NaN quieting (vectorised)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x0040).astype(np.uint16)
    return r
