"""ctypes binding of libhpt_hip.so (the C ABI declared in include/hpt_hip.h).

The library is the product: there is no fallback. If it has not been built,
loading fails with an instruction to build it.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libhpt_hip.so"

# hpt_status
OK, ERR_PARAM, ERR_SHAPE, ERR_DTYPE, ERR_MEMORY, ERR_KERNEL, ERR_DEVICE = range(7)


class HptError(RuntimeError):
    """Base of the errors raised for a non-zero hpt_status (TensorError of the reference)."""

    def __init__(self, code: int, msg: str):
        super().__init__(msg)
        self.code = code


class ParamError(HptError):
    pass


class ShapeError(HptError):
    pass


class DTypeError(HptError):
    pass


class MemoryError_(HptError):
    pass


class KernelError(HptError):
    pass


class DeviceError(HptError):
    pass


_ERRORS = {ERR_PARAM: ParamError, ERR_SHAPE: ShapeError, ERR_DTYPE: DTypeError,
           ERR_MEMORY: MemoryError_, ERR_KERNEL: KernelError, ERR_DEVICE: DeviceError}


class View(C.Structure):
    """hpt_view"""
    _fields_ = [("data", C.c_void_p), ("shape", C.POINTER(C.c_int64)),
                ("strides", C.POINTER(C.c_int64)), ("ndim", C.c_int32), ("dtype", C.c_int32)]


# name -> (restype, argtypes); every symbol include/hpt_hip.h declares
SIGNATURES = {
    "hpt_hip_last_error": (C.c_char_p, []),
    "hpt_hip_dtype_size": (C.c_size_t, [C.c_int32]),
    "hpt_hip_device_count": (C.c_int32, [C.POINTER(C.c_int32)]),
    "hpt_hip_alloc": (C.c_int32, [C.c_int32, C.c_size_t, C.c_size_t, C.c_int32, C.POINTER(C.c_void_p)]),
    "hpt_hip_free": (C.c_int32, [C.c_int32, C.c_void_p, C.c_size_t, C.c_size_t]),
    "hpt_hip_forget": (C.c_int32, [C.c_int32, C.c_void_p]),
    "hpt_hip_cache_resize": (C.c_int32, [C.c_int32, C.c_size_t]),
    "hpt_hip_cache_clear": (C.c_int32, [C.c_int32]),
    "hpt_hip_alloc_stats": (C.c_int32, [C.c_int32, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "hpt_hip_memcpy_h2d_sync": (C.c_int32, [C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t]),
    "hpt_hip_memcpy_d2h_sync": (C.c_int32, [C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t]),
    "hpt_hip_memcpy_d2d_sync": (C.c_int32, [C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t]),
    "hpt_hip_stream_synchronize": (C.c_int32, [C.c_int32, C.c_void_p]),
    "hpt_hip_device_synchronize": (C.c_int32, [C.c_int32]),
    "hpt_hip_process_axes": (C.c_int32, [C.POINTER(C.c_int64), C.c_int32, C.c_int32, C.POINTER(C.c_int64)]),
    "hpt_hip_reduce_shape": (C.c_int32, [C.POINTER(C.c_int64), C.c_int32, C.POINTER(C.c_int64), C.c_int32,
                                         C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int32)]),
    "hpt_hip_reduce_out_dtype": (C.c_int32, [C.c_int32, C.c_int32, C.POINTER(C.c_int32)]),
    "hpt_hip_reduce_plan": (C.c_int32, [C.c_int32, C.POINTER(View), C.POINTER(C.c_int64), C.c_int32,
                                        C.c_char_p, C.c_size_t]),
    "hpt_hip_normalize_plan": (C.c_int32, [C.POINTER(View), C.c_int64, C.c_int32, C.c_char_p, C.c_size_t]),
    "hpt_hip_reduce": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(View), C.POINTER(C.c_int64),
                                   C.c_int32, C.c_int32, C.POINTER(View)]),
    "hpt_hip_reduce_static": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(View), C.POINTER(C.c_int64),
                                          C.c_int32, C.c_int32, C.POINTER(View)]),
    "hpt_hip_argreduce": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(View), C.c_int64,
                                      C.POINTER(View)]),
    "hpt_hip_softmax": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(View), C.c_int64,
                                    C.POINTER(View)]),
    "hpt_hip_layernorm": (C.c_int32, [C.c_int32, C.c_void_p, C.POINTER(View), C.c_int32, C.POINTER(View),
                                      C.POINTER(View), C.c_double, C.POINTER(View)]),
    "hpt_hip_softmax_causal": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(View), C.c_double, C.c_int64,
                                           C.POINTER(View)]),
    "hpt_hip_add_layernorm": (C.c_int32, [C.c_int32, C.c_void_p, C.POINTER(View), C.POINTER(View), C.c_int32,
                                          C.POINTER(View), C.POINTER(View), C.c_double, C.POINTER(View)]),
    "hpt_hip_contiguous": (C.c_int32, [C.c_int32, C.c_void_p, C.POINTER(View), C.POINTER(View)]),
    "hpt_hip_contiguous_plan": (C.c_int32, [C.POINTER(View), C.POINTER(View), C.c_char_p, C.c_size_t]),
    "hpt_hip_binary_plan": (C.c_int32, [C.POINTER(View), C.POINTER(View), C.POINTER(View), C.c_char_p, C.c_size_t]),
    "hpt_hip_cast": (C.c_int32, [C.c_int32, C.c_void_p, C.POINTER(View), C.POINTER(View)]),
    "hpt_hip_fill": (C.c_int32, [C.c_int32, C.c_void_p, C.POINTER(View), C.c_void_p]),
    "hpt_hip_binary": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(View), C.POINTER(View),
                                   C.POINTER(View)]),
}

_lib = None


def lib() -> C.CDLL:
    """Load libhpt_hip.so once; fail loudly when it is not built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m hpt_amd.build` "
                "(hpt_amd has no fallback path)")
        l = C.CDLL(str(LIB_PATH))
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(status: int) -> None:
    if status != OK:
        msg = lib().hpt_hip_last_error().decode("utf-8", "replace")
        raise _ERRORS.get(status, HptError)(status, msg)


def i64_array(values):
    values = list(values)
    return (C.c_int64 * max(1, len(values)))(*values)


def make_view(ptr: int, shape, strides, dtype: int):
    """Build an hpt_view; returns (view, keepalive) — keep both alive during the call."""
    sh = i64_array(shape)
    st = i64_array(strides)
    v = View(C.c_void_p(ptr), C.cast(sh, C.POINTER(C.c_int64)), C.cast(st, C.POINTER(C.c_int64)),
             len(list(shape)), int(dtype))
    return v, (sh, st)
