"""hpt_amd — the MI355X (gfx950) `Hip` backend of Hpt's reduction / softmax /
layernorm path: a C-ABI library of hand-written HIP kernels (hpt_amd/csrc,
include/hpt_hip.h) and this thin host-side mirror of Hpt's tensor API over it.
"""
from ._ffi import (DeviceError, DTypeError, HptError, KernelError, MemoryError_, ParamError,
                   ShapeError, lib)
from .tensor import (ALL, ANY, BIN_ADD, BIN_DIV, BIN_MUL, BIN_SUB, DTYPES, LOGSUMEXP, MAX, MEAN, MIN, NANPROD, NANSUM, PROD, REDUCEL1,
                     REDUCEL2, REDUCEL3, SUM, SUM_SQUARE, DType, Tensor, bf16, bf16_bits_to_f32,
                     bool_, device_count, f16, f32, f32_to_bf16_bits, f64, i8, i16, i32, i64,
                     binary_plan, contiguous_plan, normalize_plan, reduce_plan, synchronize, u8, u16, u32, u64)

__all__ = [n for n in dir() if not n.startswith("_")]
