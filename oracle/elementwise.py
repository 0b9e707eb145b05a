"""CPU restatement of the steps either side of the path — TEST INFRASTRUCTURE.

Only tests/ may import this module. numpy restatements (byte / element arithmetic only):

contiguous(a)      strided_copy (hpt-cudakernels/src/strided_copy.cu:6-14): dst[i] = src at the
                   offset of the i-th index tuple of the view in row-major order
                   (hpt/src/backends/cuda/tensor_internal/normal_out_unary.rs:286-310).
                   Pinned by: brute-force enumeration of index tuples on small views
                   (tests/test_oracle_elementwise.py).
full(v, shape, dt) set_val (hpt-cudakernels/src/set_val.cu:4-12). Trivial.
binary(op, a, b)   NormalBinOps add_/sub_/mul_/div_ on one dtype (hpt-traits/src/ops/binary.rs:34-152):
                   integers wrap (hpt-types/src/scalars/impls.rs:31-48), bool add = OR and mul = AND,
                   f16 / bf16 widen to f32, operate, round to nearest even once (the `half` crate,
                   hpt-types/src/scalars/_f16.rs:10-70), f32 / f64 IEEE. Broadcasting by numpy's rule
                   (predict_broadcast_shape, hpt-common/src/shape/shape_utils.rs).
                   Pinned by: Python big-integer arithmetic mod 2^bits; exact rational arithmetic
                   (fractions.Fraction) rounded once for the half types.
"""
from __future__ import annotations

import numpy as np

ADD, SUB, MUL, DIV = range(4)


def contiguous(a: np.ndarray) -> np.ndarray:
    return np.array(a, order="C", copy=True)


def full(value, shape, dtype) -> np.ndarray:
    return np.full(shape, value, dtype)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7fffffff) > 0x7f800000
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def binary(op: int, a: np.ndarray, b: np.ndarray, bf16: bool = False) -> np.ndarray:
    """`bf16`: a and b hold bf16 bit patterns (uint16); the result does too."""
    a, b = np.broadcast_arrays(a, b)
    if bf16:
        x, y = bf16_bits_to_f32(a), bf16_bits_to_f32(b)
        with np.errstate(all="ignore"):
            r = (x + y, x - y, x * y, x / y)[op]
        return f32_to_bf16_bits(r.astype(np.float32)).reshape(a.shape)
    dt = a.dtype
    if dt == np.bool_:
        if op == ADD:
            return a | b
        if op == MUL:
            return a & b
        raise TypeError("bool: only add and mul are defined")
    with np.errstate(all="ignore"):
        if dt == np.float16:
            x, y = a.astype(np.float32), b.astype(np.float32)
            return (x + y, x - y, x * y, x / y)[op].astype(np.float16)
        if op == DIV:
            if dt.kind != "f":
                raise TypeError("div: float dtypes only")
            return a / b
        return (a + b, a - b, a * b)[op].astype(dt)   # numpy integer arithmetic wraps
