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


def cast(a: np.ndarray, to, bf16_in: bool = False):
    """Scalar<T>::cast as astype uses it (hpt/src/backends/cuda/tensor_impls.rs:129-140), to a float dtype.
    `to`: a numpy float dtype, or the string "bf16" (result: uint16 bit patterns). Integers -> f16 / bf16 go
    through f32 (the generated conversions do `self as f32` first); everything else is one rounding, which is
    what numpy's astype does. Pinned by: exact rational arithmetic on tie cases (tests/test_oracle_elementwise.py)."""
    src = bf16_bits_to_f32(a) if bf16_in else a
    if to == "bf16":
        with np.errstate(all="ignore"):
            return f32_to_bf16_bits(src.astype(np.float32)) if src.dtype != np.float64 else _f64_to_bf16(src)
    with np.errstate(all="ignore"):
        return src.astype(to)


def _f64_to_bf16(d: np.ndarray) -> np.ndarray:
    """One rounding (nearest even) of f64 to bf16, on the bit patterns."""
    u = np.ascontiguousarray(d, np.float64).view(np.uint64)
    sign = ((u >> 63) & 1).astype(np.uint16) << 15
    mag = u & np.uint64(0x7fffffffffffffff)
    out = np.zeros(d.shape, np.uint16)
    flat_mag, flat_out = mag.ravel(), out.ravel()
    vals = np.abs(d).ravel()
    for i, (m, v) in enumerate(zip(flat_mag, vals)):
        if np.isnan(v):
            flat_out[i] = 0x7fc0
        elif np.isinf(v):
            flat_out[i] = 0x7f80
        else:
            from fractions import Fraction
            fr = Fraction(float(v))
            if fr == 0:
                flat_out[i] = 0
                continue
            e = 0
            t = fr
            while t >= 2:
                t /= 2; e += 1
            while t < 1:
                t *= 2; e -= 1
            e_eff = max(e, -126)
            scale = Fraction(2) ** (e_eff - 7)
            q = fr / scale
            n = q.numerator // q.denominator
            rem = q - n
            if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
                n += 1
            r = n * scale
            if r >= Fraction(2) ** 128:
                flat_out[i] = 0x7f80
            else:
                flat_out[i] = f32_to_bf16_bits(np.array([float(r)], np.float32))[0]
    return (out | sign.reshape(out.shape)).astype(np.uint16)
