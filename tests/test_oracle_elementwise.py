"""Pins of oracle/elementwise.py (CPU only): the strided copy against brute-force enumeration of index
tuples, integer arithmetic against Python big integers reduced mod 2^bits, half arithmetic against exact
rational arithmetic rounded once."""
import itertools
from fractions import Fraction

import numpy as np
import pytest

from oracle import elementwise as ew


def brute_gather(base_flat, offset, shape, strides):
    out = []
    for idx in itertools.product(*[range(s) for s in shape]):
        out.append(base_flat[offset + sum(i * st for i, st in zip(idx, strides))])
    return out


@pytest.mark.parametrize("case", [
    ((4, 5, 6), lambda a: a.transpose(2, 0, 1)),
    ((4, 5, 6), lambda a: a[1:4, ::2, ::-1]),
    ((7, 3), lambda a: a.T[::2]),
    ((2, 3, 4, 5), lambda a: a.transpose(3, 1, 0, 2)[1:, :, 1]),
    ((6,), lambda a: a[::-2]),
])
def test_contiguous_is_row_major_gather(case):
    shape, view = case
    base = np.arange(int(np.prod(shape)), dtype=np.int32).reshape(shape) * 3 + 1
    v = view(base)
    got = ew.contiguous(v)
    assert got.flags["C_CONTIGUOUS"] and got.shape == v.shape
    off = (v.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // 4
    strides = [s // 4 for s in v.strides]
    assert got.ravel().tolist() == brute_gather(base.ravel(), off, v.shape, strides)


@pytest.mark.parametrize("npdt,bits,signed", [(np.int8, 8, True), (np.uint8, 8, False), (np.int16, 16, True),
                                              (np.uint16, 16, False), (np.int32, 32, True), (np.uint32, 32, False),
                                              (np.int64, 64, True), (np.uint64, 64, False)])
def test_integer_ops_wrap_like_big_integers_mod_2n(npdt, bits, signed):
    rng = np.random.default_rng(bits + signed)
    info = np.iinfo(npdt)
    a = rng.integers(info.min, info.max, 200, dtype=npdt, endpoint=True)
    b = rng.integers(info.min, info.max, 200, dtype=npdt, endpoint=True)
    a[:3] = [info.max, info.min, info.max]
    b[:3] = [1, info.max, info.max]

    def wrap(x):
        x &= (1 << bits) - 1
        return x - (1 << bits) if signed and x >= 1 << (bits - 1) else x

    for op, f in ((ew.ADD, lambda x, y: x + y), (ew.SUB, lambda x, y: x - y), (ew.MUL, lambda x, y: x * y)):
        got = ew.binary(op, a, b)
        assert got.dtype == npdt
        assert got.tolist() == [wrap(f(int(x), int(y))) for x, y in zip(a, b)]


def _round_to(fr: Fraction, bits_mant: int, emin: int, emax: int):
    """Round an exact rational to a binary float with `bits_mant` significant bits (RNE), as a Fraction."""
    if fr == 0:
        return Fraction(0)
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = 0
    while fr >= 2:
        fr /= 2
        e += 1
    while fr < 1:
        fr *= 2
        e -= 1
    e_eff = max(e, emin)                      # subnormals share the exponent emin
    scale = Fraction(2) ** (e_eff - (bits_mant - 1))
    q = (Fraction(2) ** e * fr) / scale
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    return sign * n * scale


def test_f16_ops_are_one_rounding_of_the_exact_result():
    rng = np.random.default_rng(9)
    a = (rng.standard_normal(300) * 10).astype(np.float16)
    b = (rng.standard_normal(300) * 0.37).astype(np.float16)
    a[:4] = [np.float16(6e-8), np.float16(1024), np.float16(-0.1), np.float16(3)]
    b[:4] = [np.float16(6e-8), np.float16(0.5), np.float16(0.3), np.float16(7)]
    for op, f in ((ew.ADD, lambda x, y: x + y), (ew.SUB, lambda x, y: x - y), (ew.MUL, lambda x, y: x * y),
                  (ew.DIV, lambda x, y: x / y)):
        got = ew.binary(op, a, b)
        for x, y, g in zip(a, b, got):
            exact = f(Fraction(float(x)), Fraction(float(y)))
            want = _round_to(exact, 11, -14, 15)
            if abs(want) > 65504:
                assert np.isinf(g)
            else:
                assert Fraction(float(g)) == want, (op, float(x), float(y), float(g), float(want))


def test_bf16_ops_are_one_rounding_of_the_exact_result():
    rng = np.random.default_rng(10)
    a = ew.f32_to_bf16_bits((rng.standard_normal(300) * 10).astype(np.float32))
    b = ew.f32_to_bf16_bits((rng.standard_normal(300) * 0.37).astype(np.float32))
    for op, f in ((ew.ADD, lambda x, y: x + y), (ew.SUB, lambda x, y: x - y), (ew.MUL, lambda x, y: x * y)):
        got = ew.bf16_bits_to_f32(ew.binary(op, a, b, bf16=True))
        for x, y, g in zip(ew.bf16_bits_to_f32(a), ew.bf16_bits_to_f32(b), got):
            exact = f(Fraction(float(x)), Fraction(float(y)))
            assert Fraction(float(g)) == _round_to(exact, 8, -126, 127)


def test_bool_and_broadcast():
    a = np.array([[True], [False]])
    b = np.array([True, False, False])
    assert ew.binary(ew.ADD, a, b).tolist() == [[True, True, True], [True, False, False]]
    assert ew.binary(ew.MUL, a, b).tolist() == [[True, False, False], [False, False, False]]
    with pytest.raises(TypeError):
        ew.binary(ew.SUB, a, b)
    x = np.arange(6, dtype=np.float32).reshape(2, 3)
    assert ew.binary(ew.MUL, x, np.array([1, 10, 100], np.float32)).tolist() == [[0, 10, 200], [3, 40, 500]]
    assert ew.full(7, (2, 2), np.int16).tolist() == [[7, 7], [7, 7]]


def test_cast_ties_and_ranges():
    # f64 -> f16: values a hair above a tie must round up (a detour through f32 would round to even first)
    d = np.array([1 + 2.0 ** -11 + 2.0 ** -40, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11, 65519.999, 65520.0, 6e-8, -2.5e-8])
    got = ew.cast(d, np.float16)
    want = [1 + 2.0 ** -10, 1.0, 1 + 2.0 ** -9, 65504.0, np.inf, 2.0 ** -24, -0.0]
    assert [float(v) for v in got] == want
    for x, g in zip(d[:4], got[:4]):
        assert Fraction(float(g)) == _round_to(Fraction(float(x)), 11, -14, 15)
    # f64 -> bf16, one rounding
    b = ew.cast(np.array([1 + 2.0 ** -8 + 2.0 ** -40, 1 + 2.0 ** -8, 3.0e38, 3.4e38]), "bf16")
    assert ew.bf16_bits_to_f32(b).tolist()[:2] == [1 + 2.0 ** -7, 1.0]
    assert np.isfinite(ew.bf16_bits_to_f32(b)[2]) and np.isinf(ew.bf16_bits_to_f32(b)[3])
    # integers
    assert ew.cast(np.array([32767, -32768, 2049, 2051], np.int16), np.float16).tolist() == [32768.0, -32768.0, 2048.0, 2052.0]
    assert ew.cast(np.array([16777217, -16777219], np.int32), np.float32).tolist() == [16777216.0, -16777220.0]
    assert ew.cast(np.array([(1 << 53) + 1, (1 << 64) - 1], np.uint64), np.float64).tolist() == [float(1 << 53), float(1 << 64)]
    assert ew.cast(np.array([True, False]), np.float16).tolist() == [1.0, 0.0]
