"""The oracle's shape logic against the reference's own known-answer tests (CPU only)."""
import itertools

import numpy as np
import pytest

BIG = 0x7FFFFFFFFFFFFFFF


def test_process_axes_kats(orc):
    # hpt-tests/src/hpt_common/axis.rs:6-50
    with pytest.raises(ValueError, match=r"Dimension out of range: expected in 0\.\.2, got 10"):
        orc.process_axes(10, 2)
    with pytest.raises(ValueError, match=r"Dimension out of range: expected in 0\.\.2, got -1"):
        orc.process_axes(-3, 2)
    assert orc.process_axes(-1, 2) == [1]
    assert orc.process_axes([1, 2, 3], 4) == [1, 2, 3]
    # hpt-common/src/error/param.rs:17
    with pytest.raises(ValueError, match="Axis 1 is duplicated"):
        orc.process_axes([1, 1], 3)


def test_mt_intervals_kats(orc):
    # doc tests of hpt-common/src/shape/shape_utils.rs:700-760
    assert orc.mt_intervals(100, 4) == [(0, 25), (25, 50), (50, 75), (75, 100)]
    assert orc.mt_intervals(10, 3) == [(0, 4), (4, 7), (7, 10)]
    assert orc.mt_intervals(5, 10) == [(0, 1), (1, 2), (2, 3), (3, 4), (4, 5)] + [(5, 5)] * 5
    assert orc.mt_intervals(0, 4) == [(0, 0)] * 4
    assert orc.mt_intervals(10, 0) == []
    # hpt-tests/src/hpt_common/shape_utils.rs:12-52
    assert orc.mt_intervals_simd(100, 4, 10) == [(0, 30), (30, 60), (60, 80), (80, 100)]
    assert orc.mt_intervals_simd(16, 10, 4) == [(0, 4), (4, 8), (8, 12), (12, 16)] + [(16, 16)] * 6
    assert orc.mt_intervals_simd(4, 10, 8) == [(0, 4)] + [(0, 0)] * 9
    assert orc.mt_intervals_simd(102, 4, 10) == [(0, 30), (30, 60), (60, 80), (80, 102)]


def test_mt_intervals_partition_property(orc):
    for size, n in itertools.product([0, 1, 7, 64, 1000, 8192], [1, 2, 3, 16, 31]):
        iv = orc.mt_intervals(size, n)
        assert iv[0][0] == 0 and iv[-1][1] == size
        assert all(a[1] == b[0] for a, b in zip(iv, iv[1:]))
        lens = [b - a for a, b in iv]
        assert max(lens) - min(lens) <= 1


def test_slice_process_kat_and_numpy(orc):
    # doc example hpt-common/src/slice.rs:30-38
    assert orc.slice_process([3, 4, 5], [20, 5, 1], [(1, BIG, 1), (0, 3, 1), (0, BIG, 2)]) == ([2, 3, 3], [20, 5, 2], 20)
    # brute force against numpy slicing on a small tensor
    rng = np.random.default_rng(7)
    a = np.arange(4 * 5 * 6).reshape(4, 5, 6)
    flat = a.reshape(-1)
    for _ in range(200):
        idx, sl = [], []
        for d in a.shape:
            step = int(rng.integers(1, 4))
            start = int(rng.integers(0, d))
            end = int(rng.integers(start + 1, d + 1))
            idx.append((start, end, step))
            sl.append(slice(start, end, step))
        shape, strides, off = orc.slice_process(list(a.shape), [30, 6, 1], idx)
        got = np.lib.stride_tricks.as_strided(flat[off:], shape, [s * 8 for s in strides])
        assert np.array_equal(got, a[tuple(sl)])
    # negative start / end wrap like Python's
    shape, strides, off = orc.slice_process([10], [1], [(-4, -1, 1)])
    assert (shape, strides, off) == ([3], [1], 6)


def test_reduce_shape(orc):
    # Layout::reduce, hpt-common/src/layout/layout_utils.rs:310-344
    assert orc.reduce_shape([2, 3, 4], [1], False) == [2, 4]
    assert orc.reduce_shape([2, 3, 4], [1], True) == [2, 1, 4]
    assert orc.reduce_shape([2, 3, 4], [0, 1, 2], False) == [1]          # full reduction -> [1]
    assert orc.reduce_shape([2, 3, 4], [0, 1, 2], True) == [1, 1, 1]
    assert orc.reduce_shape([2, 3, 4], [-1, 0], False) == [3]
    for shape in ([3], [2, 5], [4, 1, 6], [2, 3, 4, 5]):
        for r in range(1, len(shape) + 1):
            for axes in itertools.combinations(range(len(shape)), r):
                want = np.zeros(shape).sum(axis=axes)
                assert orc.reduce_shape(shape, list(axes), False) == (list(want.shape) or [1])
                assert orc.reduce_shape(shape, list(axes), True) == list(np.zeros(shape).sum(axis=axes, keepdims=True).shape)


def test_is_contiguous_and_coalesce(orc):
    rng = np.random.default_rng(8)
    a = np.zeros((3, 4, 5, 6), np.float32)
    es = a.itemsize
    for _ in range(100):
        v = a.transpose(rng.permutation(4))
        if rng.random() < 0.5:
            v = v[:, ::2]
        strides = [s // es for s in v.strides]
        assert orc.is_contiguous(list(v.shape), strides) == v.flags["C_CONTIGUOUS"]
    # zero-sized dims are skipped (layout_utils.rs:363-375)
    assert orc.is_contiguous([2, 0, 3], [3, 99, 1]) and not orc.is_contiguous([2, 0, 3], [0, 3, 1])
    # coalesce_dims: hand-worked cases (layout_utils.rs:384-410)
    assert orc.coalesce_dims([2, 3, 4], [12, 4, 1]) == [[0, 1, 2]]
    assert orc.coalesce_dims([2, 3, 4], [24, 4, 1]) == [[0], [1, 2]]
    assert orc.coalesce_dims([2, 3, 4], [12, 8, 1]) == [[0], [1], [2]]
    assert orc.coalesce_dims([64, 128, 56, 56], [401408, 3136, 56, 1]) == [[0, 1, 2, 3]]
    # invariant: merging each group into one dim of the product size and the last stride
    # addresses exactly the same offsets in the same order
    for _ in range(100):
        v = a.transpose(rng.permutation(4))[:, :, ::int(rng.integers(1, 3))]
        shape, strides = list(v.shape), [s // es for s in v.strides]
        groups = orc.coalesce_dims(shape, strides)
        mshape = [int(np.prod([shape[d] for d in g])) for g in groups]
        mstrides = [strides[g[-1]] for g in groups]
        offs = lambda sh, st: [sum(i * s for i, s in zip(ix, st)) for ix in itertools.product(*[range(n) for n in sh])]
        assert offs(shape, strides) == offs(mshape, mstrides)


def test_float_out_dtype_table(orc):
    # hpt-types/src/promotion/normal_promote/_*.rs: impl_float_out_binary_promote!(T, T, ...)
    want = {orc.BOOL: orc.F16, orc.I8: orc.F16, orc.I16: orc.F16, orc.I32: orc.F32, orc.I64: orc.F64,
            orc.U8: orc.F16, orc.U16: orc.F16, orc.U32: orc.F32, orc.U64: orc.F64, orc.F16: orc.F16,
            orc.BF16: orc.BF16, orc.F32: orc.F32, orc.F64: orc.F64}
    for dt, out in want.items():
        assert orc.reduce_out_dtype(orc.MEAN, dt) == out
        assert orc.reduce_out_dtype(orc.SUM, dt) == dt
        assert orc.reduce_out_dtype(orc.ALL, dt) == orc.BOOL


def test_half_conversions(orc):
    l = orc.lib()
    # every f16 bit pattern round-trips and matches numpy's float16
    bits = np.arange(65536, dtype=np.uint16)
    f = bits.view(np.float16).astype(np.float32)
    for b in list(range(0, 65536, 97)) + [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0xFC00, 0x8000]:
        x = l.orc_f16_to_f32(b)
        assert (np.isnan(x) and np.isnan(f[b])) or x == f[b]
        if not np.isnan(f[b]):
            assert l.orc_f32_to_f16(float(f[b])) == b
    rng = np.random.default_rng(9)
    xs = np.concatenate([rng.standard_normal(2000) * 10 ** rng.uniform(-8, 5, 2000), [65504.0, 65520.0, 1e-8, 6e-8]]).astype(np.float32)
    for x in xs:
        assert l.orc_f32_to_f16(float(x)) == int(np.float16(x).view(np.uint16)), x
    # bf16: round-to-nearest-even against the definition
    for x in xs:
        u = np.float32(x).view(np.uint32)
        lo, up = (u >> 16) << 16, ((u >> 16) + 1) << 16
        got = np.uint32(l.orc_f32_to_bf16(float(x))) << 16
        d_lo, d_up = abs(int(u) - int(lo)), abs(int(up) - int(u))
        want = lo if d_lo < d_up or (d_lo == d_up and ((lo >> 16) & 1) == 0) else up
        assert got == want
    assert np.array_equal(orc.f32_to_bf16(xs), np.array([l.orc_f32_to_bf16(float(x)) for x in xs], np.uint16))
