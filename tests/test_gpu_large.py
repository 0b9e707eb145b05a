"""Maximum sizes: tensors with more than 2^31 elements (index arithmetic must be 64-bit where it has
to be). Integer ops are bit-exact against numpy; about 2 GiB per tensor."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

BIG = (1 << 31) + 4096   # elements; > INT32_MAX


def test_one_dim_beyond_int32(hpt, dev):
    rng = np.random.default_rng(500)
    a = rng.integers(0, 256, BIG, dtype=np.uint8)
    t = hpt.Tensor.from_numpy(a).to_hip(dev)
    assert t.sum([0]).numpy()[0] == a.sum(dtype=np.uint8)
    assert t.max([0]).numpy()[0] == a.max()
    # arg-reductions carry 32-bit positions: a longer axis is refused, not mis-indexed
    with pytest.raises(hpt.ShapeError, match="exceeds 2\\^31-1"):
        t.argmax(0)
    assert t[:(1 << 31) - 1].argmax(0).numpy()[0] == int(a[:(1 << 31) - 1].argmax())
    # a view that starts beyond 2^31 elements into the buffer
    tail = t[(1 << 31) + 7:]
    assert tail.sum([0]).numpy()[0] == a[(1 << 31) + 7:].sum(dtype=np.uint8)
    # elementwise over > 2^31 elements, in place
    ones = hpt.Tensor.ones([1], hpt.u8, dev)
    t.add_(ones, t)
    back = t.to_cpu().numpy()
    assert np.array_equal(back[:1 << 20], a[:1 << 20] + np.uint8(1))
    assert np.array_equal(back[-(1 << 20):], a[-(1 << 20):] + np.uint8(1))
    assert int(back.sum(dtype=np.uint64)) == int((a + np.uint8(1)).sum(dtype=np.uint64))


def test_two_dims_total_beyond_int32(hpt, dev):
    rng = np.random.default_rng(501)
    a = rng.integers(-128, 128, (3, (1 << 30) + 64), dtype=np.int8)
    t = hpt.Tensor.from_numpy(a).to_hip(dev)
    assert np.array_equal(t.sum([1]).numpy(), a.sum(1, dtype=np.int8))          # 3 outputs, 2^30 terms each
    assert np.array_equal(t.max([0]).numpy(), a.max(0))                          # 2^30 outputs
    assert np.array_equal(t.sum([0, 1]).numpy(), np.array([a.sum(dtype=np.int8)]))
    assert np.array_equal(t.argmin(1).numpy(), a.argmin(1))
    tt = t.permute([1, 0])                                                       # [2^30 + 64, 3], strides [1, 2^30 + 64]
    assert np.array_equal(tt.sum([0]).numpy(), a.sum(1, dtype=np.int8))
    c = tt[(1 << 30) - 5:].contiguous().numpy()                                  # offsets beyond 2^31 bytes
    assert np.array_equal(c, a.T[(1 << 30) - 5:])


def test_normalisation_beyond_int32_elements(hpt, orc, dev):
    """f16 [2^20, 2304] (2.4 G elements): row kernels with 64-bit row offsets; checked on the first and last
    rows against the oracle and on every row through the sum-to-one property."""
    from conftest import assert_close
    rows, cols = 1 << 20, 2304
    rng = np.random.default_rng(502)
    block = (rng.standard_normal((1 << 12, cols)) * 2).astype(np.float16)
    a = np.tile(block, (rows >> 12, 1))
    a[-3:] += np.float16(1.5)          # make the last rows differ from the tiled pattern
    t = hpt.Tensor.from_numpy(a).to_hip(dev)
    s = t.softmax(1).numpy()
    sel = np.r_[0:64, rows - 64:rows]
    want = orc.softmax(np.ascontiguousarray(a[sel]), 1, acc=orc.ACC_F32).astype(np.float32)
    assert_close(s[sel].astype(np.float32), want, 1e-2, 6e-8, "softmax rows at both ends")
    sums = s.astype(np.float32).sum(1)
    assert np.all(np.abs(sums - 1) < 2e-2)
    del s
    g = rng.normal(1, 0.1, cols).astype(np.float16)
    ln = t.layernorm([cols], hpt.Tensor.from_numpy(g).to_hip(dev), None, 1e-5).numpy()
    want = orc.layernorm(np.ascontiguousarray(a[sel]), 1, g, None, 1e-5, acc=orc.ACC_F32).astype(np.float32)
    assert_close(ln[sel].astype(np.float32), want, 1e-2, 2e-3, "layernorm rows at both ends")
    del ln
    # columns: softmax over axis 0 of the transposed view's base layout ([cols, rows] rows contiguous)
    b = np.ascontiguousarray(a[:, :8].T)          # [8, 2^20]
    tb = hpt.Tensor.from_numpy(b).to_hip(dev)
    got = tb.softmax(0).numpy().astype(np.float32)
    want = orc.softmax(b, 0, acc=orc.ACC_F32).astype(np.float32)
    assert_close(got, want, 1e-2, 6e-8, "column softmax")


def test_short_rows_and_narrow_columns_beyond_int32_elements(hpt, dev):
    """int8 [2^29 + 5, 5] (2.7 G elements): the LDS row tiles (axis 1) and the flat column walk (axis 0)
    with offsets beyond 2^31; bit-exact against numpy."""
    rng = np.random.default_rng(503)
    rows = (1 << 29) + 5
    block = rng.integers(-128, 128, (1 << 20, 5), dtype=np.int8)
    a = np.tile(block, ((rows >> 20) + 1, 1))[:rows]
    a[-7:] = rng.integers(-128, 128, (7, 5), dtype=np.int8)
    t = hpt.Tensor.from_numpy(a).to_hip(dev)
    assert hpt.reduce_plan(t, hpt.SUM, [1]).startswith("row-tile") and hpt.reduce_plan(t, hpt.SUM, [0]).startswith("col-flat")
    assert np.array_equal(t.sum([1]).numpy(), a.sum(1, dtype=np.int8))
    assert np.array_equal(t.sum([0]).numpy(), a.sum(0, dtype=np.int8))
    assert np.array_equal(t.max([0]).numpy(), a.max(0))
    got = t.argmax(1).numpy()
    sel = np.r_[0:1 << 16, rows - (1 << 16):rows]
    assert np.array_equal(got[sel], a[sel].argmax(1))
    assert int(got.sum()) == int(a.argmax(1).sum())
    # the first extremum of each column, over 2^29 rows of a tiled pattern: always inside the first block
    assert np.array_equal(t.argmin(0).numpy(), a.argmin(0))


def test_short_row_and_channel_softmax_beyond_int32_elements(hpt, dev):
    """f16 [2^27 + 3, 17] (2.3 G elements): softmax over the short rows (row tiles in LDS), log_softmax over the
    long axis (flat column walk, two passes); f16 [40, 16, 2^22 + 8] (2.7 G elements): softmax over the channel
    axis held in registers. Checked against a float64 numpy softmax on slices at both ends, and on every
    vector through the sum-to-one property."""
    from conftest import assert_close

    def ref(x, axis):
        x = x.astype(np.float64)
        e = np.exp(x - x.max(axis, keepdims=True))
        return (e / e.sum(axis, keepdims=True)).astype(np.float32)

    rng = np.random.default_rng(504)
    rows = (1 << 27) + 3
    block = (rng.standard_normal((1 << 18, 17)) * 2).astype(np.float16)
    a = np.tile(block, ((rows >> 18) + 1, 1))[:rows]
    a[-5:] += np.float16(0.75)
    t = hpt.Tensor.from_numpy(a).to_hip(dev)
    assert "+tile" in hpt.normalize_plan(t, 1) and "flat" in hpt.normalize_plan(t, 0)
    s = t.softmax(1).numpy()
    sel = np.r_[0:4096, rows - 4096:rows]
    assert_close(s[sel].astype(np.float32), ref(a[sel], 1), 1e-2, 6e-8, "short-row softmax at both ends")
    assert np.all(np.abs(s.sum(1, dtype=np.float32) - 1) < 2e-2)
    del s
    # over the long axis the probabilities (~1e-8) are below what f16 holds: log_softmax instead
    s0 = t.log_softmax(0).numpy()
    x = a.astype(np.float64)
    want = x[sel] - (np.log(np.exp(x - x.max(0)).sum(0)) + x.max(0))
    del x
    assert_close(s0[sel].astype(np.float32), want.astype(np.float32), 1e-2, 1e-2, "long-axis log_softmax at both ends")
    total = np.zeros(17)
    for lo in range(0, rows, 1 << 24):
        total += np.exp(s0[lo:lo + (1 << 24)].astype(np.float64)).sum(0)
    assert np.all(np.abs(total - 1) < 1e-2), total
    del s0, t, a

    L = (1 << 22) + 8
    block = (rng.standard_normal((40, 16, 1 << 12)) * 2).astype(np.float16)
    b = np.tile(block, (1, 1, (L >> 12) + 1))[:, :, :L]
    b[:, :, -3:] -= np.float16(0.5)
    b = np.ascontiguousarray(b)
    tb = hpt.Tensor.from_numpy(b).to_hip(dev)
    assert hpt.normalize_plan(tb, 1).startswith("col-reg")
    sb = tb.softmax(1).numpy()
    for sl in (np.s_[:, :, :2048], np.s_[:, :, L - 2048:], np.s_[39:, :, L // 2:L // 2 + 2048]):
        assert_close(sb[sl].astype(np.float32), ref(b[sl], 1), 1e-2, 6e-8, "channel softmax")
    assert np.all(np.abs(sb.sum(1, dtype=np.float32) - 1) < 2e-2)
