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
