"""The five benchmark configurations at their full sizes: parity with the oracle where it finishes
in seconds, and size-independent properties on the whole output."""
import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol

pytestmark = pytest.mark.gpu


def test_c1_softmax_sum_max(hpt, orc, dev):
    rng = np.random.default_rng(0)
    x = rng.uniform(-10, 10, (1024, 1024)).astype(np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    s = t.softmax(1).numpy()
    assert_close(s, orc.softmax(x, 1, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, "C1 softmax")
    assert_close(s.astype(np.float64).sum(1), np.ones(1024), 1e-6, 0, "rows sum to 1")
    assert_close(t.sum([1]).numpy(), orc.reduce(orc.SUM, x, [1], acc=orc.ACC_F64), F32_RTOL, F32_ATOL, "C1 sum")
    assert np.array_equal(t.max([1]).numpy(), x.max(1))
    # against the literal f32 lane-structured CPU path: its own summation error sets the scale
    nat = orc.reduce(orc.SUM, x, [1], lanes=8)
    assert_close(t.sum([1]).numpy(), nat, 1e-5, 1e-5 * np.abs(x).sum(1).max() / 1024 * 32, "C1 sum vs f32 CPU path")


def test_c2_layernorm_log_softmax(hpt, orc, dev):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((8192, 4096), dtype=np.float32)
    x += rng.uniform(-5, 5, (8192, 1)).astype(np.float32)
    g = rng.normal(1, 0.1, 4096).astype(np.float32)
    b = rng.normal(0, 0.1, 4096).astype(np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
    y = t.layernorm([4096], tg, tb, 1e-5).numpy()
    rows = np.r_[0:96, 4000:4064, 8128:8192]
    assert_close(y[rows], orc.layernorm(x[rows], 1, g, b, 1e-5, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, "C2 layernorm")
    # whole output: undo the affine map, every row must have mean 0 and biased variance 1/(1+eps/var)
    z = (y.astype(np.float64) - b) / g
    assert np.abs(z.mean(1)).max() < 2e-6
    var = x.astype(np.float64).var(1)
    assert_close(z.var(1), 1 / (1 + 1e-5 / var), 2e-5, 0, "C2 unit variance")
    ls = t.log_softmax(1).numpy()
    assert_close(ls[rows], orc.softmax(x[rows], 1, log=True, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, "C2 log_softmax")
    assert_close(np.exp(ls.astype(np.float64)).sum(1), np.ones(8192), 1e-5, 0, "exp(log_softmax) sums to 1")
    # the multithreaded f32 restatement of Hpt's CPU layernorm agrees to its own summation error
    cpu = orc.mt_layernorm_f32(x[rows], g, b, 1e-5, 4)
    assert_close(y[rows], cpu, 1e-4, 1e-4, "C2 layernorm vs f32 CPU path")


def test_c3_axis_reductions(hpt, orc, dev):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((64, 128, 56, 56), dtype=np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    xd = x.astype(np.float64)
    assert_close(t.sum([2, 3]).numpy(), xd.sum((2, 3)), F32_RTOL, F32_ATOL, "C3 sum[2,3]")
    assert_close(t.mean([2, 3]).numpy(), xd.mean((2, 3)), F32_RTOL, F32_ATOL, "C3 mean[2,3]")
    assert np.array_equal(t.max([1]).numpy(), x.max(1))
    full = t.sum([0, 1, 2, 3]).numpy()
    assert full.shape == (1,)
    assert_close(full, [xd.sum()], F32_RTOL, F32_ATOL, "C3 full sum")
    assert_close(t.sum([2, 3], True).numpy(), orc.reduce(orc.SUM, x, [2, 3], True, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, "oracle")
    # linearity: sum over [2,3] then over everything equals the full sum
    assert_close(t.sum([2, 3]).sum([0, 1]).numpy(), [xd.sum()], F32_RTOL, 1e-5, "sum of sums")
    rng = np.random.default_rng(3)
    xi = rng.integers(-1000, 1001, (64, 128, 56, 56)).astype(np.int32)
    ti = hpt.Tensor.from_numpy(xi).to_hip(dev)
    assert np.array_equal(ti.sum([1]).numpy(), xi.sum(1, dtype=np.int32))
    am = ti.argmax(1).numpy()
    assert am.dtype == np.int64 and am.shape == (64, 56, 56)
    assert np.array_equal(am, xi.argmax(1))
    assert np.array_equal(am, orc.argreduce(True, xi, 1))
    mx = xi.max(1)
    ties = ((xi == mx[:, None]).sum(1) > 1).sum()
    assert ties > 1000, "the tie rule must actually be exercised"


def test_c4_causal_bf16_softmax(hpt, orc, dev):
    rng = np.random.default_rng(4)
    rows_total, n = 65536, 2048
    x = rng.standard_normal((rows_total, n), dtype=np.float32) * 3
    q = (np.arange(rows_total) % n)[:, None]
    x[np.arange(n)[None, :] > q] = -np.inf
    xb = hpt.f32_to_bf16_bits(x)
    del x
    t = hpt.Tensor.from_numpy(xb, hpt.bf16).to_hip(dev)
    out_bits = t.softmax(1).numpy()
    out = hpt.bf16_bits_to_f32(out_bits)
    rows = np.r_[0:48, 2040:2056, 65500:65536]
    want = hpt.bf16_bits_to_f32(orc.softmax(xb[rows], 1, acc=orc.ACC_F32, dtype=orc.BF16))
    assert_close(out[rows], want, HALF_RTOL, half_atol(want, 8), "C4 softmax")
    # first row of each head has a single finite key: exactly one-hot
    first = out[::n]
    assert np.all(first[:, 0] == 1.0) and not first[:, 1:].any()
    # masked positions are exactly zero, rows sum to 1 within bf16 rounding of up to 2048 terms
    masked = np.arange(n)[None, :] > (np.arange(4096) % n)[:, None]
    assert not out[:4096][masked].any()
    assert np.abs(out.astype(np.float64).sum(1) - 1).max() < 2e-2


def test_c5_non_contiguous_f16(hpt, orc, dev):
    rng = np.random.default_rng(5)
    base = (rng.standard_normal((4096, 8192), dtype=np.float32) * 2).astype(np.float16)
    g = rng.normal(1, 0.1, 4096).astype(np.float16)
    b = rng.normal(0, 0.1, 4096).astype(np.float16)
    t = hpt.Tensor.from_numpy(base).to_hip(dev)
    tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
    f = lambda a: a.astype(np.float32)
    for name, tv, av in (("C5a transposed", t.permute([1, 0]), base.T), ("C5b [:, ::2]", t[:, ::2], base[:, ::2])):
        rows = np.r_[0:40, av.shape[0] - 24:av.shape[0]]
        ln = f(tv.layernorm([4096], tg, tb, 1e-5).numpy())
        assert ln.shape == av.shape
        want = f(orc.layernorm(av[rows], 1, g, b, 1e-5, acc=orc.ACC_F32))
        assert_close(ln[rows], want, HALF_RTOL, half_atol(want, 11), name + " layernorm")
        z = (ln.astype(np.float64) - f(b)) / f(g)
        assert np.abs(z.mean(1)).max() < 5e-3 and np.abs(z.var(1) - 1).max() < 2e-2
        sm = f(tv.softmax(1).numpy())
        want = f(orc.softmax(av[rows], 1, acc=orc.ACC_F32))
        assert_close(sm[rows], want, HALF_RTOL, max(half_atol(want, 11), 6e-8), name + " softmax")
        assert np.abs(sm.astype(np.float64).sum(1) - 1).max() < 5e-3
        s0 = f(tv.sum([0]).numpy())
        want = f(orc.reduce(orc.SUM, av, [0], acc=orc.ACC_F32))
        assert_close(s0, want, HALF_RTOL, half_atol(want, 11), name + " sum(axis=0)")


def test_reference_published_sum_shape(hpt, orc, dev):
    """f32 [1024, 1024, 80] summed over the seven axis sets the reference publishes timings for
    (docs/benchmarks/reduce.md:62-78): every output against numpy's float64 sum of the same elements."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal((1024, 1024, 80), dtype=np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    xd = x.astype(np.float64)
    for axes in ([0], [1], [2], [0, 1], [0, 2], [1, 2], [0, 1, 2]):
        got = t.sum(axes).numpy()
        want = xd.sum(tuple(axes))
        assert_close(got.reshape(want.shape) if want.shape else got.reshape(()), want, F32_RTOL, F32_ATOL, f"sum over {axes}")
    # the exactly summed oracle on one output row of each kind (numpy's pairwise f64 sum is the other witness)
    assert_close(t.sum([0, 2]).numpy()[:8], orc.reduce(orc.SUM, x[:, :8, :], [0, 2], acc=orc.ACC_EXACT), F32_RTOL, F32_ATOL, "sum(0,2) exact")
    del xd


@pytest.mark.parametrize("n", [256, 512])
def test_reference_published_softmax_shapes(hpt, orc, dev, n):
    """f32 softmax of n^3 over each axis (docs/benchmarks/normalization.md:55-123): a sample of positions against the
    f64 oracle, and over the whole output every softmax vector sums to one and keeps the order of its inputs."""
    rng = np.random.default_rng(12 + n)
    x = rng.standard_normal((n, n, n), dtype=np.float32) * 2
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    for axis in (0, 1, 2):
        y = t.softmax(axis).numpy()
        assert_close(y.sum(axis, dtype=np.float64), np.ones((n, n)), 2e-6, 0, f"softmax({axis}) sums to one")
        sl = [slice(None)] * 3
        for d in range(3):
            if d != axis:
                sl[d] = slice(n // 2 - 3, n // 2 + 5) if d == (axis + 1) % 3 else slice(0, n, max(1, n // 16))
        sl = tuple(sl)
        assert_close(y[sl], orc.softmax(np.ascontiguousarray(x[sl]), axis, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"softmax({axis}) sample")
        # monotone: the largest input of a vector has the largest output
        assert np.array_equal(y.argmax(axis), x.argmax(axis)) or np.allclose(
            np.take_along_axis(y, np.expand_dims(x.argmax(axis), axis), axis), y.max(axis, keepdims=True))
        ly = t.log_softmax(axis).numpy()
        assert_close(ly[sl], orc.softmax(np.ascontiguousarray(x[sl]), axis, log=True, acc=orc.ACC_F64), F32_RTOL, F32_ATOL,
                     f"log_softmax({axis}) sample")
        del y, ly
