"""hpt_hip_reduce_static: the entry point that allocates nothing must give what hpt_hip_reduce gives.

Every case here is a reduction that is split over workgroups (its partials go to scratch), called
twice in a row through the C ABI, the second time on a smaller input, and compared bit for bit with
hpt_hip_reduce on the same input (the same kernels run in the same launch shape)."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as orc

pytestmark = pytest.mark.gpu


def _mallocs(hpt, dev):
    n = C.c_uint64()
    hpt._ffi.check(hpt.lib().hpt_hip_alloc_stats(dev, None, None, C.byref(n)))
    return n.value


CASES = [
    # (name, op, dtype, first shape, second (smaller) shape, axes)
    ("full sum f32", "SUM", np.float32, (64, 128, 56, 56), (1000003,), None),
    ("full max f32", "MAX", np.float32, (4194304,), (300001,), None),
    ("rows split f32", "SUM", np.float32, (2, 1048576), (2, 262144), [1]),
    ("cols split u8", "SUM", np.uint8, (30000, 8192), (12000, 8192), [0]),
    ("cols split i32 prod", "PROD", np.int32, (65536, 2048), (40000, 2048), [0]),
    ("flat wide f64", "SUM", np.float64, (2000, 50257), (1200, 50257), [0]),
    ("mean f16", "MEAN", np.float16, (8388608,), (2097157,), None),
]


@pytest.mark.parametrize("name,op,dt,shape1,shape2,axes", CASES, ids=[c[0] for c in CASES])
def test_reduce_static_matches_reduce_twice_in_a_row(hpt, dev, name, op, dt, shape1, shape2, axes):
    rng = np.random.default_rng(7)
    opc = getattr(hpt, op)
    for shape in (shape1, shape2):
        if np.issubdtype(dt, np.floating):
            x = rng.standard_normal(shape).astype(dt)
        else:
            x = rng.integers(0, 100, shape).astype(dt)
        t = hpt.Tensor.from_numpy(x).to_hip(dev)
        ax = list(range(x.ndim)) if axes is None else axes
        assert "split=1 " not in hpt.reduce_plan(t, opc, ax), "the case must be one that uses scratch"
        want = t._reduce(opc, ax, False)
        out = hpt.Tensor.empty(want.shape, want.dtype, dev)
        hpt.synchronize(dev)
        before = _mallocs(hpt, dev)
        got = t._reduce(opc, ax, False, out=out, static_scratch=True)
        assert _mallocs(hpt, dev) == before, "the static entry point reached the device allocator"
        g, w = got.numpy(), want.numpy()
        assert g.tobytes() == w.tobytes(), f"{name} {shape}: static scratch result differs from hpt_hip_reduce"
        # and the oracle, so that both being wrong the same way does not pass
        if op == "SUM" and dt == np.float32:
            ref = orc.reduce(orc.SUM, x, ax, acc=orc.ACC_EXACT)
            np.testing.assert_allclose(g, ref.reshape(g.shape), rtol=1e-5, atol=1e-6)
        if op == "SUM" and dt == np.uint8:
            assert np.array_equal(g, x.sum(0, dtype=np.uint8))
        del t, want, out, got


def test_reduce_static_accumulates_and_refuses_what_does_not_fit(hpt, dev):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((3, 524288)).astype(np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    base = rng.standard_normal(3).astype(np.float32)
    o1 = hpt.Tensor.from_numpy(base).to_hip(dev)
    o2 = hpt.Tensor.from_numpy(base).to_hip(dev)
    t.sum_([1], False, False, o1)
    t._reduce(hpt.SUM, [1], False, init_out=False, out=o2, static_scratch=True)
    assert o1.numpy().tobytes() == o2.numpy().tobytes()
    # 4097 outputs x 204 partials x 8-byte accumulators = 6.4 MiB: beyond the static array
    wide = hpt.Tensor.empty((8190, 4097), hpt.f32, dev)
    outw = hpt.Tensor.empty((4097,), hpt.f32, dev)
    assert "split=204" in hpt.reduce_plan(wide, hpt.SUM, [0])
    with pytest.raises(hpt.MemoryError_, match="static scratch holds"):
        wide._reduce(hpt.SUM, [0], False, out=outw, static_scratch=True)
