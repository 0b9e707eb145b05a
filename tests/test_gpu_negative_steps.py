"""Views with negative steps (`x[::-1]`, `x[:, ::-2]`: hpt-common/src/slice.rs:96-101 turns a negative
step into a negative stride and a start at the far end) through every op of the path, against the
oracle walking the same strides. Small shapes reach the general kernels, the large ones the lean /
register / tile kernels whose planner rules look at |stride|."""
import itertools

import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol, upload

pytestmark = pytest.mark.gpu

R = (None, None, -1)     # reversed
R2 = (None, None, -2)    # reversed, every second
F = (None, None, 1)      # untouched


def views_for(nd):
    """Slice tuples that reverse one dim, all dims, or step backwards by two; plus one after a permute."""
    out = []
    for d in range(nd):
        out.append((f"rev{d}", (("slice", tuple(R if i == d else F for i in range(nd))),)))
    out.append(("rev_all", (("slice", tuple(R for _ in range(nd))),)))
    out.append(("back2_last", (("slice", tuple(R2 if i == nd - 1 else F for i in range(nd))),)))
    out.append(("back2_first", (("slice", tuple(R2 if i == 0 else F for i in range(nd))),)))
    if nd >= 2:
        perm = tuple(range(nd))[::-1]
        out.append(("permuted_rev", (("permute", perm), ("slice", tuple(R if i == 0 else F for i in range(nd))))))
        out.append(("window_rev", (("slice", tuple((-2, 0, -1) if i == nd - 1 else (1, None, 1) for i in range(nd))),)))
    return out


SHAPES = [[37], [9, 40], [6, 33, 10], [3, 4, 5, 6], [300, 1024], [64, 96, 196], [2051, 257]]


@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_reductions_over_negative_step_views(hpt, orc, dev, shape):
    rng = np.random.default_rng(sum(shape))
    base = rng.standard_normal(shape).astype(np.float32)
    ibase = rng.integers(-1000, 1001, shape).astype(np.int32)
    nd = len(shape)
    for name, ops in views_for(nd):
        t, a = upload(hpt, base, ops, dev=dev)
        ti, ai = upload(hpt, ibase, ops, dev=dev)
        if a.size == 0:
            continue
        assert any(s < 0 for s in t.strides), f"{name}: the view must have a negative stride"
        subsets = [list(c) for r in range(1, nd + 1) for c in itertools.combinations(range(nd), r)]
        for axes in subsets:
            want = orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F64)
            assert_close(t.sum(axes).numpy(), want, F32_RTOL, F32_ATOL, f"sum {shape} {name} {axes}")
            assert np.array_equal(ti.sum(axes).numpy(), orc.reduce(orc.SUM, ai, axes)), f"i32 sum {shape} {name} {axes}"
            assert np.array_equal(t.max(axes).numpy(), orc.reduce(orc.MAX, a, axes)), f"max {shape} {name} {axes}"
        # ties: integers in a small range; "lowest index" is the lowest index OF THE VIEW
        ts, small = upload(hpt, (ibase % 7).astype(np.int32), ops, dev=dev)
        flat = lambda r: np.asarray(r).reshape(-1)
        for axis in range(nd):
            assert np.array_equal(ts.argmax(axis).numpy(), orc.argreduce(True, small, axis)), f"argmax {shape} {name} {axis}"
            assert np.array_equal(flat(ts.argmin(axis).numpy()), flat(small.argmin(axis))), f"argmin {shape} {name} {axis}"
            assert np.array_equal(flat(t.argmax(axis).numpy()), flat(a.argmax(axis))), f"argmax f32 {shape} {name} {axis}"


@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_normalisations_over_negative_step_views(hpt, orc, dev, shape):
    rng = np.random.default_rng(1000 + sum(shape))
    base = (rng.standard_normal(shape) * 3).astype(np.float32)
    hbase = (rng.standard_normal(shape) * 2).astype(np.float16)
    nd = len(shape)
    for name, ops in views_for(nd):
        t, a = upload(hpt, base, ops, dev=dev)
        th, ah = upload(hpt, hbase, ops, dev=dev)
        if a.size == 0:
            continue
        for axis in range(nd):
            for log in (False, True):
                want = orc.softmax(a, axis, log=log, acc=orc.ACC_F64)
                got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
                assert_close(got, want, F32_RTOL, 2 * F32_ATOL if log else F32_ATOL, f"softmax log={log} {shape} {name} axis={axis}")
            wanth = orc.softmax(ah, axis, acc=orc.ACC_F32)
            assert_close(th.softmax(axis).numpy(), wanth, HALF_RTOL, max(half_atol(wanth, 11), 6e-8),
                         f"f16 softmax {shape} {name} axis={axis}")
        for nn in range(1, nd + 1):
            ns = list(a.shape[nd - nn:])
            g = rng.normal(1, 0.1, ns).astype(np.float32)
            b = rng.normal(0, 0.1, ns).astype(np.float32)
            tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
            if int(np.prod(ns)) < 2:
                continue
            want = orc.layernorm(a, nn, g, b, 1e-5, acc=orc.ACC_F64)
            assert_close(t.layernorm(ns, tg, tb, 1e-5).numpy(), want, F32_RTOL, 4 * F32_ATOL, f"layernorm {shape} {name} nn={nn}")


def test_negative_step_views_of_the_benchmark_shapes(hpt, orc, dev):
    """The configurations' own shapes, reversed: the lean column / row kernels and the register rows."""
    rng = np.random.default_rng(77)
    x = rng.standard_normal((16, 128, 56, 56)).astype(np.float32)
    xi = rng.integers(-1000, 1001, x.shape).astype(np.int32)
    for name, ops in (("rev_channels", (("slice", (F, R, F, F)),)), ("rev_rows", (("slice", (F, F, R, F)),)),
                      ("rev_inner", (("slice", (F, F, F, R)),)), ("back2_channels", (("slice", (F, R2, F, F)),))):
        t, a = upload(hpt, x, ops, dev=dev)
        ti, ai = upload(hpt, xi, ops, dev=dev)
        assert_close(t.sum([2, 3]).numpy(), orc.reduce(orc.SUM, a, [2, 3], acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"sum[2,3] {name}")
        assert np.array_equal(t.max([1]).numpy(), a.max(1)), f"max(1) {name}"
        assert np.array_equal(ti.sum([1]).numpy(), ai.sum(1, dtype=np.int32)), f"i32 sum(1) {name}"
        assert np.array_equal(ti.argmax(1).numpy(), orc.argreduce(True, ai, 1)), f"i32 argmax(1) {name}"
        want = orc.reduce(orc.SUM, a, [0, 1, 2, 3], acc=orc.ACC_F64)
        assert_close(t.sum([0, 1, 2, 3]).numpy(), want, F32_RTOL, F32_ATOL, f"sum(all) {name}")
    y = (rng.standard_normal((2048, 4096)) + rng.uniform(-5, 5, (2048, 1))).astype(np.float32)
    g, b = rng.normal(1, 0.1, 4096).astype(np.float32), rng.normal(0, 0.1, 4096).astype(np.float32)
    tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
    for name, ops in (("rev_rows", (("slice", (R, F)),)), ("rev_cols", (("slice", (F, R)),)), ("back2_cols", (("slice", (F, R2)),))):
        t, a = upload(hpt, y, ops, dev=dev)
        ns = [a.shape[1]]
        gg, bb = (g, b) if a.shape[1] == 4096 else (g[:2048], b[:2048])
        tgg = tg if a.shape[1] == 4096 else hpt.Tensor.from_numpy(gg).to_hip(dev)
        tbb = tb if a.shape[1] == 4096 else hpt.Tensor.from_numpy(bb).to_hip(dev)
        rows = slice(0, 2048, 13)
        want = orc.layernorm(np.ascontiguousarray(a[rows]), 1, gg, bb, 1e-5, acc=orc.ACC_F64)
        assert_close(t.layernorm(ns, tgg, tbb, 1e-5).numpy()[rows], want, F32_RTOL, 4 * F32_ATOL, f"layernorm {name}")
        want = orc.softmax(np.ascontiguousarray(a[rows]), 1, log=True, acc=orc.ACC_F64)
        assert_close(t.log_softmax(1).numpy()[rows], want, F32_RTOL, 2 * F32_ATOL, f"log_softmax {name}")
