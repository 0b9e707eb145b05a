"""GPU parity of the axis reductions against the CPU oracle, through the C ABI.

Mirrors the reference's reduce tests (hpt-tests/src/hpt/cpu/reduce.rs:63-650,
hpt-tests/src/hpt/cuda/reduce.rs:17-206, 1421-1612): random shapes, every axis
subset, keep_dims, the four layouts (contiguous / permuted / sliced / stepped),
integer inputs compared exactly, arg-reductions with ties.
"""
import itertools

import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol, layouts_for, upload

pytestmark = pytest.mark.gpu


def axis_subsets(nd):
    for r in range(1, nd + 1):
        for c in itertools.combinations(range(nd), r):
            yield list(c)


def test_sum_f32_random_shapes_all_axis_subsets_all_layouts(hpt, orc, dev):
    rng = np.random.default_rng(100)
    for case in range(24):
        nd = int(rng.integers(1, 4))
        shape = [int(rng.integers(1, 33)) for _ in range(nd)]
        base = rng.standard_normal(shape).astype(np.float32)
        for lname, ops in layouts_for(shape, rng):
            t, a = upload(hpt, base, ops, dev=dev)
            if a.size == 0:
                continue
            for axes in axis_subsets(a.ndim):
                for keep in (False, True):
                    got = t.sum(axes, keep).numpy()
                    want = orc.reduce(orc.SUM, a, axes, keep, acc=orc.ACC_F64)
                    assert_close(got, want, F32_RTOL, F32_ATOL, f"sum {shape} {lname} axes={axes} keep={keep}")


@pytest.mark.parametrize("op", ["sum", "prod", "max", "min", "mean", "nansum", "nanprod", "reducel1",
                                "reducel2", "reducel3", "sum_square", "logsumexp"])
def test_float_ops_f32_f64(hpt, orc, dev, op):
    rng = np.random.default_rng(101)
    code = getattr(orc, op.upper())
    for npdt in (np.float32, np.float64):
        for shape in ([2, 5, 10], [7, 33], [129], [3, 4, 5, 6]):
            base = (rng.standard_normal(shape) * (0.5 if op in ("prod", "nanprod") else 1.0) +
                    (1.0 if op in ("prod", "nanprod") else 0.0)).astype(npdt)
            if op.startswith("nan"):
                base.reshape(-1)[::7] = np.nan
            for lname, ops in layouts_for(shape, rng):
                t, a = upload(hpt, base, ops, dev=dev)
                for axes in ([0], [a.ndim - 1], list(range(a.ndim))):
                    got = getattr(t, op)(axes).numpy()
                    want = orc.reduce(code, a, axes, acc=orc.ACC_F64)
                    if op in ("max", "min"):
                        assert np.array_equal(got, want), f"{op} {shape} {lname} {axes}"
                    else:
                        assert_close(got, want, F32_RTOL, F32_ATOL, f"{op} {npdt.__name__} {shape} {lname} {axes}")


INT_DTYPES = [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64]


@pytest.mark.parametrize("npdt", INT_DTYPES)
def test_integer_ops_bit_exact(hpt, orc, dev, npdt):
    """Integer sums/products wrap (hpt-types/src/scalars/impls.rs:31-48): bit-exact, any layout."""
    rng = np.random.default_rng(102)
    info = np.iinfo(npdt)
    lo, hi = max(info.min, -1000), min(info.max, 1000)
    for shape in ([6, 40, 9], [300, 17], [5000]):
        base = rng.integers(lo, hi + 1, shape).astype(npdt)
        for lname, ops in layouts_for(shape, rng):
            t, a = upload(hpt, base, ops, dev=dev)
            for axes in ([0], [a.ndim - 1], list(range(a.ndim))):
                for op in ("sum", "prod", "max", "min", "reducel1", "sum_square"):
                    got = getattr(t, op)(axes).numpy()
                    want = orc.reduce(getattr(orc, op.upper()), a, axes)
                    assert got.dtype == want.dtype
                    assert np.array_equal(got, want), f"{op} {npdt.__name__} {shape} {lname} {axes}"
                # and the closed form: numpy's wrap-around sum in the same dtype
                assert np.array_equal(t.sum(axes).numpy().reshape(-1),
                                      np.asarray(a.sum(axis=tuple(axes), dtype=npdt)).reshape(-1))
                # mean of integers is computed in FloatBinaryType<T>
                gm = t.mean(axes).numpy()
                wm = orc.reduce(orc.MEAN, a, axes, acc=orc.ACC_F64)
                assert gm.dtype == wm.dtype
                tol = 1e-3 if gm.dtype == np.float16 else 1e-5
                assert_close(gm, wm, tol, tol, f"mean {npdt.__name__} {shape} {lname} {axes}")


def test_bool_and_all_any(hpt, orc, dev):
    rng = np.random.default_rng(103)
    base = rng.random((9, 31, 5)) < 0.9
    for lname, ops in layouts_for(list(base.shape), rng):
        t, a = upload(hpt, base, ops, dev=dev)
        for axes in ([0], [1], [2], [0, 1, 2]):
            for op in ("sum", "prod", "max", "min", "all", "any"):
                got = getattr(t, op)(axes).numpy()
                want = orc.reduce(getattr(orc, op.upper()), a, axes)
                assert np.array_equal(got, want), f"{op} bool {lname} {axes}"
    f = rng.standard_normal((17, 65)).astype(np.float32)
    f[f < -1.5] = 0.0
    t, a = upload(hpt, f, dev=dev)
    assert np.array_equal(t.all([1]).numpy(), (a != 0).all(1))
    assert np.array_equal(t.any([0]).numpy(), (a != 0).any(0))


@pytest.mark.parametrize("npdt", [np.int32, np.int64, np.float32, np.float64, np.int8, np.uint16, np.float16])
def test_argmax_argmin_ties_resolve_to_lowest_index(hpt, orc, dev, npdt):
    rng = np.random.default_rng(104)
    for shape in ([7, 128, 33], [64, 300], [1000], [4, 5, 6, 3]):
        # few distinct values => many ties
        base = rng.integers(-3, 4, shape).astype(npdt)
        for lname, ops in layouts_for(shape, rng):
            t, a = upload(hpt, base, ops, dev=dev)
            for axis in range(a.ndim):
                for keep in (False, True):
                    gmax = t.argmax(axis, keep).numpy()
                    gmin = t.argmin(axis, keep).numpy()
                    assert gmax.dtype == np.int64
                    assert np.array_equal(gmax, orc.argreduce(True, a, axis, keep)), f"argmax {shape} {lname} {axis}"
                    assert np.array_equal(gmin, orc.argreduce(False, a, axis, keep)), f"argmin {shape} {lname} {axis}"
                    assert np.array_equal(gmax.reshape(-1), a.argmax(axis).reshape(-1))
                    assert np.array_equal(gmin.reshape(-1), a.argmin(axis).reshape(-1))


def test_argmax_docstring_kat_and_nan(hpt, dev):
    # hpt-traits/src/ops/reduce.rs:21-39
    t = hpt.Tensor.from_numpy(np.array([10.0, 3.0, 2.0], np.float32)).to_hip(dev)
    assert t.argmax(0).numpy().tolist() == [0]
    assert t.argmin(0).numpy().tolist() == [2]
    # NaN never wins (strict compares): argreduce_kernels.rs:13-21
    t = hpt.Tensor.from_numpy(np.array([[np.nan, 1.0, 5.0, 5.0], [np.nan, np.nan, -np.inf, -np.inf]], np.float32)).to_hip(dev)
    assert t.argmax(1).numpy().tolist() == [2, 0]
    assert t.argmin(1).numpy().tolist() == [1, 2]


def test_docstring_kats(hpt, dev):
    # hpt-traits/src/ops/reduce.rs:58-62, 146-149, 166-168, 294-297, 328-331, 347-350
    a = hpt.Tensor.from_numpy(np.array([[1.0, 2.0], [3.0, 4.0]], np.float32)).to_hip(dev)
    assert a.sum([0, 1]).numpy().tolist() == [10.0]
    assert a.sum([0, 1], True).numpy().tolist() == [[10.0]]
    assert a.mean([0, 1]).numpy().tolist() == [2.5]
    assert a.sum_square([0, 1]).numpy().tolist() == [30.0]
    assert a.reducel1([0, 1]).numpy().tolist() == [10.0]
    assert a.prod([0, 1]).numpy().tolist() == [24.0]
    c = hpt.Tensor.from_numpy(np.array([[1.0, 2.0], [2.0, 3.0]], np.float32)).to_hip(dev)
    assert abs(c.reducel2([0, 1], True).numpy()[0, 0] - 4.2426405) < 1e-5   # "sqrt(1+4+4+9) ~ 4.24"
    assert abs(c.reducel3([0, 1], True).numpy()[0, 0] - 3.5303483) < 1e-5   # "[[3.5303]]"
    assert abs(a.logsumexp([0, 1]).numpy()[0] - 4.4401898) < 1e-5
    assert a.max([0]).numpy().tolist() == [3.0, 4.0]
    assert a.min([1]).numpy().tolist() == [1.0, 3.0]


@pytest.mark.parametrize("name", ["f16", "bf16"])
def test_half_types_f32_accumulate(hpt, orc, dev, name):
    rng = np.random.default_rng(105)
    for shape in ([33, 1000], [64, 8, 24], [4096]):
        x = rng.standard_normal(shape).astype(np.float32) * 2
        if name == "f16":
            base, dt, odt, bits = x.astype(np.float16), None, None, 11
            tof = lambda v: v.astype(np.float32)
        else:
            base, dt, odt, bits = hpt.f32_to_bf16_bits(x), hpt.bf16, orc.BF16, 8
            tof = hpt.bf16_bits_to_f32
        for lname, ops in layouts_for(shape, rng):
            t, a = upload(hpt, base, ops, dtype=dt, dev=dev)
            for axes in ([0], [a.ndim - 1], list(range(a.ndim))):
                for op in ("sum", "mean", "max", "min", "sum_square", "reducel2"):
                    got = tof(getattr(t, op)(axes).numpy())
                    want = tof(orc.reduce(getattr(orc, op.upper()), a, axes, acc=orc.ACC_F32, dtype=odt))
                    if op in ("max", "min"):
                        assert np.array_equal(got, want)
                    else:
                        assert_close(got, want, HALF_RTOL, half_atol(want, bits), f"{op} {name} {shape} {lname} {axes}")


def test_multi_stage_and_large_shapes(hpt, orc, dev):
    """Shapes that take the several-workgroups-per-output paths (row and column) and run twice
    to check that the arrival counters were reset."""
    rng = np.random.default_rng(106)
    cases = [((3, 1 << 20), [1]), ((1 << 21,), [0]), ((1 << 16, 40), [0]), ((2, 70000, 3), [1]),
             ((64, 128, 56, 56), [1]), ((700, 3, 900), [0, 2])]
    for shape, axes in cases:
        base = rng.standard_normal(shape).astype(np.float32)
        t, a = upload(hpt, base, dev=dev)
        want = orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F64)
        for rep in range(2):
            got = t.sum(axes).numpy()
            assert_close(got, want, F32_RTOL, F32_ATOL, f"sum {shape} axes={axes} rep={rep}")
        gi = t.argmax(axes[0]).numpy() if len(axes) == 1 else None
        if gi is not None:
            assert np.array_equal(gi, orc.argreduce(True, a, axes[0]))
        ib = rng.integers(-1000, 1001, shape).astype(np.int32)
        ti, ai = upload(hpt, ib, dev=dev)
        assert np.array_equal(ti.sum(axes).numpy(), orc.reduce(orc.SUM, ai, axes))
        # run-to-run determinism of the multi-stage float path
        assert np.array_equal(t.sum(axes).numpy().view(np.uint32), t.sum(axes).numpy().view(np.uint32))


def test_narrow_inner_dim_flat_walk(hpt, orc, dev):
    """Contiguous [N, k] slabs with k not a whole number of 128-bit vectors (3, 33, 257 columns),
    reduced over N: the slab is walked as a flat array of aligned vectors. Sizes leave a partial
    last period; one case has an outer kept dim; ties and all-equal columns check the index rule."""
    rng = np.random.default_rng(116)
    assert "col-flat " in hpt.reduce_plan(hpt.Tensor.empty([700001, 3], hpt.f32, dev), hpt.SUM, [0])
    assert "col-flat-wide" in hpt.reduce_plan(hpt.Tensor.empty([2051, 4097], hpt.f32, dev), hpt.SUM, [0])
    for shape, axis, npdt in (((700001, 3), 0, np.float32), ((70003, 33), 0, np.float32), ((4, 500000, 5), 1, np.float32),
                              ((140001, 33), 0, np.float16), ((20001, 257), 0, np.float16), ((1100003, 1, 3), 0, np.float64),
                              ((700, 2048, 3), 1, np.float32), ((900, 1031, 5), 1, np.float16),   # many small slabs
                              ((257, 4097, 23), 1, np.float16), ((31, 70001, 3), 1, np.float32),    # slabs off 16-byte boundaries
                              ((2100001, 3), 0, np.int32), ((3000001, 3), 0, np.uint8), ((600011, 7), 0, np.int16),
                              # rows wider than a workgroup: the period spans several workgroups ("flat-wide")
                              ((2051, 4097), 0, np.float32), ((1031, 5003), 0, np.float16), ((2, 1028, 2051), 1, np.float32),
                              ((1101, 8191), 0, np.uint8), ((1501, 2051), 0, np.int32), ((301, 4099), 0, np.float64)):
        if np.issubdtype(npdt, np.floating):
            base = rng.standard_normal(shape).astype(npdt)
        else:
            base = rng.integers(0, 100, shape).astype(npdt)   # many ties
        t, a = upload(hpt, base, dev=dev)
        tag = f"{np.dtype(npdt).name} {shape} axis={axis}"
        gi, wi = t.argmax(axis).numpy(), orc.argreduce(True, a, axis)
        assert np.array_equal(gi, wi), tag
        assert np.array_equal(t.argmin(axis).numpy(), orc.argreduce(False, a, axis)), tag
        assert np.array_equal(t.max([axis]).numpy(), a.max(axis)), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F32)
            assert_close(t.sum([axis]).numpy().astype(np.float32), want.astype(np.float32), HALF_RTOL, half_atol(want.astype(np.float32), 11), tag)
        elif np.issubdtype(npdt, np.floating):
            want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64)
            assert_close(t.sum([axis]).numpy(), want, F32_RTOL, F32_ATOL if npdt == np.float32 else 1e-9, tag)
            assert_close(t.mean([axis]).numpy(), a.astype(np.float64).mean(axis), F32_RTOL, F32_ATOL, tag)
        else:
            assert np.array_equal(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis])), tag
    # a constant slab: every index ties, the lowest wins on every path
    c = hpt.Tensor.full(2.5, [900001, 3], hpt.f32, dev)
    assert c.argmax(0).numpy().tolist() == [0, 0, 0] and c.argmin(0).numpy().tolist() == [0, 0, 0]
    assert c.sum([0]).numpy().tolist() == [900001 * 2.5] * 3


def test_short_rows_staged_through_lds(hpt, orc, dev):
    """Contiguous [N, k] with short rows reduced over k: 16 KiB tiles of whole rows are brought in
    with aligned vectors and reduced out of LDS. Row lengths that are / are not whole vectors, a
    partial last tile and a partial last vector; ties for the index rule."""
    rng = np.random.default_rng(117)
    assert hpt.reduce_plan(hpt.Tensor.empty([1400001, 3], hpt.f32, dev), hpt.SUM, [1]).startswith("row-tile")
    for shape, npdt in (((1400001, 3), np.float32), ((200003, 33), np.float16), ((50001, 100), np.int32),
                        ((30001, 255), np.float32), ((300001, 17), np.uint8), ((70001, 9), np.float64),
                        ((1100001, 8), np.float16), ((40, 30001, 5), np.float32), ((9001, 512), np.int16)):
        if np.issubdtype(npdt, np.floating):
            base = rng.standard_normal(shape).astype(npdt)
        else:
            base = rng.integers(0, 50, shape).astype(npdt)   # many ties
        t, a = upload(hpt, base, dev=dev)
        ax = len(shape) - 1
        tag = f"{np.dtype(npdt).name} {shape}"
        assert np.array_equal(t.argmax(ax).numpy(), orc.argreduce(True, a, ax)), tag
        assert np.array_equal(t.argmin(ax).numpy(), orc.argreduce(False, a, ax)), tag
        assert np.array_equal(t.min([ax]).numpy(), a.min(ax)), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [ax], acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum([ax]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag)
        elif np.issubdtype(npdt, np.floating):
            assert_close(t.sum([ax]).numpy(), orc.reduce(orc.SUM, a, [ax], acc=orc.ACC_F64), F32_RTOL, F32_ATOL, tag)
            assert_close(t.reducel2([ax]).numpy(), np.sqrt((a.astype(np.float64) ** 2).sum(ax)), F32_RTOL, F32_ATOL, tag)
        else:
            assert np.array_equal(t.sum([ax]).numpy(), orc.reduce(orc.SUM, a, [ax])), tag
            assert np.array_equal(t.prod([ax]).numpy(), orc.reduce(orc.PROD, a, [ax])), tag
    b = rng.integers(0, 2, (900001, 7)).astype(np.bool_)
    tb, ab = upload(hpt, b, dev=dev)
    assert np.array_equal(tb.all([1]).numpy(), ab.all(1)) and np.array_equal(tb.any([1]).numpy(), ab.any(1))
    # accumulate into an existing output
    x = rng.standard_normal((1200000, 3)).astype(np.float32)
    tx, ax_ = upload(hpt, x, dev=dev)
    out = hpt.Tensor.full(2.0, [1200000], hpt.f32, dev)
    tx.sum_([1], False, False, out)
    assert_close(out.numpy(), ax_.astype(np.float64).sum(1) + 2.0, F32_RTOL, F32_ATOL, "sum_ accumulate, short rows")


def test_special_values_on_the_large_shape_kernels(hpt, orc, dev):
    """NaN, +-inf on the kernels that only large shapes reach (LDS row tiles, the flat column walk, its
    wide form, the flat (outer, inner) row walk): max / min skip NaN, a NaN never wins an arg
    reduction (all-NaN -> index 0), nansum skips it, sum propagates it."""
    rng = np.random.default_rng(118)
    for shape, axes, plan in (((500001, 5), [1], "row-tile"), ((500001, 5), [0], "col-flat "), ((2051, 4097), [0], "col-flat-wide"),
                              ((40, 24, 56, 56), [0, 2, 3], "row-general"), ((8192, 1024), [0], "col vec=4")):
        x = rng.standard_normal(shape).astype(np.float32)
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, flat.size // 50)] = np.nan
        flat[rng.integers(0, flat.size, flat.size // 200)] = np.inf
        flat[rng.integers(0, flat.size, flat.size // 200)] = -np.inf
        if len(axes) == 1:       # one output with nothing but NaN
            idx = [0] * len(shape)
            idx[axes[0]] = slice(None)
            x[tuple(idx)] = np.nan
        t, a = upload(hpt, x, dev=dev)
        assert hpt.reduce_plan(t, hpt.SUM, axes).startswith(plan), hpt.reduce_plan(t, hpt.SUM, axes)
        tag = f"{shape} {axes}"
        assert np.array_equal(t.max(axes).numpy(), orc.reduce(orc.MAX, a, axes)), tag
        assert np.array_equal(t.min(axes).numpy(), orc.reduce(orc.MIN, a, axes)), tag
        with np.errstate(invalid="ignore"):
            want = orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F64)
            got = t.sum(axes).numpy()
            assert np.array_equal(np.isnan(got), np.isnan(want)), tag
            fin = np.isfinite(want)
            assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)]), tag
            assert_close(got[fin], want[fin], F32_RTOL, 1e-5, "sum " + tag)
            wn = orc.reduce(orc.NANSUM, a, axes, acc=orc.ACC_F64)
            gn = t.nansum(axes).numpy()
            assert np.array_equal(np.isnan(gn), np.isnan(wn)) and np.array_equal(np.isinf(gn), np.isinf(wn)), tag
            ok = np.isfinite(wn)
            assert_close(gn[ok], wn[ok], F32_RTOL, 1e-5, "nansum " + tag)
        if len(axes) == 1:
            assert np.array_equal(t.argmax(axes[0]).numpy(), orc.argreduce(True, a, axes[0])), tag
            assert np.array_equal(t.argmin(axes[0]).numpy(), orc.argreduce(False, a, axes[0])), tag


def test_long_rows_off_the_vector_grid(hpt, orc, dev):
    """Long contiguous rows whose length, pitch or start is not a whole number of 128-bit vectors (the
    sum of a whole array of odd length, a slice that drops the first element): the first and last
    elements of each row are folded one by one, the rest as aligned vectors. Ties check the index rule
    across the peeled ends; a row shorter than its own peel and the two-stage form are included."""
    rng = np.random.default_rng(121)
    assert hpt.reduce_plan(hpt.Tensor.empty([3000001], hpt.u8, dev), hpt.SUM, [0]).startswith("row-ragged")
    for shape, view, npdt in (((3000001,), (), np.uint8), ((1000003,), (("slice", ((3, 1000000, 1),)),), np.float32),
                              ((2000001,), (("slice", ((1, 2000001, 1),)),), np.int16), ((7, 300001), (), np.float16),
                              ((300, 5001), (), np.float32), ((33, 40007), (("slice", ((0, 33, 1), (5, 40000, 1))),), np.int32),
                              ((5001, 1100), (("slice", ((0, 5001, 1), (1, 1040, 1))),), np.uint8), ((4000003,), (), np.bool_), ((12, 100003), (), np.float64)):
        if npdt == np.bool_:
            base = rng.integers(0, 2, shape).astype(npdt)
        elif np.issubdtype(npdt, np.floating):
            base = rng.standard_normal(shape).astype(npdt)
        else:
            base = rng.integers(0, 60, shape).astype(npdt)   # many ties
        t, a = upload(hpt, base, view, dev=dev)
        ax = len(shape) - 1
        tag = f"{np.dtype(npdt).name} {shape} {view}"
        assert hpt.reduce_plan(t, hpt.SUM, [ax]).startswith("row-ragged"), hpt.reduce_plan(t, hpt.SUM, [ax])
        assert np.array_equal(t.argmax(ax).numpy(), orc.argreduce(True, a, ax)), tag
        assert np.array_equal(t.argmin(ax).numpy(), orc.argreduce(False, a, ax)), tag
        if npdt == np.bool_:
            assert np.array_equal(t.all([ax]).numpy().reshape(-1), a.all(ax).reshape(-1)) and np.array_equal(t.any([ax]).numpy().reshape(-1), a.any(ax).reshape(-1)), tag
            continue
        assert np.array_equal(t.max([ax]).numpy(), orc.reduce(orc.MAX, a, [ax])), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [ax], acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum([ax]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag)
        elif np.issubdtype(npdt, np.floating):
            assert_close(t.sum([ax]).numpy(), orc.reduce(orc.SUM, a, [ax], acc=orc.ACC_F64), F32_RTOL, 2e-5, tag)
        else:
            assert np.array_equal(t.sum([ax]).numpy(), orc.reduce(orc.SUM, a, [ax])), tag
    # the extreme value sits in a peeled end: first element, last element
    for pos in (0, 1000002):
        x = np.zeros(1000003, np.float32)
        x[pos] = 7.0
        t, a = upload(hpt, x, dev=dev)
        assert int(t.argmax(0).numpy()) == pos and float(t.max([0]).numpy()) == 7.0 and float(t.sum([0]).numpy()) == 7.0


def test_short_runs_off_the_vector_grid(hpt, orc, dev):
    """Contiguous runs that are not whole, aligned vectors and too short to peel (the batch-norm sums of
    [N, C, 7, 7]: runs of 49; rows of 103 at an odd pitch): unaligned 128-bit loads, the last vector of
    a run taken from its end backwards with the shared elements skipped. Runs barely longer than a
    vector, exactly one vector, and ties for the index rule."""
    rng = np.random.default_rng(122)
    for shape, view, axes, npdt in (((64, 96, 7, 7), (), [0, 2, 3], np.float32), ((64, 96, 7, 7), (), [0, 2, 3], np.float16),
                                    ((40, 30, 14, 14), (), [0, 2, 3], np.float16), ((33, 17, 5, 3), (), [0, 2, 3], np.int32),
                                    ((16, 8, 57, 57), (), [0, 2, 3], np.uint8), ((300, 103), (), [1], np.float32),
                                    ((300, 120), (("slice", ((0, 300, 1), (3, 106, 1))),), [1], np.int16),
                                    ((5000, 17), (("slice", ((0, 5000, 1), (1, 17, 1))),), [1], np.uint8),
                                    ((9, 4, 6, 9), (), [1, 3], np.float32), ((12, 5, 3, 2, 11), (), [0, 2, 4], np.float64),
                                    ((50, 9), (), [1], np.float16), ((50, 8), (("slice", ((0, 50, 1), (0, 8, 1))),), [1], np.float16)):
        if np.issubdtype(npdt, np.floating):
            base = rng.standard_normal(shape).astype(npdt)
        else:
            base = rng.integers(0, 40, shape).astype(npdt)   # many ties
        t, a = upload(hpt, base, view, dev=dev)
        tag = f"{np.dtype(npdt).name} {shape} {view} {axes}"
        plan = hpt.reduce_plan(t, hpt.SUM, axes)
        if (shape, view) != ((50, 8), (("slice", ((0, 50, 1), (0, 8, 1))),)):
            assert "-unaligned" in plan and plan.startswith("row"), plan
        assert np.array_equal(t.max(axes).numpy(), orc.reduce(orc.MAX, a, axes)), tag
        assert np.array_equal(t.min(axes).numpy(), orc.reduce(orc.MIN, a, axes)), tag
        if len(axes) == 1:
            assert np.array_equal(t.argmax(axes[0]).numpy(), orc.argreduce(True, a, axes[0])), tag
            assert np.array_equal(t.argmin(axes[0]).numpy(), orc.argreduce(False, a, axes[0])), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum(axes).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag)
        elif np.issubdtype(npdt, np.floating):
            assert_close(t.sum(axes).numpy(), orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F64), F32_RTOL, 2e-5, tag)
            assert_close(t.mean(axes).numpy(), a.astype(np.float64).mean(tuple(axes)), F32_RTOL, F32_ATOL, tag)
        else:
            assert np.array_equal(t.sum(axes).numpy(), orc.reduce(orc.SUM, a, axes)), tag
    # a view that ends on the buffer's last element: the last vector must not reach past it
    x = rng.integers(0, 9, (64, 3, 7, 7)).astype(np.int32)
    t, a = upload(hpt, x, dev=dev)
    assert np.array_equal(t.sum([0, 2, 3]).numpy(), orc.reduce(orc.SUM, a, [0, 2, 3]))


def test_small_groups_staged_through_lds(hpt, orc, dev):
    """Contiguous [outer, R, k] reduced over the short middle axis with small R * k ([N, 2, 3], [N, 3, 16],
    [N, 4, 12]): 16 KiB tiles of whole groups are brought into LDS with aligned vectors and one lane
    per output folds its R elements from there. Partial last tiles and vectors, ties for the index rule,
    NaN handling, the accumulate form."""
    rng = np.random.default_rng(123)
    assert "group-tile" in hpt.reduce_plan(hpt.Tensor.empty([700001, 2, 3], hpt.f32, dev), hpt.SUM, [1])
    for shape, ax, npdt in (((700001, 2, 3), 1, np.float32), ((300001, 3, 16), 1, np.float16), ((5, 70001, 4, 12), 2, np.float16),
                            ((150001, 7, 33), 1, np.uint8), ((40001, 50, 9), 1, np.int32), ((60001, 16, 8), 1, np.float64),
                            ((90001, 2, 255), 1, np.int16), ((3, 11, 20001, 16, 2), 3, np.float32)):
        if np.issubdtype(npdt, np.floating):
            base = rng.standard_normal(shape).astype(npdt)
        else:
            base = rng.integers(0, 40, shape).astype(npdt)   # many ties
        t, a = upload(hpt, base, dev=dev)
        tag = f"{np.dtype(npdt).name} {shape}"
        assert "group-tile" in hpt.reduce_plan(t, hpt.SUM, [ax]), hpt.reduce_plan(t, hpt.SUM, [ax])
        assert np.array_equal(t.argmax(ax).numpy(), orc.argreduce(True, a, ax)), tag
        assert np.array_equal(t.argmin(ax).numpy(), orc.argreduce(False, a, ax)), tag
        assert np.array_equal(t.max([ax]).numpy(), a.max(ax)), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [ax], acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum([ax]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag)
        elif np.issubdtype(npdt, np.floating):
            assert_close(t.sum([ax]).numpy(), orc.reduce(orc.SUM, a, [ax], acc=orc.ACC_F64), F32_RTOL, F32_ATOL, tag)
            assert_close(t.mean([ax]).numpy(), a.astype(np.float64).mean(ax), F32_RTOL, F32_ATOL, tag)
        else:
            assert np.array_equal(t.sum([ax]).numpy(), orc.reduce(orc.SUM, a, [ax])), tag
            assert np.array_equal(t.prod([ax]).numpy(), orc.reduce(orc.PROD, a, [ax])), tag
    # NaN / inf: max skips NaN, a NaN never wins an arg reduction, sum propagates, nansum skips
    x = rng.standard_normal((400001, 3, 4)).astype(np.float32)
    flat = x.reshape(-1)
    flat[rng.integers(0, flat.size, flat.size // 20)] = np.nan
    flat[rng.integers(0, flat.size, flat.size // 100)] = np.inf
    x[7] = np.nan
    t, a = upload(hpt, x, dev=dev)
    assert np.array_equal(t.max([1]).numpy(), orc.reduce(orc.MAX, a, [1]))
    assert np.array_equal(t.argmax(1).numpy(), orc.argreduce(True, a, 1))
    with np.errstate(invalid="ignore"):
        want = orc.reduce(orc.SUM, a, [1], acc=orc.ACC_F64)
        got = t.sum([1]).numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = np.isfinite(want)
        assert_close(got[ok], want[ok], F32_RTOL, 1e-5, "sum with special values")
        wn = orc.reduce(orc.NANSUM, a, [1], acc=orc.ACC_F64)
        gn = t.nansum([1]).numpy()
        ok = np.isfinite(wn)
        assert np.array_equal(np.isinf(gn), np.isinf(wn))
        assert_close(gn[ok], wn[ok], F32_RTOL, 1e-5, "nansum with special values")
    # accumulate into an existing output
    y = rng.standard_normal((500000, 2, 3)).astype(np.float32)
    ty, ay = upload(hpt, y, dev=dev)
    out = hpt.Tensor.full(2.0, [500000, 3], hpt.f32, dev)
    ty.sum_([1], False, False, out)
    assert_close(out.numpy(), ay.astype(np.float64).sum(1) + 2.0, F32_RTOL, F32_ATOL, "sum_ accumulate, small groups")
    b = rng.integers(0, 2, (900001, 3, 5)).astype(np.bool_)
    tb, ab = upload(hpt, b, dev=dev)
    assert np.array_equal(tb.all([1]).numpy(), ab.all(1)) and np.array_equal(tb.any([1]).numpy(), ab.any(1))


def test_reduction_over_the_last_axis_of_a_permuted_view(hpt, orc, dev):
    """x.permute(2, 1, 0).sum(2): the first kept dim is the contiguous one. The lanes run along it and
    the outputs are scattered (one launch, and the two-stage form with its second-stage remap)."""
    rng = np.random.default_rng(119)
    for shape, npdt in (((96, 40, 72), np.float32), ((2000, 70, 36), np.float32), ((3000, 9, 64), np.int32), ((700, 33, 24), np.float16)):
        base = (rng.standard_normal(shape) * 3).astype(npdt) if np.issubdtype(npdt, np.floating) else rng.integers(-9, 9, shape).astype(npdt)
        t, a = upload(hpt, base, (("permute", (2, 1, 0)),), dev=dev)
        assert hpt.reduce_plan(t, hpt.SUM, [2]).startswith("col-swapped"), hpt.reduce_plan(t, hpt.SUM, [2])
        tag = f"{np.dtype(npdt).name} {shape}"
        assert np.array_equal(t.argmax(2).numpy(), orc.argreduce(True, a, 2)), tag
        assert np.array_equal(t.max([2]).numpy(), a.max(2)), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [2], acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum([2]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag)
        elif npdt == np.float32:
            want = orc.reduce(orc.SUM, a, [2], acc=orc.ACC_F64)
            assert_close(t.sum([2], True).numpy(), want.reshape(want.shape + (1,)), F32_RTOL, F32_ATOL, tag)
            out = hpt.Tensor.full(1.0, list(want.shape), hpt.f32, dev)
            t.sum_([2], False, False, out)
            assert_close(out.numpy(), want + 1.0, F32_RTOL, F32_ATOL, "accumulate " + tag)
        else:
            assert np.array_equal(t.sum([2]).numpy(), orc.reduce(orc.SUM, a, [2])), tag


def test_column_reduction_over_rows_that_are_not_whole_vectors(hpt, orc, dev):
    """Reductions over a long axis whose inner rows are odd-length or start off 16-byte boundaries:
    a lane still takes a vector's worth of neighbouring outputs (unaligned 128-bit loads); the last
    lane of a row, with fewer, loads them one by one."""
    rng = np.random.default_rng(120)
    cases = [((600, 259), (), 0, np.float32), ((5000, 301), (), 0, np.float16), ((3, 300, 1001), (), 1, np.float32),
             ((601, 270), (("slice", ((1, 601, 1), (3, 264, 1))),), 0, np.float16), ((700, 263), (), 0, np.int32),
             ((400, 257), (), 0, np.float64), ((2, 300, 513), (("permute", (1, 0, 2)),), 0, np.float32)]
    for shape, ops, axis, npdt in cases:
        base = (rng.standard_normal(shape) * 3).astype(npdt) if np.issubdtype(npdt, np.floating) else rng.integers(-9, 9, shape).astype(npdt)
        t, a = upload(hpt, base, ops, dev=dev)
        plan = hpt.reduce_plan(t, hpt.SUM, [axis])
        assert "unaligned" in plan or "swapped" in plan, plan
        tag = f"{np.dtype(npdt).name} {shape} {ops} axis={axis}"
        assert np.array_equal(t.argmax(axis).numpy(), orc.argreduce(True, a, axis)), tag
        assert np.array_equal(t.min([axis]).numpy(), a.min(axis)), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum([axis]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag)
        elif np.issubdtype(npdt, np.floating):
            want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64)
            assert_close(t.sum([axis]).numpy(), want, F32_RTOL, F32_ATOL, tag)
            out = hpt.Tensor.full(1.0, list(want.shape), t.dtype, dev)
            t.sum_([axis], False, False, out)
            assert_close(out.numpy(), want + 1.0, F32_RTOL, F32_ATOL, "accumulate " + tag)
        else:
            assert np.array_equal(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis])), tag


def test_sum_inplace_out_and_accumulate(hpt, orc, dev):
    """sum_ with init_out: true overwrites, false adds to what `out` holds (reduce.rs:84-92)."""
    rng = np.random.default_rng(107)
    base = rng.standard_normal((40, 50)).astype(np.float32)
    t, a = upload(hpt, base, dev=dev)
    out = hpt.Tensor.from_numpy(np.full((40,), 5.0, np.float32)).to_hip(dev)
    r = t.sum_([1], False, True, out)
    assert_close(r.numpy(), a.astype(np.float64).sum(1), F32_RTOL, F32_ATOL, "sum_ init_out")
    assert_close(out.numpy(), a.astype(np.float64).sum(1), F32_RTOL, F32_ATOL, "sum_ writes into out")
    out2 = hpt.Tensor.from_numpy(np.full((40,), 5.0, np.float32)).to_hip(dev)
    t.sum_([1], False, False, out2)
    assert_close(out2.numpy(), a.astype(np.float64).sum(1) + 5.0, F32_RTOL, F32_ATOL, "sum_ accumulate")
    with pytest.raises(hpt.ShapeError):
        t.sum_([1], False, True, hpt.Tensor.empty([41], hpt.f32, dev))


def test_empty_and_degenerate(hpt, orc, dev):
    z = hpt.Tensor.from_numpy(np.zeros((4, 0, 3), np.float32)).to_hip(dev)
    assert z.sum([1]).numpy().tolist() == np.zeros((4, 3)).tolist()          # reduced dim empty -> identity
    assert z.prod([1]).numpy().tolist() == np.ones((4, 3)).tolist()
    assert np.all(np.isneginf(z.max([1]).numpy()))
    assert z.sum([0]).numpy().shape == (0, 3)                                 # no outputs
    one = hpt.Tensor.from_numpy(np.arange(6, dtype=np.float32).reshape(1, 6, 1)).to_hip(dev)
    assert one.sum([0, 2]).numpy().tolist() == [0, 1, 2, 3, 4, 5]              # only size-1 axes reduced
    assert one.argmax(0).numpy().tolist() == [[0]] * 6
    with pytest.raises(hpt.ShapeError, match=r"Dimension out of range: expected in 0\.\.3, got 3"):
        one.sum([3])
    with pytest.raises(hpt.ParamError, match="Axis 1 is duplicated"):
        one.sum([1, 1])


XCD_ROW_CASES = [
    # neighbouring outputs whose runs lie back to back (general row kernel, row blocks numbered per XCD):
    # output counts that are and are not multiples of eight, with and without a split of the reduced range
    ([37, 67, 80], [0, 2]), ([64, 1000, 20], [0, 2]), ([9, 130, 7, 12], [0, 3]), ([4096, 70, 24], [0, 2]),
    ([3, 200, 5, 16], [0, 2]), ([1024, 65, 80], [0, 2]), ([16, 513, 33], [0, 2]),
]


@pytest.mark.parametrize("case", XCD_ROW_CASES, ids=[f"{c[0]} over {c[1]}" for c in XCD_ROW_CASES])
def test_neighbouring_outputs_with_runs_back_to_back(hpt, orc, dev, case):
    shape, axes = case
    rng = np.random.default_rng(77)
    xi = rng.integers(-1000, 1001, shape).astype(np.int32)
    ti = hpt.Tensor.from_numpy(xi).to_hip(dev)
    assert np.array_equal(ti.sum(axes).numpy(), xi.sum(tuple(axes), dtype=np.int32)), "i32 sum"
    assert np.array_equal(ti.max(axes).numpy(), xi.max(tuple(axes))), "i32 max"
    x = rng.standard_normal(shape).astype(np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    assert_close(t.sum(axes).numpy(), orc.reduce(orc.SUM, x, axes, acc=orc.ACC_EXACT), F32_RTOL, F32_ATOL, "f32 sum")
    assert_close(t.mean(axes).numpy(), orc.reduce(orc.MEAN, x, axes, acc=orc.ACC_EXACT), F32_RTOL, F32_ATOL, "f32 mean")
    h = x.astype(np.float16)
    th = hpt.Tensor.from_numpy(h).to_hip(dev)
    assert np.array_equal(th.max(axes).numpy(), h.max(tuple(axes))), "f16 max"


FEW_PARTIAL_CASES = [
    # (shape, axes, words of the plan): few outputs of 2 ... 16 partials each, folded by one thread per output
    ([64, 128, 784], [0, 2], "split=4(4x1)"), ([40, 300000], [1], "split=12(1x12)"), ([200, 100000], [1], "split=2(1x2)"),
    ([130, 70001], [1], "split=3(1x3)"), ([96, 33, 4000], [1, 2], "split=5(1x5)"),
]


@pytest.mark.parametrize("case", FEW_PARTIAL_CASES, ids=[f"{'x'.join(map(str, c[0]))}-{c[2]}" for c in FEW_PARTIAL_CASES])
def test_few_outputs_of_few_partials_each(hpt, orc, dev, case):
    shape, axes, words = case
    rng = np.random.default_rng(131)
    base = rng.standard_normal(shape).astype(np.float32)
    # ties for the arg-reductions across the split: the maximum sits in the first and in the last partial's range
    idx_first = tuple(0 if i in axes else slice(None) for i in range(len(shape)))
    idx_last = tuple(shape[i] - 1 if i in axes else slice(None) for i in range(len(shape)))
    base[idx_first] = 9.0
    base[idx_last] = 9.0
    t, a = upload(hpt, base, dev=dev)
    assert words in hpt.reduce_plan(t, hpt.SUM, axes), hpt.reduce_plan(t, hpt.SUM, axes)
    assert_close(t.sum(axes).numpy(), orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"sum {shape}")
    assert_close(t.mean(axes).numpy(), orc.reduce(orc.MEAN, a, axes, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"mean {shape}")
    assert np.array_equal(t.max(axes).numpy(), a.max(tuple(axes)))
    assert np.array_equal(t.min(axes).numpy(), a.min(tuple(axes)))
    if len(axes) == 1:
        assert np.array_equal(t.argmax(axes[0]).numpy(), orc.argreduce(True, a, axes[0]))   # lowest index wins
        assert np.array_equal(t.argmin(axes[0]).numpy(), orc.argreduce(False, a, axes[0]))
    ib = rng.integers(-1000, 1001, shape).astype(np.int32)
    ti, ai = upload(hpt, ib, dev=dev)
    assert np.array_equal(ti.sum(axes).numpy(), orc.reduce(orc.SUM, ai, axes))
    hb = (rng.standard_normal(shape) * 0.5).astype(np.float16)
    th, ah = upload(hpt, hb, dev=dev)
    want = orc.reduce(orc.SUM, ah, axes, acc=orc.ACC_F32).astype(np.float32)
    assert_close(th.sum(axes).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), f"f16 sum {shape}")
    # accumulate into the output, and the same bits from run to run
    out = hpt.Tensor.from_numpy(np.ones(want.shape, np.float32)).to_hip(dev)
    t.sum_(axes, False, False, out)
    assert_close(out.numpy(), orc.reduce(orc.SUM, a, axes, acc=orc.ACC_F64) + 1, F32_RTOL, F32_ATOL, f"sum into out {shape}")
    assert np.array_equal(t.sum(axes).numpy().view(np.uint32), t.sum(axes).numpy().view(np.uint32))


INTERLEAVED_ROW_CASES = [  # (dtype, shape, axis): the middle axis of a contiguous [B, C, L], L a divisor of the 16-byte vector
    (np.float32, (600, 2048, 2), 1), (np.float32, (700, 1000, 4), 1), (np.float32, (8000, 100, 2), 1), (np.float32, (3, 300, 1000, 2), 2),
    (np.float32, (600, 8192, 2), 1), (np.float16, (900, 1000, 8), 1), (np.float16, (4000, 300, 4), 1), (np.float16, (800, 3000, 2), 1),
    (np.float64, (600, 1000, 2), 1), (np.int32, (700, 1000, 4), 1), (np.int64, (600, 1000, 2), 1), (np.int16, (900, 1000, 8), 1),
    (np.int8, (1200, 1000, 4), 1), (np.uint8, (300, 3000, 8), 1),
]


@pytest.mark.parametrize("npdt,shape,axis", INTERLEAVED_ROW_CASES, ids=lambda v: getattr(v, "__name__", str(v).replace(" ", "")))
def test_reduction_over_the_middle_axis_with_an_inner_dim_that_divides_the_vector(hpt, orc, dev, npdt, shape, axis):
    """The [C, L] slab runs as one row of C * L elements, a thread keeping L accumulators (one per place in the vector).
    Inner positions get offsets far apart so that an accumulator fed from the wrong place shows; ties for the
    arg-reductions sit at both ends of the axis (the lowest index wins)."""
    rng = np.random.default_rng(733)
    L, C = shape[-1], shape[axis]
    if np.issubdtype(npdt, np.floating):
        base = (rng.standard_normal(shape) + (np.arange(L) * 3.0 - 2.0)).astype(npdt)
    else:
        info = np.iinfo(npdt)
        lo, hi = max(info.min, -100), min(info.max, 100)
        base = (rng.integers(lo, hi + 1, shape) // 2 + (np.arange(L) % 3)).astype(npdt)
    first = tuple(0 if i == axis else slice(None) for i in range(len(shape)))
    last = tuple(C - 1 if i == axis else slice(None) for i in range(len(shape)))
    top = np.asarray(base.max() + 1, dtype=np.float64).astype(npdt)
    base[first] = top
    base[last] = top
    t, a = upload(hpt, base, dev=dev)
    assert hpt.reduce_plan(t, hpt.SUM, [axis]).startswith("row-interleaved"), hpt.reduce_plan(t, hpt.SUM, [axis])
    assert np.array_equal(t.max([axis]).numpy(), a.max(axis))
    assert np.array_equal(t.min([axis]).numpy(), a.min(axis))
    assert np.array_equal(t.argmax(axis).numpy(), orc.argreduce(True, a, axis))
    assert np.array_equal(t.argmin(axis).numpy(), orc.argreduce(False, a, axis))
    if npdt == np.float16:
        want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F32).astype(np.float32)
        assert_close(t.sum([axis]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), f"f16 sum {shape}")
    elif np.issubdtype(npdt, np.floating):
        rtol, atol = (F32_RTOL, F32_ATOL) if npdt == np.float32 else (1e-12, 1e-12)
        assert_close(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64), rtol, atol, f"sum {shape}")
        assert_close(t.mean([axis]).numpy(), orc.reduce(orc.MEAN, a, [axis], acc=orc.ACC_F64), rtol, atol, f"mean {shape}")
        out = hpt.Tensor.from_numpy(np.ones(t.sum([axis]).shape, npdt)).to_hip(dev)
        t.sum_([axis], False, False, out)
        assert_close(out.numpy(), orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64) + 1, rtol, atol, f"sum into out {shape}")
    else:
        assert np.array_equal(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis]))
        assert np.array_equal(t.prod([axis]).numpy(), orc.reduce(orc.PROD, a, [axis]))


MODULAR_ROW_CASES = [  # (dtype, shape, axis): the middle axis of a contiguous [B, C, L], L = 3, 5, 6, 7
    (np.float32, (600, 2000, 3), 1), (np.float32, (2000, 1001, 3), 1), (np.float32, (1500, 401, 5), 1), (np.float32, (800, 3000, 7), 1),
    (np.float32, (3, 400, 1000, 6), 2), (np.float32, (512, 20001, 3), 1), (np.float16, (900, 1000, 3), 1), (np.float16, (2000, 999, 5), 1),
    (np.float16, (600, 2047, 7), 1), (np.float64, (600, 1001, 3), 1), (np.float64, (700, 333, 5), 1), (np.int32, (700, 1001, 3), 1),
    (np.int64, (600, 1000, 7), 1), (np.int16, (900, 1001, 6), 1), (np.int8, (1200, 1501, 3), 1), (np.uint8, (600, 3001, 5), 1),
    # slabs just above the 2 KiB that the LDS group tiles take
    (np.float32, (6000, 200, 3), 1), (np.float16, (5000, 500, 3), 1), (np.float32, (9000, 90, 7), 1),
    # eight-byte elements: inner dims of 4 and 6 are no divisors of the two-element vector either
    (np.float64, (6633, 80, 4), 1), (np.int64, (700, 1001, 4), 1), (np.float64, (900, 333, 6), 1),
]


@pytest.mark.parametrize("npdt,shape,axis", MODULAR_ROW_CASES, ids=lambda v: getattr(v, "__name__", str(v).replace(" ", "")))
def test_reduction_over_the_middle_axis_with_an_inner_dim_of_3_5_6_7(hpt, orc, dev, npdt, shape, axis):
    """The [C, L] slab runs as one row; lanes in multiples of L keep an accumulator per vector place and rotate them into
    the L outputs at the end; rows start off the 16-byte grid and end with a few single elements. Inner positions get
    offsets far apart; ties for the arg-reductions sit at both ends of the axis (the lowest index wins)."""
    rng = np.random.default_rng(734)
    L, C = shape[-1], shape[axis]
    if np.issubdtype(npdt, np.floating):
        base = (rng.standard_normal(shape) + (np.arange(L) * 3.0 - 2.0)).astype(npdt)
    else:
        info = np.iinfo(npdt)
        lo, hi = max(info.min, -100), min(info.max, 100)
        base = (rng.integers(lo, hi + 1, shape) // 2 + (np.arange(L) % 3)).astype(npdt)
    first = tuple(0 if i == axis else slice(None) for i in range(len(shape)))
    last = tuple(C - 1 if i == axis else slice(None) for i in range(len(shape)))
    top = np.asarray(base.max() + 1, dtype=np.float64).astype(npdt)
    base[first] = top
    base[last] = top
    t, a = upload(hpt, base, dev=dev)
    assert hpt.reduce_plan(t, hpt.SUM, [axis]).startswith("row-modular"), hpt.reduce_plan(t, hpt.SUM, [axis])
    assert np.array_equal(t.max([axis]).numpy(), a.max(axis))
    assert np.array_equal(t.min([axis]).numpy(), a.min(axis))
    assert np.array_equal(t.argmax(axis).numpy(), orc.argreduce(True, a, axis))
    assert np.array_equal(t.argmin(axis).numpy(), orc.argreduce(False, a, axis))
    if npdt == np.float16:
        want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F32).astype(np.float32)
        assert_close(t.sum([axis]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), f"f16 sum {shape}")
    elif np.issubdtype(npdt, np.floating):
        rtol, atol = (F32_RTOL, F32_ATOL) if npdt == np.float32 else (1e-12, 1e-12)
        assert_close(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64), rtol, atol, f"sum {shape}")
        assert_close(t.mean([axis]).numpy(), orc.reduce(orc.MEAN, a, [axis], acc=orc.ACC_F64), rtol, atol, f"mean {shape}")
        out = hpt.Tensor.from_numpy(np.ones(t.sum([axis]).shape, npdt)).to_hip(dev)
        t.sum_([axis], False, False, out)
        assert_close(out.numpy(), orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64) + 1, rtol, atol, f"sum into out {shape}")
    else:
        assert np.array_equal(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis]))
        assert np.array_equal(t.prod([axis]).numpy(), orc.reduce(orc.PROD, a, [axis]))


@pytest.mark.parametrize("shape,bool_shape,plan", [((700, 1000, 4), (1500, 1000, 4), "row-interleaved"), ((600, 2000, 3), (1500, 2000, 3), "row-modular")],
                         ids=["interleaved", "modular"])
def test_every_op_over_the_middle_axis_of_narrow_slabs(hpt, orc, dev, shape, bool_shape, plan):
    """Every op family of the reductions through the row kernels that keep an accumulator per place in the vector."""
    rng = np.random.default_rng(735)
    base = (rng.standard_normal(shape) * 0.05 + 1.0).astype(np.float32)   # products of 1000 ... 2000 factors stay finite
    t, a = upload(hpt, base, dev=dev)
    assert hpt.reduce_plan(t, hpt.SUM, [1]).startswith(plan), hpt.reduce_plan(t, hpt.SUM, [1])
    for op in ("sum", "prod", "mean", "reducel1", "reducel2", "reducel3", "sum_square", "logsumexp"):
        got = getattr(t, op)([1]).numpy()
        want = orc.reduce(getattr(orc, op.upper()), a, [1], acc=orc.ACC_F64)
        assert_close(got, want, F32_RTOL, F32_ATOL * max(1.0, float(np.max(np.abs(want)))), f"{op} {shape}")
    holes = base.copy()
    holes.reshape(-1)[::7] = np.nan
    th, ah = upload(hpt, holes, dev=dev)
    for op in ("nansum", "nanprod"):
        want = orc.reduce(getattr(orc, op.upper()), ah, [1], acc=orc.ACC_F64)
        assert_close(getattr(th, op)([1]).numpy(), want, F32_RTOL, F32_ATOL * max(1.0, float(np.max(np.abs(want)))), f"{op} {shape}")
    assert np.all(np.isnan(th.sum([1]).numpy()))          # every column meets a NaN
    flags = rng.random(bool_shape) < 0.999
    flags[3, :, 1] = True
    flags[5, :, 0] = False
    tb, ab = upload(hpt, flags, dev=dev)
    assert hpt.reduce_plan(tb, hpt.SUM, [1]).startswith(plan), hpt.reduce_plan(tb, hpt.SUM, [1])
    for op in ("sum", "max", "min", "all", "any"):
        assert np.array_equal(getattr(tb, op)([1]).numpy(), orc.reduce(getattr(orc, op.upper()), ab, [1])), f"{op} bool {shape}"
    assert np.array_equal(t.all([1]).numpy(), (a != 0).all(1))
