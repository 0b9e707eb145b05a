"""The reference's own device tests for this path, restated: hpt-tests/src/hpt/cuda/reduce.rs builds ten
random 3-D i64 tensors (randint(-1000, 1000), dims 1..512), reduces them over the axis sets {1}, {2},
{0,1}, {0,2}, {1,2}, {0,1,2} with keep_dims = true, repeats each into the result with the in-place form
(`sum_(axes, keep_dims, init_out = true, out)`) and compares EXACTLY (:17-37, 158-213); the same for
nansum, prod, min, max (:215-565) and argmax / argmin over one axis (:1421-1612, the only place of the
reference's tests where ties occur); f64 randn inputs are compared with a relative difference (:54-87,
here: the f64 tolerance of the other tests). The four layout classes of docs/dev_guide/test_rules.md:3-7
(contiguous, permuted, sliced, sliced with a step) are run for every shape. Shapes are seeded here and
capped at 2^24 elements."""
import numpy as np
import pytest

from util import layouts_for, upload

pytestmark = pytest.mark.gpu

AXIS_SETS = ([1], [2], [0, 1], [0, 2], [1, 2], [0, 1, 2])


def shapes(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        s = [int(rng.integers(1, 512)) for _ in range(3)]
        if s[0] * s[1] * s[2] <= 1 << 24:
            out.append(s)
    return out


@pytest.mark.parametrize("shape", shapes(31, 10), ids=str)
def test_i64_reductions_are_exact_on_the_references_random_shapes(hpt, dev, shape):
    rng = np.random.default_rng(sum(shape))
    base = rng.integers(-1000, 1000, shape).astype(np.int64)
    for lname, ops in layouts_for(shape, rng):
        t, a = upload(hpt, base, ops, dev=dev)
        if a.size == 0:
            continue
        for axes in AXIS_SETS:
            ax = tuple(axes)
            for name, want in (("sum", a.sum(ax, keepdims=True)), ("nansum", a.sum(ax, keepdims=True)),
                               ("max", a.max(ax, keepdims=True)), ("min", a.min(ax, keepdims=True))):
                got = getattr(t, name)(axes, keep_dims=True)
                assert got.shape == list(want.shape), f"{name} {shape} {lname} {axes}: shape {got.shape}"
                assert np.array_equal(got.numpy(), want), f"{name} {shape} {lname} {axes}"
                if name == "sum":
                    # sum_(axes, keep_dims, init_out = true, out): the previous result is overwritten, not added to
                    again = t.sum_(axes, True, True, got)
                    assert np.array_equal(again.numpy(), want), f"sum_ {shape} {lname} {axes}"
        # prod of values up to 1000 wraps at once: small factors keep it meaningful (and it still wraps)
        small = (base % 5 - 2).astype(np.int64)
        ts, s = upload(hpt, small, ops, dev=dev)
        for axes in ([1], [0, 2]):
            want = np.multiply.reduce(s, axis=tuple(axes), keepdims=True) if len(axes) == 1 else \
                np.multiply.reduce(np.multiply.reduce(s, axis=2, keepdims=True), axis=0, keepdims=True)
            assert np.array_equal(ts.prod(axes, keep_dims=True).numpy(), want), f"prod {shape} {lname} {axes}"
        for axis in range(3):
            # ties everywhere (2000 values over up to 511 positions, and the % 5 tensor): the first extremum wins
            for tt, aa in ((t, a), (ts, s)):
                assert np.array_equal(tt.argmax(axis, keep_dims=True).numpy(), np.expand_dims(aa.argmax(axis), axis)), \
                    f"argmax {shape} {lname} axis {axis}"
                assert np.array_equal(tt.argmin(axis, keep_dims=True).numpy(), np.expand_dims(aa.argmin(axis), axis)), \
                    f"argmin {shape} {lname} axis {axis}"


@pytest.mark.parametrize("shape", shapes(32, 4), ids=str)
def test_f64_reductions_on_the_references_random_shapes(hpt, orc, dev, shape):
    rng = np.random.default_rng(sum(shape) + 1)
    base = rng.standard_normal(shape)
    for lname, ops in layouts_for(shape, rng):
        t, a = upload(hpt, base, ops, dev=dev)
        if a.size == 0:
            continue
        for axes in AXIS_SETS:
            ax = tuple(axes)
            n = int(np.prod([a.shape[i] for i in axes]))
            for name, want in (("sum", a.sum(ax, keepdims=True)), ("mean", a.mean(ax, keepdims=True)),
                               ("max", a.max(ax, keepdims=True)), ("min", a.min(ax, keepdims=True)),
                               ("reducel2", np.sqrt((a * a).sum(ax, keepdims=True))),
                               ("sum_square", (a * a).sum(ax, keepdims=True))):
                got = getattr(t, name)(axes, keep_dims=True).numpy()
                if name in ("max", "min"):
                    assert np.array_equal(got, want), f"{name} {shape} {lname} {axes}"
                else:
                    # numpy's pairwise f64 sums and the device's tree differ by rounding only
                    np.testing.assert_allclose(got, want, rtol=1e-11, atol=1e-13 * max(1.0, float(np.sqrt(n))) * 10,
                                               err_msg=f"{name} {shape} {lname} {axes}")
