"""Randomised parity: random shapes (1-D to 4-D, from a few elements to two million), random views of
them (permuted, sliced, stepped forwards and backwards, permuted and stepped), random dtypes, every
op family of the path against the oracle on the same view. The seeds are fixed: a failure names
its case, and every planner region a small or mid-sized tensor can reach is visited by some seed
(general kernels, lean rows / columns, LDS tiles, flat walks, the unaligned forms, splits)."""
import os

import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL, HALF_RTOL, apply_view_np, apply_view_t, half_acc, half_atol

pytestmark = pytest.mark.gpu

CASES_PER_SEED = 60


def rand_shape(rng):
    nd = int(rng.integers(1, 5))
    kind = int(rng.integers(0, 4))
    if kind == 0:
        return [int(rng.integers(1, 9)) for _ in range(nd)]
    if kind == 1:
        return [int(rng.integers(1, 70)) for _ in range(nd)]
    total = int(rng.integers(1 << 10, 1 << 21))
    dims, rem = [], total
    for i in range(nd - 1):
        d = int(rng.integers(1, max(2, int(rem ** (1.0 / (nd - i))) * 2)))
        dims.append(d)
        rem = max(1, rem // d)
    dims.append(rem)
    rng.shuffle(dims)
    if kind == 3:  # sizes that allow whole 128-bit vectors
        dims = [max(8, (d // 8) * 8) if d > 8 else d for d in dims]
    return [int(d) for d in dims]


def rand_view(rng, shape):
    nd = len(shape)
    r = int(rng.integers(0, 7))
    perm = ("permute", tuple(int(p) for p in rng.permutation(nd)))
    if r == 1 and nd >= 2:
        return (perm,)
    if r == 2:  # a window
        return (("slice", tuple((int(rng.integers(0, s // 3 + 1)), int(s - rng.integers(0, s // 3 + 1)), 1) for s in shape)),)
    if r == 3:  # forward steps
        return (("slice", tuple((0, s, int(rng.integers(1, 4))) for s in shape)),)
    if r == 4 and nd >= 2:
        return (perm, ("slice", tuple((0, None, int(rng.integers(1, 3))) for _ in shape)))
    if r == 5:  # backward steps
        return (("slice", tuple((None, None, -int(rng.integers(1, 3))) if rng.integers(0, 2) else (0, None, 1) for _ in shape)),)
    if r == 6 and nd >= 2:
        return (perm, ("slice", tuple((None, None, -1) if i == 0 else (0, None, 1) for i in range(nd))))
    return ()


def rand_base(rng, shape):
    k = int(rng.integers(0, 8))
    if k == 0:
        return rng.integers(-1000, 1000, shape).astype(np.int32)
    if k == 1:
        return rng.integers(-100, 100, shape).astype(np.int64)
    if k == 2:
        return (rng.standard_normal(shape) * 3).astype(np.float64)
    if k == 3:
        return (rng.standard_normal(shape) * 2).astype(np.float16)
    if k == 4:
        return rng.integers(0, 256, shape).astype(np.uint8)
    return (rng.standard_normal(shape) * 3).astype(np.float32)


def layernorm_floor(a, nn, g, ulp):
    """Per-element absolute floor for a layernorm computed in arithmetic of relative precision `ulp`:
    x - mean loses |x| * ulp absolutely whatever the row's spread is, and the result scales that by
    rstd * |gamma|. (Two elements 0.004 apart around 3 normalise to +-0.5: an amplification of 1000.)"""
    x = a.astype(np.float64)
    red = tuple(range(a.ndim - nn, a.ndim))
    var = x.var(axis=red, keepdims=True)
    rstd = 1.0 / np.sqrt(var + 1e-5)
    return 4.0 * ulp * np.abs(x).max(axis=red, keepdims=True) * rstd * np.abs(g.astype(np.float64))


# (HPT_RANDOM_VIEW_SEEDS=200 widens the search on a machine with time to spare)
@pytest.mark.parametrize("seed", range(int(os.environ.get("HPT_RANDOM_VIEW_SEEDS", "16"))))
def test_random_views_against_the_oracle(hpt, orc, dev, seed):
    rng = np.random.default_rng(9000 + seed)
    done = 0
    for it in range(CASES_PER_SEED):
        shape = rand_shape(rng)
        ops = rand_view(rng, shape)
        base = rand_base(rng, shape)
        t = apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)
        a = apply_view_np(base, ops)
        if a.size == 0:
            continue
        nd = a.ndim
        axes = sorted(int(x) for x in rng.choice(nd, int(rng.integers(1, nd + 1)), replace=False))
        what = f"seed={seed} case={it} shape={shape} view={ops} dtype={base.dtype} axes={axes}"
        kind = base.dtype.kind
        half = base.dtype == np.float16
        n_red = int(np.prod([a.shape[x] for x in axes]))
        if kind == "f":
            # f32 / f64: the truth is the compensated f64 sum (exact to an f64 ulp of the result whatever the
            # number of terms); a running f64 sum drifts by ~1e-10 over a million terms of size 3
            acc = half_acc(orc, n_red) if half else orc.ACC_EXACT
            rtol, atol = (HALF_RTOL, None) if half else ((1e-12, 1e-12) if base.dtype == np.float64 else (F32_RTOL, F32_ATOL))
            for name, code in (("sum", orc.SUM), ("mean", orc.MEAN), ("max", orc.MAX), ("min", orc.MIN)):
                got, want = getattr(t, name)(axes).numpy(), orc.reduce(code, a, axes, acc=acc)
                if name in ("max", "min"):
                    assert np.array_equal(got, want), f"{name} {what}"
                else:
                    # f16: a sum of n terms of size ~3 that cancel, rounded once to 11 bits. f32: the device adds
                    # in f64 and rounds once, so the stated 1e-6 holds for any n. f64: the device's own pairwise
                    # f64 adds, 2^-53 of a partial sum each (partial sums ~3 sqrt(n)): a few of those, not n of them
                    floor = (half_atol(want, 11) + 2e-3 * np.sqrt(n_red)) if half else \
                        max(atol, 12 * 2.0 ** -52 * np.sqrt(n_red)) if base.dtype == np.float64 else atol
                    assert_close(got, want, rtol, floor, f"{name} {what}")
        else:
            for name, code in (("sum", orc.SUM), ("prod", orc.PROD), ("max", orc.MAX), ("min", orc.MIN)):
                assert np.array_equal(getattr(t, name)(axes).numpy(), orc.reduce(code, a, axes)), f"{name} {what}"
        ax = int(rng.integers(0, nd))
        assert np.array_equal(t.argmax(ax).numpy(), orc.argreduce(True, a, ax)), f"argmax axis={ax} {what}"
        assert np.array_equal(t.argmin(ax).numpy(), orc.argreduce(False, a, ax)), f"argmin axis={ax} {what}"
        if kind == "f":
            ax = int(rng.integers(0, nd))
            acc = half_acc(orc, a.shape[ax]) if half else orc.ACC_F64
            for log in (False, True):
                got = (t.log_softmax(ax) if log else t.softmax(ax)).numpy()
                want = orc.softmax(a, ax, log=log, acc=acc)
                if half:
                    assert_close(got, want, HALF_RTOL, max(half_atol(want, 11), 6e-8), f"softmax log={log} axis={ax} {what}")
                elif base.dtype == np.float64:
                    assert_close(got, want, 1e-12, 1e-13, f"softmax log={log} axis={ax} {what}")
                else:
                    assert_close(got, want, F32_RTOL, 2 * F32_ATOL if log else F32_ATOL, f"softmax log={log} axis={ax} {what}")
            nn = int(rng.integers(1, nd + 1))
            ns = list(a.shape[nd - nn:])
            if int(np.prod(ns)) >= 2:
                g, b = rng.normal(1, 0.1, ns).astype(base.dtype), rng.normal(0, 0.1, ns).astype(base.dtype)
                tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
                got = t.layernorm(ns, tg, tb, 1e-5).numpy()
                acc = half_acc(orc, int(np.prod(ns))) if half else orc.ACC_F64
                want = orc.layernorm(a, nn, g, b, 1e-5, acc=acc)
                if half:  # (the arithmetic is f32; the result is rounded to f16 once)
                    assert_close(got, want, HALF_RTOL, max(half_atol(want, 10), 6e-8) + layernorm_floor(a, nn, g, 2.0 ** -24),
                                 f"layernorm nn={nn} {what}")
                elif base.dtype == np.float64:
                    assert_close(got, want, 1e-11, 1e-12 + layernorm_floor(a, nn, g, 2.0 ** -53), f"layernorm nn={nn} {what}")
                else:
                    assert_close(got, want, F32_RTOL, 4 * F32_ATOL + layernorm_floor(a, nn, g, 2.0 ** -24), f"layernorm nn={nn} {what}")
        assert np.array_equal(t.contiguous().numpy(), np.ascontiguousarray(a)), f"contiguous {what}"
        done += 1
    assert done >= CASES_PER_SEED // 2
