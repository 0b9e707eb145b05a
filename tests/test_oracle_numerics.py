"""The oracle's arithmetic against golden vectors, closed forms and library routines (CPU only).

What each check pins: integer ops are bit-exact against numpy's wrap-around arithmetic;
max/min/argmax are exact; float sums against float64; softmax / layernorm against the torch
float64 fixtures in tests/golden (the reference's own yardstick) and against invariants; the
lane-structured and per-op-rounded modes against properties that a dropped term, a wrong
index or a transposed operand would break.
"""
import ast
import itertools

import numpy as np
import pytest

from conftest import assert_close
from util import apply_view_np

GOLD = None


def gold():
    global GOLD
    if GOLD is None:
        from pathlib import Path
        GOLD = np.load(Path(__file__).parent / "golden" / "golden.npz")
    return GOLD


def cases(prefix):
    from pathlib import Path
    names = (Path(__file__).parent / "golden" / "cases.txt").read_text().split()
    return [n for n in names if n.startswith(prefix)]


def load_case(name):
    g = gold()
    base = g[f"base/{int(g[name + '/base_ref'])}"]
    ops = [(k, tuple(tuple(x) if isinstance(x, (list, tuple)) else x for x in a)) for k, a in ast.literal_eval(str(g[name + "/ops"]))]
    return base, ops, apply_view_np(base, ops)


@pytest.mark.parametrize("name", cases("softmax/"))
def test_softmax_golden(orc, name):
    base, ops, v = load_case(name)
    axis = int(gold()[name + "/axis"])
    for log, key in ((False, "softmax"), (True, "log_softmax")):
        want = gold()[f"{name}/{key}"]
        assert_close(orc.softmax(v, axis, log=log, acc=orc.ACC_F64), want, 1e-6, 1e-7, f"{name} {key} f64")
        assert_close(orc.softmax(v, axis, log=log, acc=orc.ACC_NATIVE, lanes=8), want, 1e-5, 2e-6, f"{name} {key} native")


@pytest.mark.parametrize("name", cases("layernorm/"))
def test_layernorm_golden(orc, name):
    base, ops, v = load_case(name)
    g = gold()
    nn = int(g[name + "/n_norm"])
    gamma, beta = g[name + "/gamma"], g[name + "/beta"]
    assert_close(orc.layernorm(v, nn, gamma, beta, 1e-5, acc=orc.ACC_F64), g[name + "/out"], 1e-6, 1e-6, name)
    assert_close(orc.layernorm(v, nn, None, None, 1e-5, acc=orc.ACC_F64), g[name + "/out_plain"], 1e-6, 1e-6, name)
    assert_close(orc.layernorm(v, nn, gamma, beta, 1e-5, acc=orc.ACC_NATIVE), g[name + "/out"], 2e-4, 2e-5, name + " native")


@pytest.mark.parametrize("name", cases("reduce/"))
def test_reduce_golden(orc, name):
    base, ops, v = load_case(name)
    g = gold()
    axes = [int(a) for a in g[name + "/axes"]]
    for op in ("sum", "mean", "max", "min", "sum_square", "reducel1", "reducel2", "reducel3"):
        want = np.atleast_1d(g[f"{name}/{op}"])
        got = orc.reduce(getattr(orc, op.upper()), v, axes, acc=orc.ACC_F64)
        assert_close(got.reshape(-1), want.reshape(-1), 1e-6, 1e-6, f"{name} {op}")
        nat = orc.reduce(getattr(orc, op.upper()), v, axes, acc=orc.ACC_NATIVE, lanes=8)
        scale = np.abs(want).max() + 1.0
        assert_close(nat.reshape(-1), want.reshape(-1), 1e-5, 1e-5 * scale, f"{name} {op} native")


@pytest.mark.parametrize("name", cases("argreduce"))
def test_argreduce_golden(orc, name):
    base, ops, v = load_case(name)
    axis = int(gold()[name + "/axis"])
    assert np.array_equal(orc.argreduce(True, v, axis), gold()[name + "/argmax"])
    assert np.array_equal(orc.argreduce(False, v, axis), gold()[name + "/argmin"])


@pytest.mark.parametrize("name", cases("reduce_i32/"))
def test_reduce_i32_golden(orc, name):
    base, ops, v = load_case(name)
    axes = [int(a) for a in gold()[name + "/axes"]]
    assert np.array_equal(orc.reduce(orc.SUM, v, axes).reshape(-1), np.atleast_1d(gold()[name + "/sum"]).reshape(-1))
    assert np.array_equal(orc.reduce(orc.MAX, v, axes).reshape(-1), np.atleast_1d(gold()[name + "/max"]).reshape(-1))


def test_docstring_kats(orc):
    # hpt-traits/src/ops/reduce.rs:21-39, 58-62, 146-149, 166-168, 294-350
    a = np.array([[1.0, 2.0], [3.0, 4.0]], np.float32)
    assert orc.reduce(orc.SUM, a, [0, 1]).tolist() == [10.0]
    assert orc.reduce(orc.SUM, a, [0, 1], True).tolist() == [[10.0]]
    assert orc.reduce(orc.MEAN, a, [0, 1]).tolist() == [2.5]
    assert orc.reduce(orc.SUM_SQUARE, a, [0, 1]).tolist() == [30.0]
    assert orc.reduce(orc.REDUCEL1, a, [0, 1]).tolist() == [10.0]
    assert abs(orc.reduce(orc.LOGSUMEXP, a, [0, 1])[0] - 4.4401898) < 1e-6
    c = np.array([[1.0, 2.0], [2.0, 3.0]], np.float32)
    assert abs(orc.reduce(orc.REDUCEL2, c, [0, 1])[0] - 4.2426405) < 1e-6
    assert abs(orc.reduce(orc.REDUCEL3, c, [0, 1])[0] - 3.5303483) < 1e-6
    v = np.array([10.0, 3.0, 2.0], np.float32)
    assert orc.argreduce(True, v, 0).tolist() == [0] and orc.argreduce(False, v, 0).tolist() == [2]


@pytest.mark.parametrize("npdt", [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64])
def test_integer_wraparound_bit_exact(orc, npdt):
    rng = np.random.default_rng(3)
    info = np.iinfo(npdt)
    a = rng.integers(info.min, info.max, (7, 50, 9), dtype=npdt, endpoint=True)
    for axes in ([0], [1], [2], [0, 2], [0, 1, 2]):
        for v in (a, a.transpose(2, 0, 1), a[:, ::3, 1:]):
            assert np.array_equal(orc.reduce(orc.SUM, v, axes).reshape(-1), np.atleast_1d(v.sum(axis=tuple(axes), dtype=npdt)).reshape(-1))
            assert np.array_equal(orc.reduce(orc.PROD, v, axes).reshape(-1), np.atleast_1d(v.prod(axis=tuple(axes), dtype=npdt)).reshape(-1))
            assert np.array_equal(orc.reduce(orc.MAX, v, axes).reshape(-1), np.atleast_1d(v.max(axis=tuple(axes))).reshape(-1))
            assert np.array_equal(orc.reduce(orc.MIN, v, axes).reshape(-1), np.atleast_1d(v.min(axis=tuple(axes))).reshape(-1))
            with np.errstate(over="ignore"):
                assert np.array_equal(orc.reduce(orc.SUM_SQUARE, v, axes).reshape(-1), np.atleast_1d((v * v).sum(axis=tuple(axes), dtype=npdt)).reshape(-1))


@pytest.mark.parametrize("npdt", [np.float32, np.float64, np.float16])
def test_float_prod_nansum_nanprod_all_any_against_numpy_float64(orc, npdt):
    """The float branches of prod / nansum / nanprod / all / any against numpy in float64 on the same three
    layouts (contiguous, permuted, sliced with a step). Values near 1 keep a product of 50 terms in range;
    NaNs are planted so that nansum / nanprod have something to skip, zeros so that all / any see both answers.
    A dropped NaN test, a sum where a product belongs or a wrong identity (0 for prod) fails here."""
    rng = np.random.default_rng(33)
    a = (1.0 + 0.2 * rng.standard_normal((7, 50, 9))).astype(npdt)
    withnan = a.copy()
    withnan[rng.random(a.shape) < 0.1] = np.nan
    withnan[3, :, 4] = np.nan                    # one output with nothing but NaN: the identities show
    zeros = a.copy()
    zeros[rng.random(a.shape) < 0.3] = 0
    zeros[2, :, :] = 0                           # all-zero outputs for `any`
    zeros[5, :, 1::2] = 1                        # all-nonzero outputs for `all`
    zeros[0, 0, 0] = np.nan                      # NaN is not zero: it counts as true
    half = npdt == np.float16
    acc = orc.ACC_F32 if half else orc.ACC_F64
    rtol = 2e-3 if half else (1e-6 if npdt == np.float32 else 1e-12)
    patol = 6e-8 if half else 0   # f16 products of many terms reach the subnormals (spacing 2^-24)
    for axes in ([0], [1], [2], [0, 2], [0, 1, 2]):
        ax = tuple(axes)
        for mk in (lambda v: v, lambda v: v.transpose(2, 0, 1), lambda v: v[:, ::3, 1:]):
            v, vn, vz = mk(a), mk(withnan), mk(zeros)
            v64, vn64 = v.astype(np.float64), vn.astype(np.float64)
            flat = lambda r: np.atleast_1d(r).reshape(-1)
            assert_close(flat(orc.reduce(orc.PROD, v, axes, acc=acc)), flat(v64.prod(axis=ax)), rtol, patol, f"prod {axes}")
            assert_close(flat(orc.reduce(orc.NANSUM, vn, axes, acc=acc)), flat(np.nansum(vn64, axis=ax)), rtol, 1e-3 if half else 1e-6,
                         f"nansum {axes}")
            assert_close(flat(orc.reduce(orc.NANPROD, vn, axes, acc=acc)), flat(np.nanprod(vn64, axis=ax)), rtol, patol,
                         f"nanprod {axes}")
            # a NaN poisons the plain forms
            assert np.isnan(flat(orc.reduce(orc.PROD, vn, axes, acc=acc))).tolist() == np.isnan(flat(vn64.prod(axis=ax))).tolist()
            assert np.isnan(flat(orc.reduce(orc.SUM, vn, axes, acc=acc))).tolist() == np.isnan(flat(vn64.sum(axis=ax))).tolist()
            got_all, got_any = orc.reduce(orc.ALL, vz, axes), orc.reduce(orc.ANY, vz, axes)
            assert got_all.dtype == np.bool_ and got_any.dtype == np.bool_
            assert np.array_equal(flat(got_all), flat(np.all(vz, axis=ax)))
            assert np.array_equal(flat(got_any), flat(np.any(vz, axis=ax)))
    # the identities: nothing but NaN -> nansum 0, nanprod 1
    col = withnan[3, :, 4]
    assert orc.reduce(orc.NANSUM, col, [0], acc=acc)[0] == 0 and orc.reduce(orc.NANPROD, col, [0], acc=acc)[0] == 1


def test_argmax_strict_compare_rules(orc):
    # ties -> first; NaN never wins; an all -inf / all MIN row -> 0 (argreduce_kernels.rs:13-21)
    a = np.array([[1, 5, 5, 2], [7, 7, 7, 7], [-3, -9, -3, -9]], np.int32)
    assert orc.argreduce(True, a, 1).tolist() == [1, 0, 0]
    assert orc.argreduce(False, a, 1).tolist() == [0, 0, 1]
    f = np.array([[np.nan, 1.0, 5.0, 5.0], [-np.inf] * 4, [np.nan] * 4], np.float32)
    assert orc.argreduce(True, f, 1).tolist() == [2, 0, 0]
    assert orc.argreduce(False, f, 1).tolist() == [1, 0, 0]
    m = np.full((2, 5), np.iinfo(np.int32).min, np.int32)
    assert orc.argreduce(True, m, 1).tolist() == [0, 0]


def test_softmax_invariants(orc):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((9, 257)) * 4).astype(np.float32)
    s = orc.softmax(x, 1, acc=orc.ACC_F64).astype(np.float64)
    assert_close(s.sum(1), np.ones(9), 1e-6, 0, "rows sum to 1")
    # shift invariance and monotonicity
    assert_close(orc.softmax(x + np.float32(3.0), 1, acc=orc.ACC_F64), s, 2e-5, 1e-9, "shift invariance")
    order = np.argsort(x[0])
    assert np.all(np.diff(s[0][order]) >= 0)
    # log_softmax = x - max - ln(sum exp(x - max)), computed independently here in float64
    xd = x.astype(np.float64)
    ref = xd - xd.max(1, keepdims=True) - np.log(np.exp(xd - xd.max(1, keepdims=True)).sum(1, keepdims=True))
    assert_close(orc.softmax(x, 1, log=True, acc=orc.ACC_F64), ref, 1e-6, 1e-6, "log_softmax definition")
    # a row with one finite entry: exactly one-hot; log form 0 / -inf; an all -inf row: NaN
    m = np.full((3, 40), -np.inf, np.float32)
    m[0, 7] = 2.0
    m[1, :] = 1.0
    out = orc.softmax(m, 1)
    assert out[0, 7] == 1.0 and out[0].sum() == 1.0
    assert_close(out[1], np.full(40, 1 / 40), 1e-6, 0, "uniform row")
    assert np.isnan(out[2]).all()
    lo = orc.softmax(m, 1, log=True)
    assert lo[0, 7] == 0.0 and np.isneginf(np.delete(lo[0], 7)).all()
    # column softmax on a transposed view equals row softmax on the transposed data
    assert_close(orc.softmax(x.T, 0, acc=orc.ACC_F64), s.T, 1e-7, 0, "strided axis")


def test_layernorm_closed_forms(orc):
    x = np.full((3, 33), 7.25, np.float32)
    g = np.linspace(0.5, 2, 33).astype(np.float32)
    b = np.linspace(-1, 1, 33).astype(np.float32)
    assert np.array_equal(orc.layernorm(x, 1, g, b, 1e-5), np.broadcast_to(b, x.shape))    # constant rows -> beta
    x2 = np.array([[1.0, 3.0], [-2.0, 6.0]], np.float32)
    var = np.array([1.0, 16.0])
    want = np.stack([-1 / np.sqrt(1 + 1e-5 / var), 1 / np.sqrt(1 + 1e-5 / var)], 1)
    assert_close(orc.layernorm(x2, 1, None, None, 1e-5, acc=orc.ACC_F64), want, 1e-6, 1e-7, "2-element rows")
    # pre-affine invariants: mean 0, biased variance 1/(1 + eps/var)
    rng = np.random.default_rng(5)
    x3 = (rng.standard_normal((6, 500)) * 3 + 2).astype(np.float32)
    y = orc.layernorm(x3, 1, None, None, 1e-5, acc=orc.ACC_F64).astype(np.float64)
    assert np.abs(y.mean(1)).max() < 1e-6
    v = x3.astype(np.float64).var(1)
    assert_close(y.var(1), 1 / (1 + 1e-5 / v), 1e-5, 0, "unit variance")
    # gamma only / beta only (normalization.rs:187-192)
    g3, b3 = rng.normal(1, 0.1, 500).astype(np.float32), rng.normal(0, 0.1, 500).astype(np.float32)
    assert_close(orc.layernorm(x3, 1, g3, None, 1e-5, acc=orc.ACC_F64), y * g3, 1e-6, 1e-6, "gamma only")
    assert_close(orc.layernorm(x3, 1, None, b3, 1e-5, acc=orc.ACC_F64), y + b3, 1e-6, 1e-6, "beta only")
    # several normalised dims == one flattened dim
    x4 = x3.reshape(6, 20, 25)
    assert np.array_equal(orc.layernorm(x4, 2, g3.reshape(20, 25), b3.reshape(20, 25), 1e-5).reshape(6, 500),
                          orc.layernorm(x3, 1, g3, b3, 1e-5))


def test_lane_structure_and_rounding_modes(orc):
    """lanes=L folds lane accumulators in lane order (vectors/utils.rs:83-105): for a row whose
    length is a multiple of L it equals summing the L interleaved sub-rows first. The literal
    per-op-rounded f16 mode differs from f32 accumulation exactly where theory says it must."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal((4, 64)).astype(np.float32)
    got = orc.reduce(orc.SUM, x, [1], lanes=8)
    want = np.zeros(4, np.float32)
    for r in range(4):
        lanes = np.zeros(8, np.float32)
        for v in range(8):
            lanes = (lanes + x[r, v * 8:(v + 1) * 8]).astype(np.float32)
        acc = np.float32(0)
        for l in range(8):
            acc = np.float32(acc + lanes[l])
        want[r] = acc
    assert np.array_equal(got, want)
    # sequential f16 accumulation of 4096 ones stalls at 2048 (ulp 2 above 2048); f32 accumulation does not
    ones = np.ones((1, 4096), np.float16)
    assert orc.reduce(orc.SUM, ones, [1], acc=orc.ACC_NATIVE, lanes=1)[0] == 2048
    assert orc.reduce(orc.SUM, ones, [1], acc=orc.ACC_F32)[0] == 4096
    # bf16: 256 + 1 is not representable (8-bit significand)
    onesb = orc.f32_to_bf16(np.ones((1, 1024), np.float32))
    assert orc.bf16_to_f32(orc.reduce(orc.SUM, onesb, [1], acc=orc.ACC_NATIVE, dtype=orc.BF16))[0] == 256
    assert orc.bf16_to_f32(orc.reduce(orc.SUM, onesb, [1], acc=orc.ACC_F32, dtype=orc.BF16))[0] == 1024


def test_sequential_f32_accumulation_is_no_truth_for_long_half_rows(orc):
    """f16 layernorm over ALL dims of a [63, 50, 53, 37] tensor permuted (1, 2, 0, 3): one row of
    6 177 150 elements. A randomised device run once disagreed with the oracle's ACC_F32 mode here on
    4 elements (outputs next to zero, where a relative tolerance does not help). Which side was off is
    decided on the host: the f64-accumulating mode agrees with numpy's float64 statistics to f16
    rounding; the sequential-f32 mode does not, because its running sum of (x - mean)^2 passes 2^24,
    where f32 moves in steps of 2 and terms below 1 vanish: it ends ~0.8 % low, the reciprocal
    standard deviation ~0.4 % high. So long half rows are checked against ACC_F64 (tests/util.py half_acc)."""
    rng = np.random.default_rng(0)
    x = (rng.standard_normal([63, 50, 53, 37]) * 2).astype(np.float16)
    a = x.transpose(1, 2, 0, 3)
    g = rng.normal(1, 0.1, a.shape).astype(np.float16)
    b = rng.normal(0, 0.1, a.shape).astype(np.float16)
    xd = a.astype(np.float64)
    ref = (xd - xd.mean()) / np.sqrt(xd.var() + 1e-5) * g.astype(np.float64) + b.astype(np.float64)
    w64 = orc.layernorm(a, 4, g, b, 1e-5, acc=orc.ACC_F64).astype(np.float64)
    w32 = orc.layernorm(a, 4, g, b, 1e-5, acc=orc.ACC_F32).astype(np.float64)
    big = np.abs(ref) > 0.5
    # f64 mode: half an ulp of f16 (2^-11 relative) and nothing more
    assert (np.abs(w64 - ref)[big] / np.abs(ref)[big]).max() < 2.0 ** -11 * 1.01
    assert np.abs(w64 - ref).max() < 2.0 ** -9 * 1.01            # |y| < 8: half an ulp is 2^-9
    # sequential f32 mode: off by several parts in a thousand, everywhere
    rel32 = (np.abs(w32 - ref)[big] / np.abs(ref)[big])
    assert np.median(rel32) > 2e-3 and rel32.max() < 1e-2
    # the cause, in isolation: the same running sum of squares in numpy's sequential f32 cumsum
    xf = a.astype(np.float32).reshape(-1)
    sq = ((xf - np.float32(xd.mean())) ** 2).astype(np.float32)
    seq = float(np.cumsum(sq, dtype=np.float32)[-1])
    true = float(sq.astype(np.float64).sum())
    assert seq > 2.0 ** 24 and 0.990 < seq / true < 0.995


def test_timed_restatement_equals_oracle(orc):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((67, 1030)) * 2 + 1).astype(np.float32)
    g, b = rng.normal(1, 0.1, 1030).astype(np.float32), rng.normal(0, 0.1, 1030).astype(np.float32)
    for nt in (1, 3, 8):
        assert np.array_equal(orc.mt_layernorm_f32(x, g, b, 1e-5, nt), orc.layernorm(x, 1, g, b, 1e-5))
        assert_close(orc.mt_softmax_f32(x, False, nt), orc.softmax(x, 1, lanes=8), 2e-6, 1e-9, "mt softmax")
        assert_close(orc.mt_softmax_f32(x, True, nt), orc.softmax(x, 1, log=True, lanes=8), 2e-6, 2e-6, "mt log_softmax")
        assert np.array_equal(orc.mt_reduce_rows_f32(x, orc.SUM, nt), orc.reduce(orc.SUM, x, [1], lanes=8))
        assert np.array_equal(orc.mt_reduce_rows_f32(x, orc.MAX, nt), x.max(1))
    # the vectorisable exp is within 2 ulp of libm over the softmax range
    l = orc.lib()
    xs = np.concatenate([np.linspace(-100, 0, 5001), np.linspace(0, 80, 1001)]).astype(np.float32)
    got = np.array([l.orc_vexpf(float(v)) for v in xs], np.float64)
    want = np.exp(xs.astype(np.float64))
    assert (np.abs(got - want) <= 3e-7 * want + 1e-45).all()
    assert orc.physical_cores() >= 1


def test_compensated_f64_mode_against_fsum(orc):
    """ACC_EXACT (the truth for long f64 sums) equals math.fsum where a running f64 sum does not:
    ill-conditioned sums whose large terms cancel, and a million random terms; views and several axes go
    through the same path; mean / sum_square / reducel1 are built on it."""
    import math
    x = np.array([1e100, 1.0, -1e100, 1e-5, 3.0, -1e80, 1e80] * 1000)
    assert orc.reduce(orc.SUM, x, [0], acc=orc.ACC_EXACT)[0] == math.fsum(x)
    assert orc.reduce(orc.SUM, x, [0], acc=orc.ACC_F64)[0] != math.fsum(x)   # the plain mode loses the small terms
    rng = np.random.default_rng(5)
    y = rng.standard_normal(1_300_000) * 3
    assert orc.reduce(orc.SUM, y, [0], acc=orc.ACC_EXACT)[0] == math.fsum(y)
    assert abs(orc.reduce(orc.SUM, y, [0], acc=orc.ACC_F64)[0] - math.fsum(y)) > 1e-12
    m = orc.reduce(orc.MEAN, y, [0], acc=orc.ACC_EXACT)[0]
    assert m == math.fsum(y) / y.size
    assert orc.reduce(orc.SUM_SQUARE, y, [0], acc=orc.ACC_EXACT)[0] == math.fsum(v * v for v in y)
    assert orc.reduce(orc.REDUCEL1, y, [0], acc=orc.ACC_EXACT)[0] == math.fsum(abs(v) for v in y)
    z = rng.standard_normal((7, 300, 11)) * np.array([1e12, 1.0, 1e-9] * 100)[None, :, None]
    v = z.transpose(2, 0, 1)[::2, :, 5:]
    got = orc.reduce(orc.SUM, v, [1, 2], acc=orc.ACC_EXACT)
    want = [math.fsum(v[i].ravel()) for i in range(v.shape[0])]
    assert np.array_equal(got, want)
    # f32 input: the exact sum rounded once to f32
    w = (rng.standard_normal(200_000) * 3).astype(np.float32)
    assert orc.reduce(orc.SUM, w, [0], acc=orc.ACC_EXACT)[0] == np.float32(math.fsum(w.astype(np.float64)))
    # infinities and NaN pass through as in the plain mode
    assert orc.reduce(orc.SUM, np.array([1.0, np.inf, 2.0]), [0], acc=orc.ACC_EXACT)[0] == np.inf
    assert np.isnan(orc.reduce(orc.SUM, np.array([1.0, np.inf, -np.inf]), [0], acc=orc.ACC_EXACT)[0])
    assert np.isnan(orc.reduce(orc.SUM, np.array([1.0, np.nan, 2.0]), [0], acc=orc.ACC_EXACT)[0])
    assert orc.reduce(orc.NANSUM, np.array([1.0, np.nan, 2.0]), [0], acc=orc.ACC_EXACT)[0] == 3.0
