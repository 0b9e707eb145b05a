"""GPU parity of softmax / log_softmax / layernorm against the CPU oracle, through the C ABI.

Mirrors hpt-tests/src/hpt/cpu/softmax.rs:30-87 (random 1-2-D shapes, gamma/beta, eps 1e-5) and
hpt-tests/src/hpt/cuda/normalization.rs:39-53 (one shape per kernel size class, both axes),
extended to the four layouts and the half types.
"""
import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol, layouts_for, upload

pytestmark = pytest.mark.gpu

SIZE_CLASS_SHAPES = [[1, 13], [2, 1024], [3, 1123], [3, 4096], [3, 5551]]


@pytest.mark.parametrize("log", [False, True])
def test_softmax_f32_size_classes_both_axes(hpt, orc, dev, log):
    rng = np.random.default_rng(200)
    for shape in SIZE_CLASS_SHAPES + [[5, 40000], [2, 70001], [300, 7], [1, 1]]:
        base = rng.uniform(-10, 10, shape).astype(np.float32)
        t, a = upload(hpt, base, dev=dev)
        for axis in (0, 1, -1):
            got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
            want = orc.softmax(a, axis, log=log, acc=orc.ACC_F64)
            assert_close(got, want, F32_RTOL, F32_ATOL, f"softmax log={log} {shape} axis={axis}")


@pytest.mark.parametrize("log", [False, True])
def test_softmax_random_shapes_layouts(hpt, orc, dev, log):
    rng = np.random.default_rng(201)
    for case in range(20):
        nd = int(rng.integers(1, 4))
        shape = [int(rng.integers(1, 40)) for _ in range(nd)]
        for npdt in (np.float32, np.float64):
            base = (rng.standard_normal(shape) * 3).astype(npdt)
            for lname, ops in layouts_for(shape, rng):
                t, a = upload(hpt, base, ops, dev=dev)
                if a.size == 0:
                    continue
                for axis in range(a.ndim):
                    got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
                    want = orc.softmax(a, axis, log=log, acc=orc.ACC_F64)
                    assert_close(got, want, F32_RTOL, F32_ATOL, f"softmax log={log} {npdt.__name__} {shape} {lname} axis={axis}")
                    if not log:
                        assert_close(got.sum(axis), np.ones_like(got.sum(axis)), 1e-5, 0, "rows sum to 1")


def test_softmax_masked_rows(hpt, orc, dev):
    """-inf entries (a causal mask is data): one finite entry -> exactly one-hot / (0, -inf);
    an all -inf row -> NaN, as x - max = -inf - -inf on the CPU."""
    x = np.full((4, 300), -np.inf, np.float32)
    x[0, 0] = 1.5
    x[1, :7] = np.arange(7)
    x[2, 299] = -3.0
    t, a = upload(hpt, x, dev=dev)
    s = t.softmax(1).numpy()
    assert s[0, 0] == 1.0 and np.all(s[0, 1:] == 0)
    assert s[2, 299] == 1.0 and np.all(s[2, :299] == 0)
    assert_close(s[1], orc.softmax(a, 1, acc=orc.ACC_F64)[1], F32_RTOL, F32_ATOL, "partly masked row")
    assert np.all(np.isnan(s[3]))
    ls = t.log_softmax(1).numpy()
    assert ls[0, 0] == 0.0 and np.all(np.isneginf(ls[0, 1:]))


@pytest.mark.parametrize("name", ["f16", "bf16"])
@pytest.mark.parametrize("log", [False, True])
def test_softmax_half_types(hpt, orc, dev, name, log):
    rng = np.random.default_rng(202)
    for shape in ([7, 2048], [5, 333], [64, 64], [3, 9000]):
        x = (rng.standard_normal(shape) * 3).astype(np.float32)
        if name == "f16":
            base, dt, odt, bits, tof = x.astype(np.float16), None, None, 11, lambda v: v.astype(np.float32)
        else:
            base, dt, odt, bits, tof = hpt.f32_to_bf16_bits(x), hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32
        for lname, ops in layouts_for(shape, rng):
            t, a = upload(hpt, base, ops, dtype=dt, dev=dev)
            for axis in range(a.ndim):
                got = tof((t.log_softmax(axis) if log else t.softmax(axis)).numpy())
                want = tof(orc.softmax(a, axis, log=log, acc=orc.ACC_F32, dtype=odt))
                # floor: f16 results below its smallest normal lose bits; half an ulp of the scale otherwise
                atol = max(half_atol(want, bits), 6.2e-5 * 2.0 ** -bits if name == "f16" else 0.0)
                if name == "f16" and not log:
                    atol = max(atol, 6e-8)
                assert_close(got, want, HALF_RTOL, atol, f"softmax {name} log={log} {shape} {lname} axis={axis}")


def test_layernorm_f32_random_shapes(hpt, orc, dev):
    rng = np.random.default_rng(203)
    for case in range(40):
        nd = int(rng.integers(1, 3))
        shape = [int(rng.integers(1, 10)) for _ in range(nd)]
        base = rng.standard_normal(shape).astype(np.float32)
        n = shape[-1]
        g = np.arange(n, dtype=np.float32)
        b = np.arange(n, dtype=np.float32)
        t, a = upload(hpt, base, dev=dev)
        tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
        got = t.layernorm([n], tg, tb, 1e-5).numpy()
        want = orc.layernorm(a, 1, g, b, 1e-5, acc=orc.ACC_F64)
        assert_close(got, want, 1e-5, 1e-5, f"layernorm {shape}")


def test_layernorm_sizes_layouts_affine_variants(hpt, orc, dev):
    rng = np.random.default_rng(204)
    for shape, nn in (([6, 13], 1), ([5, 1024], 1), ([3, 1123], 1), ([4, 4096], 1), ([2, 5551], 1),
                      ([3, 40000], 1), ([2, 70001], 1), ([4, 6, 32], 2), ([2, 3, 4, 5], 3), ([7, 5], 2)):
        for npdt in (np.float32, np.float64):
            base = (rng.standard_normal(shape) + rng.uniform(-5, 5, shape[:1] + [1] * (len(shape) - 1))).astype(npdt)
            for lname, ops in layouts_for(shape, rng):
                t, a = upload(hpt, base, ops, dev=dev)
                if a.size == 0:
                    continue
                ns = list(a.shape[a.ndim - nn:])
                g = rng.normal(1, 0.1, ns).astype(npdt)
                b = rng.normal(0, 0.1, ns).astype(npdt)
                tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
                for gg, bb, tgg, tbb in ((g, b, tg, tb), (g, None, tg, None), (None, b, None, tb), (None, None, None, None)):
                    got = t.layernorm(ns, tgg, tbb, 1e-5).numpy()
                    want = orc.layernorm(a, nn, gg, bb, 1e-5, acc=orc.ACC_F64)
                    assert_close(got, want, F32_RTOL, F32_ATOL, f"layernorm {npdt.__name__} {shape} {lname} g={gg is not None} b={bb is not None}")


def test_layernorm_closed_forms(hpt, dev):
    # constant rows: x - mean = 0 -> output = beta
    x = np.full((3, 257), 7.25, np.float32)
    g = np.linspace(0.5, 2, 257).astype(np.float32)
    b = np.linspace(-1, 1, 257).astype(np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    out = t.layernorm([257], hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev), 1e-5).numpy()
    assert np.array_equal(out, np.broadcast_to(b, out.shape))
    # two-element rows: +-1/sqrt(1 + eps/var)
    x2 = np.array([[1.0, 3.0], [-2.0, 6.0]], np.float32)
    out2 = hpt.Tensor.from_numpy(x2).to_hip(dev).layernorm([2], None, None, 1e-5).numpy()
    var = np.array([1.0, 16.0])
    want = np.stack([-1 / np.sqrt(1 + 1e-5 / var), 1 / np.sqrt(1 + 1e-5 / var)], 1)
    assert_close(out2, want, 1e-6, 1e-7, "2-element rows")
    with pytest.raises(hpt.ShapeError, match="normalized dims must match last dims"):
        hpt.Tensor.from_numpy(x2).to_hip(dev).layernorm([3])


@pytest.mark.parametrize("name", ["f16", "bf16"])
def test_layernorm_half_types(hpt, orc, dev, name):
    rng = np.random.default_rng(205)
    for shape in ([9, 4096], [5, 333], [130, 64]):
        x = (rng.standard_normal(shape) * 2).astype(np.float32)
        n = shape[-1]
        gf, bf = rng.normal(1, 0.1, n).astype(np.float32), rng.normal(0, 0.1, n).astype(np.float32)
        if name == "f16":
            cv, dt, odt, bits, tof = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32))
        else:
            cv, dt, odt, bits, tof = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32
        base, g, b = cv(x), cv(gf), cv(bf)
        tg, tb = hpt.Tensor.from_numpy(g, dt).to_hip(dev), hpt.Tensor.from_numpy(b, dt).to_hip(dev)
        for lname, ops in layouts_for(shape, rng):
            if lname != "contiguous" and ops and ops[0][0] == "permute":
                continue  # the normalised size changes under a permutation; covered by the f32 test
            t, a = upload(hpt, base, ops, dtype=dt, dev=dev)
            m = a.shape[-1]
            got = tof(t.layernorm([m], tg[:m] if m != n else tg, tb[:m] if m != n else tb, 1e-5).numpy()) if m == n else None
            if got is None:
                g2, b2 = np.ascontiguousarray(g[:m]), np.ascontiguousarray(b[:m])
                tg2, tb2 = hpt.Tensor.from_numpy(g2, dt).to_hip(dev), hpt.Tensor.from_numpy(b2, dt).to_hip(dev)
                got = tof(t.layernorm([m], tg2, tb2, 1e-5).numpy())
                want = tof(orc.layernorm(a, 1, g2, b2, 1e-5, acc=orc.ACC_F32, dtype=odt))
            else:
                want = tof(orc.layernorm(a, 1, g, b, 1e-5, acc=orc.ACC_F32, dtype=odt))
            assert_close(got, want, HALF_RTOL, half_atol(want, bits), f"layernorm {name} {shape} {lname}")


# ---- transposed views whose row blocks fit the register file: the single-pass kernel ----------
# (base shape [cols, rows] viewed as [rows, cols]; the expected plan prefix pins the kernel)
TILE_CASES = [
    # name, numpy dtype / "bf16", base shape, perm, expected plan prefix
    ("f32 rg8 one wavefront", np.float32, [40, 8192], [1, 0], "transposed-tile rows=8192 cols=40 vec=4 tpr=8 rpb=1 "),
    ("f32 rg4 paired blocks", np.float32, [4096, 2048], [1, 0], "transposed-tile rows=2048 cols=4096 vec=4 tpr=4 rpb=16 "),
    ("f16 ragged rows and cols", np.float16, [264, 16392], [1, 0], "transposed-tile rows=16392 cols=264 vec=8 tpr=8 rpb=3 "),
    ("bf16 rg8", "bf16", [1000, 16384], [1, 0], "transposed-tile rows=16384 cols=1000 vec=8 tpr=8 rpb=8 "),
    ("f64 rg4", np.float64, [3000, 1024], [1, 0], "transposed-tile rows=1024 cols=3000 vec=2 tpr=4 rpb=12 "),
    ("f32 batched", np.float32, [3, 520, 2048], [0, 2, 1], "transposed-tile rows=6144 cols=520 vec=4 tpr=8 rpb=5 "),
    ("f32 too many columns: three passes", np.float32, [4100, 2048], [1, 0], "transposed rows=2048 cols=4100 "),
]


@pytest.mark.parametrize("case", TILE_CASES, ids=[c[0] for c in TILE_CASES])
def test_transposed_tile_softmax_layernorm(hpt, orc, dev, case):
    name, npdt, shape, perm, plan = case
    rng = np.random.default_rng(206)
    x = (rng.standard_normal(shape) * 2 + rng.uniform(-3, 3, shape[:-1] + [1])).astype(np.float32)
    if npdt == "bf16":
        cv, dt, odt, bits, tof, acc = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32, orc.ACC_F32
    elif npdt == np.float16:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32)), orc.ACC_F32
    else:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(npdt)), None, None, 0, (lambda v: v), orc.ACC_F64
    base = cv(x)
    t, a = upload(hpt, base, (("permute", tuple(perm)),), dtype=dt, dev=dev)
    axis = a.ndim - 1
    assert hpt.normalize_plan(t, axis).startswith(plan), hpt.normalize_plan(t, axis)
    n = a.shape[-1]
    g, b = cv(rng.normal(1, 0.1, n).astype(np.float32)), cv(rng.normal(0, 0.1, n).astype(np.float32))
    tg, tb = hpt.Tensor.from_numpy(g, dt).to_hip(dev), hpt.Tensor.from_numpy(b, dt).to_hip(dev)

    def check(got, want, what):
        got, want = tof(got), tof(want)
        if bits:
            atol = half_atol(want, bits)
            if npdt == np.float16:
                atol = max(atol, 6e-8)
            assert_close(got, want, HALF_RTOL, atol, f"{what} {name}")
        else:
            assert_close(got, want, F32_RTOL, F32_ATOL, f"{what} {name}")

    check(t.softmax(axis).numpy(), orc.softmax(a, axis, acc=acc, dtype=odt), "softmax")
    check(t.log_softmax(axis).numpy(), orc.softmax(a, axis, log=True, acc=acc, dtype=odt), "log_softmax")
    check(t.layernorm([n], tg, tb, 1e-5).numpy(), orc.layernorm(a, 1, g, b, 1e-5, acc=acc, dtype=odt), "layernorm")
    check(t.layernorm([n], None, None, 1e-5).numpy(), orc.layernorm(a, 1, None, None, 1e-5, acc=acc, dtype=odt),
          "layernorm without gamma/beta")


def test_transposed_tile_masked_and_constant_rows(hpt, dev):
    """Closed forms through the single-pass kernel: a row with one finite entry -> one-hot; an all -inf
    row -> NaN; constant rows -> beta exactly."""
    base = np.full((96, 4096), -np.inf, np.float32)   # viewed as [4096 rows, 96 cols]
    base[5, 0] = 2.0
    base[:, 1] = np.arange(96)
    base[95, 2] = -1.0
    t = hpt.Tensor.from_numpy(base).to_hip(dev).permute([1, 0])
    assert hpt.normalize_plan(t, 1).startswith("transposed-tile")
    s = t.softmax(1).numpy()
    assert s[0, 5] == 1.0 and s[0].sum() == 1.0
    assert s[2, 95] == 1.0 and s[2].sum() == 1.0
    assert np.all(np.isnan(s[3]))
    e = np.exp(np.arange(96, dtype=np.float64) - 95)
    assert_close(s[1], e / e.sum(), F32_RTOL, F32_ATOL, "dense row")
    # (multiples of 1/4: the sum of a row is exact in f32, so the mean is too)
    c = np.repeat((np.round(np.linspace(-4, 4, 4096) * 4) / 4).astype(np.float32)[None, :], 200, 0)   # [200 cols, 4096 rows]
    g = np.linspace(0.5, 2, 200).astype(np.float32)
    b = np.linspace(-1, 1, 200).astype(np.float32)
    tc = hpt.Tensor.from_numpy(c).to_hip(dev).permute([1, 0])
    assert hpt.normalize_plan(tc, 1).startswith("transposed-tile")
    out = tc.layernorm([200], hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev), 1e-5).numpy()
    assert np.array_equal(out, np.broadcast_to(b, out.shape))


INTERLEAVED_CASES = [  # (dtype, shape, axis): softmax over the middle axis, the inner dim a divisor of the 16-byte vector
    ("f32", (600, 2048, 2), 1), ("f32", (700, 1000, 4), 1), ("f32", (3000, 200, 4), 1), ("f32", (300, 4000, 4), 1), ("f32", (3, 300, 1000, 2), 2),
    ("f32", (2000, 1001, 4), 1), ("f32", (2000, 330, 2), 1), ("f16", (900, 1000, 8), 1), ("f16", (800, 3000, 2), 1), ("f16", (4000, 300, 4), 1),
    ("f16", (256, 4096, 8), 1), ("bf16", (700, 1500, 4), 1), ("bf16", (600, 700, 8), 1), ("f64", (600, 1000, 2), 1), ("f64", (256, 4096, 2), 1),
    # inner dims of two vectors along an axis beyond 1024: neighbouring threads hold different places
    ("f32", (600, 1280, 8), 1), ("f32", (300, 2048, 8), 1), ("f32", (260, 4096, 8), 1), ("f16", (300, 1536, 16), 1), ("f16", (256, 2048, 16), 1),
    ("bf16", (1000, 1500, 16), 1), ("f64", (600, 1040, 4), 1), ("f64", (300, 2048, 4), 1), ("f32", (2, 200, 1536, 8), 2),
    # slabs of 128 KiB
    ("f32", (256, 16384, 2), 1), ("f16", (256, 6144, 4), 1),
]


@pytest.mark.parametrize("dname,shape,axis", INTERLEAVED_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_softmax_over_the_middle_axis_with_an_inner_dim_that_divides_the_vector(hpt, orc, dev, dname, shape, axis):
    """Contiguous [B, C, L] slabs with L | 16 bytes run as rows of C * L elements in registers, one (max, sum) per place in
    the vector. The inner positions get offsets far apart, so a statistic taken over the wrong place shows at once."""
    rng = np.random.default_rng(978)
    x = (rng.standard_normal(shape) * 3).astype(np.float32) + ((np.arange(shape[-1], dtype=np.float32) * 37.0) % 250.0 - 40.0)
    base = hpt.f32_to_bf16_bits(x) if dname == "bf16" else x.astype({"f16": np.float16, "f32": np.float32, "f64": np.float64}[dname])
    t, a = upload(hpt, base, dtype=hpt.bf16 if dname == "bf16" else None, dev=dev)
    assert hpt.normalize_plan(t, axis).startswith("rowreg-interleaved rows"), hpt.normalize_plan(t, axis)
    for log in (False, True):
        res = t.log_softmax(axis) if log else t.softmax(axis)
        if dname in ("f16", "bf16"):
            tof = hpt.bf16_bits_to_f32 if dname == "bf16" else (lambda v: v.astype(np.float32))
            got = tof(res.numpy())
            want = tof(orc.softmax(a, axis, log=log, acc=orc.ACC_F32, dtype=orc.BF16 if dname == "bf16" else None))
            assert_close(got, want, HALF_RTOL, max(half_atol(want, 8 if dname == "bf16" else 11), 6e-8), f"{dname} {shape} log={log}")
        elif dname == "f32":
            assert_close(res.numpy(), orc.softmax(a, axis, log=log, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"f32 {shape} log={log}")
        else:
            assert_close(res.numpy(), orc.softmax(a, axis, log=log, acc=orc.ACC_F64), 1e-12, 1e-14, f"f64 {shape} log={log}")


UNALIGNED_SPLIT_CASES = [  # (dtype, shape, axis, slice of the inner dim or None)
    ("f32", (1100, 4097), 0, None), ("f16", (1200, 4097), 0, None), ("bf16", (1030, 1025), 0, None), ("f64", (1025, 2049), 0, None),
    ("f32", (3, 1100, 515), 1, None), ("f16", (2, 1500, 1029), 1, None), ("f32", (300, 259), 0, None), ("f16", (300, 519), 0, None),
    ("f32", (1100, 4100), 0, (1, 4098)), ("f16", (1100, 2056), 0, (3, 2052)),
]


@pytest.mark.parametrize("dname,shape,axis,cut", UNALIGNED_SPLIT_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_softmax_over_an_outer_axis_with_an_odd_wide_inner_dim(hpt, orc, dev, dname, shape, axis, cut):
    """Inner rows that are not whole aligned vectors and too wide for the flat walk: lanes take unaligned vectors, the last
    lane of an inner row one that overlaps its neighbour's (both then write the same values)."""
    rng = np.random.default_rng(977)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    base = hpt.f32_to_bf16_bits(x) if dname == "bf16" else x.astype({"f16": np.float16, "f32": np.float32, "f64": np.float64}[dname])
    ops = () if cut is None else (("slice", tuple((0, n, 1) for n in shape[:-1]) + ((cut[0], cut[1], 1),)),)
    t, a = upload(hpt, base, ops, dtype=hpt.bf16 if dname == "bf16" else None, dev=dev)
    assert hpt.normalize_plan(t, axis).startswith("col-split-unaligned rows"), hpt.normalize_plan(t, axis)
    for log in (False, True):
        res = t.log_softmax(axis) if log else t.softmax(axis)
        if dname in ("f16", "bf16"):
            tof = hpt.bf16_bits_to_f32 if dname == "bf16" else (lambda v: v.astype(np.float32))
            got = tof(res.numpy())
            want = tof(orc.softmax(a, axis, log=log, acc=orc.ACC_F32, dtype=orc.BF16 if dname == "bf16" else None))
            assert_close(got, want, HALF_RTOL, max(half_atol(want, 8 if dname == "bf16" else 11), 6e-8), f"{dname} {shape} log={log}")
        elif dname == "f32":
            assert_close(res.numpy(), orc.softmax(a, axis, log=log, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"f32 {shape} log={log}")
        else:
            assert_close(res.numpy(), orc.softmax(a, axis, log=log, acc=orc.ACC_F64), 1e-12, 1e-14, f"f64 {shape} log={log}")


def test_softmax_over_axis_0_with_a_wide_inner_dim(hpt, orc, dev):
    """Inner dims wider than a workgroup's period (more than 1024 vectors) keep lanes along the inner dim:
    statistics over the axis dealt to wavefronts and workgroups, finalize, apply."""
    rng = np.random.default_rng(213)
    for npdt, shape in ((np.float32, (1500, 5000)), (np.float16, (1100, 8200)), (np.float32, (3, 1100, 4100))):
        base = (rng.standard_normal(shape) * 3).astype(npdt)
        t, a = upload(hpt, base, dev=dev)
        ax = len(shape) - 2
        assert hpt.normalize_plan(t, ax).startswith("col-split rows"), hpt.normalize_plan(t, ax)
        for log in (False, True):
            got = (t.log_softmax(ax) if log else t.softmax(ax)).numpy().astype(np.float32)
            if npdt == np.float16:
                want = orc.softmax(a, ax, log=log, acc=orc.ACC_F32).astype(np.float32)
                assert_close(got, want, HALF_RTOL, max(half_atol(want, 11), 6e-8), f"f16 {shape} log={log}")
            else:
                assert_close(got, orc.softmax(a, ax, log=log, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"f32 {shape} log={log}")


def test_log_softmax_long_columns_keep_the_absolute_tolerance(hpt, orc, dev):
    """Column softmax where one lane sums a whole column (1012 terms one after the other): the entry at the
    column's maximum is -ln(sum) ~ -0.004, so the sum must be right to better than 1e-6 relative for the
    absolute tolerance to hold; the running sum is carried in f64."""
    rng = np.random.default_rng(207)
    base = (rng.standard_normal((1012, 1266)) * 3).astype(np.float32)
    t, a = upload(hpt, base, dev=dev)
    assert hpt.normalize_plan(t, 0).startswith("col")
    got = t.log_softmax(0).numpy()
    want = orc.softmax(a, 0, log=True, acc=orc.ACC_F64)
    assert_close(got, want, F32_RTOL, F32_ATOL, "log_softmax over 1012-term columns")
    assert_close(t.softmax(0).numpy(), orc.softmax(a, 0, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, "softmax columns")


ROW_SPLIT_CASES = [
    ("a decode batch of logits", np.float32, [32, 131072], ()),
    ("one row", np.float32, [1, 65544], ()),
    ("odd length: unaligned vectors, the last one from the row's end", np.float32, [7, 20001], ()),
    ("odd length, f16 (vocabulary of 50257)", np.float16, [32, 50257], ()),
    ("odd length, bf16, one row", "bf16", [1, 128257], ()),
    ("rows at an odd offset of a wider buffer", np.float32, [6, 70001], (("slice", ((1, 6, 1), (3, 65539, 1))),)),
    ("f64 odd length", np.float64, [3, 100003], ()),
    ("rows of a wider buffer", np.float32, [12, 40000], (("slice", ((1, 11, 1), (64, 32832, 1))),)),
    ("f64", np.float64, [5, 33000], ()),
    ("f16", np.float16, [16, 65536], ()),
    ("bf16", "bf16", [9, 49152], ()),
]


@pytest.mark.parametrize("case", ROW_SPLIT_CASES, ids=[c[0] for c in ROW_SPLIT_CASES])
def test_few_long_rows_are_shared_by_workgroups(hpt, orc, dev, case):
    name, npdt, shape, ops = case
    rng = np.random.default_rng(208)
    x = (rng.standard_normal(shape) * 3 + rng.uniform(-4, 4, shape[:1] + [1])).astype(np.float32)
    if npdt == "bf16":
        cv, dt, odt, bits, tof, acc = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32, orc.ACC_F32
    elif npdt == np.float16:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32)), orc.ACC_F32
    else:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(npdt)), None, None, 0, (lambda v: v), orc.ACC_F64
    base = cv(x)
    t, a = upload(hpt, base, ops, dtype=dt, dev=dev)
    assert hpt.normalize_plan(t, 1).startswith("rowsplit"), hpt.normalize_plan(t, 1)
    n = a.shape[-1]
    g, b = cv(rng.normal(1, 0.1, n).astype(np.float32)), cv(rng.normal(0, 0.1, n).astype(np.float32))
    r = cv(rng.standard_normal(a.shape).astype(np.float32))
    tg, tb, tr = (hpt.Tensor.from_numpy(v, dt).to_hip(dev) for v in (g, b, r))

    def check(got, want, what, atol32=F32_ATOL):
        got, want = tof(got), tof(want)
        if bits:
            assert_close(got, want, HALF_RTOL, max(half_atol(want[np.isfinite(want)], bits), 6e-8), f"{what} {name}")
        else:
            assert_close(got, want, F32_RTOL, atol32, f"{what} {name}")

    ac = np.ascontiguousarray(a)
    check(t.softmax(1).numpy(), orc.softmax(ac, 1, acc=acc, dtype=odt), "softmax")
    check(t.log_softmax(-1).numpy(), orc.softmax(ac, 1, log=True, acc=acc, dtype=odt), "log_softmax")
    check(t.layernorm([n], tg, tb, 1e-5).numpy(), orc.layernorm(ac, 1, g, b, 1e-5, acc=acc, dtype=odt), "layernorm")
    check(t.layernorm([n], None, None, 1e-5).numpy(), orc.layernorm(ac, 1, None, None, 1e-5, acc=acc, dtype=odt),
          "layernorm without gamma / beta")
    if not bits:
        from oracle import elementwise as ew
        summed = ew.binary(ew.ADD, ac, r)
        check(t.add_layernorm(tr, [n], tg, tb, 1e-5).numpy(), orc.layernorm(summed, 1, g, b, 1e-5, acc=acc), "add_layernorm")


WIDE_ROW_CASES = [
    # more rows than the 512 workgroups launched: each walks two or three rows, the last ones fewer
    ("f32 2050 vectors, 1024 threads per row", np.float32, [1300, 8200]),
    ("f32 odd number of chunks", np.float32, [1100, 10000]),
    ("f64", np.float64, [1030, 4100]),
    ("f16 two vectors per thread", np.float16, [1100, 8192]),
    ("f16 eight vectors per thread", np.float16, [600, 65536]),
    ("bf16", "bf16", [1111, 16384]),
    ("bf16 rows of 128256: the raw row in registers, sixteen vectors per thread", "bf16", [530, 128256]),
    ("f16 rows of 100000: the same, the last chunks partly filled", np.float16, [515, 100000]),
    # odd lengths: aligned vectors, masked row ends (registers up to 2048 vectors, then streaming)
    ("f32 rows of 4097", np.float32, [2100, 4097]),
    ("f16 rows of 197", np.float16, [30011, 197]),
    ("f32 rows of 257 in a 3-D tensor", np.float32, [7, 1500, 257]),
    ("bf16 rows of 10001", "bf16", [700, 10001]),
    # f32 rows of 32769 ... 65536: half the row in registers, half in LDS; odd lengths shifted
    ("f32 rows of 50304: registers and LDS", np.float32, [300, 50304]),
    ("f32 rows of 50257: registers and LDS, shifted", np.float32, [270, 50257]),
    ("f32 rows of 65536: every LDS slot in use", np.float32, [140, 65536]),
    ("f32 rows of 32772: one vector beyond the registers", np.float32, [200, 32772]),
    ("f32 rows of 65501: the longest shifted row", np.float32, [131, 65501]),
    ("f32 rows of 32771 in a view that starts 29 elements into a line", np.float32, [135, 32771]),
    # layernorm rows beyond 16384 elements stream (softmax of the same rows: registers and LDS)
    ("f32 rows of 20480", np.float32, [300, 20480]),
    ("f32 rows of 16385, shifted", np.float32, [290, 16385]),
    ("f16 rows of 20480", np.float16, [300, 20480]),
    ("bf16 rows of 40001, shifted", "bf16", [280, 40001]),
    # odd lengths of two-byte rows beyond 32768: the raw row in registers over aligned vectors, masked ends
    ("f16 rows of 50257: raw row, eight vectors per thread, shifted", np.float16, [523, 50257]),
    ("bf16 rows of 65521: the longest shifted raw row", "bf16", [517, 65521]),
    ("f16 rows of 65537: registers and LDS, shifted", np.float16, [130, 65537]),
    ("bf16 rows of 131001: the longest shifted two-byte row on chip", "bf16", [133, 131001]),
    ("f16 rows of 131003: registers and LDS-direct loads, shifted", np.float16, [131, 131003]),
    # longer rows on chip: 512 threads with 48 (f32) / 32 (two-byte) vectors in registers and 16 in LDS,
    # which arrive by LDS-direct loads
    ("f32 rows of 128256: registers and LDS-direct loads", np.float32, [270, 128256]),
    ("f32 rows of 65540: one vector beyond the sixteen-vector kernel", np.float32, [133, 65540]),
    ("f32 rows of 131072: every slot in use", np.float32, [70, 131072]),
    ("f32 rows of 98308: the first LDS slots only", np.float32, [131, 98308]),
    ("f32 rows of 100277: shifted", np.float32, [261, 100277]),
    ("f32 rows of 122849: the longest shifted f32 row on chip", np.float32, [67, 122849]),
    ("f16 rows of 151936: registers and LDS-direct loads", np.float16, [263, 151936]),
    ("bf16 rows of 196608: every slot in use", "bf16", [70, 196608]),
    ("bf16 rows of 131080: one vector beyond the raw-row kernel", "bf16", [131, 131080]),
    ("f16 rows of 150001: shifted", np.float16, [259, 150001]),
    ("bf16 rows of 196545: the longest shifted two-byte row on chip", "bf16", [66, 196545]),
    ("f16 rows of 196610: streamed", np.float16, [35, 196610]),
    # the same kernel with 256 threads: odd lengths beyond 2048 vectors, and aligned rows that would leave
    # a sixteenth of a power-of-two row's slots idle
    ("f32 rows of 30522: shifted, 512 threads", np.float32, [1300, 30522]),
    ("f32 rows of 8197: the shortest such row", np.float32, [2100, 8197]),
    ("f32 rows of 28641: the longest shifted row of 256 threads", np.float32, [530, 28641]),
    ("f32 rows of 28645: shifted, 512 threads", np.float32, [530, 28645]),
    ("f32 rows of 16388: 256 threads", np.float32, [1100, 16388]),
    ("f16 rows of 32001: shifted, 256 threads", np.float16, [1100, 32001]),
    ("bf16 rows of 16392: 256 threads", "bf16", [1500, 16392]),
    ("f16 rows of 50304: 512 threads, 16 + 8 vectors", np.float16, [600, 50304]),
    ("bf16 rows of 98304: every slot of 512 threads in use", "bf16", [270, 98304]),
    # rows of 3, 5, 6 or 7 times a power of two: that many vectors per thread, no idle lanes
    ("f32 rows of 768: 64 threads x 3 vectors", np.float32, [5003, 768]),
    ("f32 rows of 1280: 64 x 5", np.float32, [4100, 1280]),
    ("f32 rows of 1536: 128 x 3", np.float32, [2300, 1536]),
    ("f32 rows of 2560: 128 x 5", np.float32, [2100, 2560]),
    ("f32 rows of 3584: softmax 128 x 7", np.float32, [2051, 3584]),
    ("f32 rows of 6144: softmax 256 x 6, layernorm 512 x 3 with prefetch", np.float32, [1100, 6144]),
    ("f32 rows of 12288: 512 x 6 with prefetch", np.float32, [700, 12288]),
    ("f64 rows of 1536: 256 x 3", np.float64, [1500, 1536]),
    ("f16 rows of 768: 32 x 3", np.float16, [9001, 768]),
    ("f16 rows of 3072: 128 x 3", np.float16, [2101, 3072]),
    ("bf16 rows of 2560: 128 x 3, the last vectors of each thread empty", "bf16", [2300, 2560]),
    ("f16 rows of 5120: softmax 256 x 3, layernorm 128 x 5 with gamma / beta in LDS", np.float16, [1300, 5120]),
    ("bf16 rows of 1152: layernorm 32 x 5 with gamma / beta in LDS", "bf16", [9001, 1152]),
    ("f16 rows of 10240: layernorm 256 x 5 with gamma / beta in LDS", np.float16, [1100, 10240]),
    ("bf16 rows of 12288: softmax 512 x 3", "bf16", [600, 12288]),
    # odd lengths with 3 or 5 vectors per thread (softmax; layernorm keeps powers of two there)
    ("f16 rows of 577: shifted, 32 x 3", np.float16, [9000, 577]),
    ("bf16 rows of 1500 (8-byte row starts): shifted, 64 x 3", "bf16", [4400, 1500]),
    ("f32 rows of 2051: shifted, 128 x 5", np.float32, [2300, 2051]),
    ("f32 rows of 3001: shifted, 256 x 3", np.float32, [2100, 3001]),
    # two-byte layernorm rows of 513 ... 1024 shifted vectors: 512 threads, two vectors each, rows walked
    ("f16 rows of 4097: layernorm from registers, 512 threads", np.float16, [2100, 4097]),
    ("bf16 rows of 8185: the longest such row", "bf16", [1500, 8185]),
    ("f16 rows of 6148 (rows start on 8-byte boundaries)", np.float16, [1300, 6148]),
]


@pytest.mark.parametrize("case", WIDE_ROW_CASES, ids=[c[0] for c in WIDE_ROW_CASES])
def test_long_and_odd_rows_walked_with_prefetch(hpt, orc, dev, case):
    """Rows of 512 / 1024 threads are walked by at most 512 workgroups that issue the next row's loads
    before the current row's statistics; odd-length rows move aligned vectors with masked ends. Every
    row must come out as from the plain kernels: first, middle and last rows of the walk alike."""
    name, npdt, shape = case
    rng = np.random.default_rng(209)
    x = (rng.standard_normal(shape) * 2 + rng.uniform(-3, 3, shape[:-1] + [1])).astype(np.float32)
    if npdt == "bf16":
        cv, dt, odt, bits, tof, acc = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32, orc.ACC_F32
    elif npdt == np.float16:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32)), orc.ACC_F32
    else:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(npdt)), None, None, 0, (lambda v: v), orc.ACC_F64
    a = cv(x)
    t = hpt.Tensor.from_numpy(a, dt).to_hip(dev)
    n = shape[-1]
    ax = len(shape) - 1
    g, b = cv(rng.normal(1, 0.1, n).astype(np.float32)), cv(rng.normal(0, 0.1, n).astype(np.float32))
    tg, tb = (hpt.Tensor.from_numpy(v, dt).to_hip(dev) for v in (g, b))

    def check(got, want, what, atol32=F32_ATOL):
        got, want = tof(got), tof(want)
        if bits:
            assert_close(got, want, HALF_RTOL, max(half_atol(want[np.isfinite(want)], bits), 6e-8), f"{what} {name}")
        else:
            assert_close(got, want, F32_RTOL, atol32, f"{what} {name}")

    check(t.softmax(ax).numpy(), orc.softmax(a, ax, acc=acc, dtype=odt), "softmax")
    check(t.log_softmax(-1).numpy(), orc.softmax(a, ax, log=True, acc=acc, dtype=odt), "log_softmax")
    check(t.layernorm([n], tg, tb, 1e-5).numpy(), orc.layernorm(a, 1, g, b, 1e-5, acc=acc, dtype=odt), "layernorm")
    if not bits:
        from oracle import elementwise as ew
        r = cv(rng.standard_normal(shape).astype(np.float32))
        tr = hpt.Tensor.from_numpy(r, dt).to_hip(dev)
        check(t.add_layernorm(tr, [n], tg, tb, 1e-5).numpy(), orc.layernorm(ew.binary(ew.ADD, a, r), 1, g, b, 1e-5, acc=acc),
              "add_layernorm")


SHORT_ROW_CASES = [
    ("f32 rows of 3", np.float32, [400001, 3]),
    ("f32 rows of 8 (whole vectors)", np.float32, [140001, 8]),
    ("f32 rows of 33 in a 3-D tensor", np.float32, [11, 3001, 33]),
    ("f32 rows of 100", np.float32, [12001, 100]),
    ("f64 rows of 65", np.float64, [9001, 65]),
    ("f16 rows of 33", np.float16, [70001, 33]),
    ("f16 rows of 64 (whole vectors)", np.float16, [40001, 64]),
    ("bf16 rows of 197", "bf16", [12001, 197]),
    ("f32 rows of 511", np.float32, [2501, 511]),
]


@pytest.mark.parametrize("case", SHORT_ROW_CASES, ids=[c[0] for c in SHORT_ROW_CASES])
def test_short_rows_normalised_in_lds_tiles(hpt, orc, dev, case):
    """Short rows laid back to back go through 16 KiB LDS tiles (aligned vectors in and out whatever
    the row length). The row counts leave a partial last tile and a partial last vector; masked and
    constant rows keep their closed forms."""
    name, npdt, shape = case
    rng = np.random.default_rng(210)
    x = (rng.standard_normal(shape) * 2 + rng.uniform(-3, 3, shape[:-1] + [1])).astype(np.float32)
    if npdt == "bf16":
        cv, dt, odt, bits, tof, acc = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32, orc.ACC_F32
    elif npdt == np.float16:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32)), orc.ACC_F32
    else:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(npdt)), None, None, 0, (lambda v: v), orc.ACC_F64
    x.reshape(-1, shape[-1])[5, :] = 1.25           # a constant row
    x.reshape(-1, shape[-1])[7, 1:] = -np.inf       # a row with one finite entry
    a = cv(x)
    t = hpt.Tensor.from_numpy(a, dt).to_hip(dev)
    n = shape[-1]
    ax = len(shape) - 1
    assert "+tile" in hpt.normalize_plan(t, ax), hpt.normalize_plan(t, ax)
    g, b = cv(rng.normal(1, 0.1, n).astype(np.float32)), cv(rng.normal(0, 0.1, n).astype(np.float32))
    tg, tb = (hpt.Tensor.from_numpy(v, dt).to_hip(dev) for v in (g, b))

    def check(got, want, what, atol32=F32_ATOL):
        got, want = tof(got), tof(want)
        if bits:
            assert_close(got, want, HALF_RTOL, max(half_atol(want[np.isfinite(want)], bits), 6e-8), f"{what} {name}")
        else:
            assert_close(got, want, F32_RTOL, atol32, f"{what} {name}")

    sm = t.softmax(ax).numpy()
    check(sm, orc.softmax(a, ax, acc=acc, dtype=odt), "softmax")
    smf = tof(sm).reshape(-1, n)
    assert np.all(smf[7, 0] == 1.0) and np.all(smf[7, 1:] == 0.0), "one finite entry -> exactly (1, 0, 0, ...)"
    check(t.log_softmax(-1).numpy(), orc.softmax(a, ax, log=True, acc=acc, dtype=odt), "log_softmax")
    fin = np.where(np.isfinite(x), x, 0.0).astype(np.float32)   # layernorm of -inf is NaN: compare finite rows
    af = cv(fin)
    tf_ = hpt.Tensor.from_numpy(af, dt).to_hip(dev)
    if "+tile" in hpt.normalize_plan(tf_, 0, 1):
        ln = tf_.layernorm([n], tg, tb, 1e-5).numpy()
        check(ln, orc.layernorm(af, 1, g, b, 1e-5, acc=acc, dtype=odt), "layernorm")
        assert np.array_equal(tof(ln).reshape(-1, n)[5], tof(b)), "constant row -> beta exactly"
        check(tf_.layernorm([n], None, None, 1e-5).numpy(), orc.layernorm(af, 1, None, None, 1e-5, acc=acc, dtype=odt),
              "layernorm without gamma / beta")


FLAT_COLUMN_CASES = [
    ("f32 [N, 3] axis 0", np.float32, [1000001, 3], 0),
    ("f16 [N, 8] axis 0", np.float16, [600001, 8], 0),
    ("f32 [N, 33] axis 0", np.float32, [70001, 33], 0),
    ("bf16 [N, 100] axis 0", "bf16", [50001, 100], 0),
    ("f16 [N, 257] axis 0", np.float16, [20001, 257], 0),
    ("f32 [3, N, 5] axis 1", np.float32, [3, 500000, 5], 1),
    ("f64 [N, 7] axis 0", np.float64, [200001, 7], 0),
    # batch slabs that start off 16-byte boundaries: the same walk with unaligned vectors
    ("f16 [257, 13988, 7] axis 1 (misaligned slabs)", np.float16, [257, 13988, 7], 1),
    ("f32 [31, 70001, 3] axis 1 (misaligned slabs)", np.float32, [31, 70001, 3], 1),
    # many small slabs: fewer threads per slab, so that each is still worth two periods
    ("f32 [300, 6000, 3] axis 1 (72 KiB slabs)", np.float32, [300, 6000, 3], 1),
    ("f16 [200, 5031, 7] axis 1 (small misaligned slabs)", np.float16, [200, 5031, 7], 1),
]


@pytest.mark.parametrize("case", FLAT_COLUMN_CASES, ids=[c[0] for c in FLAT_COLUMN_CASES])
def test_softmax_over_a_long_axis_with_a_narrow_inner_dim(hpt, orc, dev, case):
    """softmax over axis 0 of [N, 3]: lanes along the inner dim would idle, so the slab is walked as a
    flat array (statistics, finalize, apply). A column that is all -inf comes out NaN, a column with
    one finite entry comes out exactly one-hot."""
    name, npdt, shape, axis = case
    rng = np.random.default_rng(211)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    idx = [slice(None)] * len(shape)
    idx[-1] = 1
    x[tuple(idx)] = -np.inf                                   # inner index 1: nothing finite
    idx[-1] = 2
    x[tuple(idx)] = -np.inf
    one = list(idx)
    one[axis] = min(12345, shape[axis] - 1)
    x[tuple(one)] = 0.5                                       # inner index 2: one finite entry
    if npdt == "bf16":
        cv, dt, odt, bits, tof, acc = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32, orc.ACC_F32
    elif npdt == np.float16:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32)), orc.ACC_F32
    else:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(npdt)), None, None, 0, (lambda v: v), orc.ACC_F64
    a = cv(x)
    t = hpt.Tensor.from_numpy(a, dt).to_hip(dev)
    assert hpt.normalize_plan(t, axis).startswith("col-split-flat"), hpt.normalize_plan(t, axis)
    for log in (False, True):
        got = tof((t.log_softmax(axis) if log else t.softmax(axis)).numpy())
        want = tof(orc.softmax(a, axis, log=log, acc=acc, dtype=odt))
        idx[-1] = 1
        assert np.all(np.isnan(got[tuple(idx)])), f"{name}: a column without a finite entry is NaN"
        if not log:
            idx[-1] = 2
            col = got[tuple(idx)]
            assert np.count_nonzero(col) == col.size // shape[axis] and np.all(col[col != 0] == 1.0), f"{name}: one-hot"
        keep = np.ones(shape[-1], bool)
        keep[1] = False
        g, w = got[..., keep], want[..., keep]
        if bits:
            assert_close(g, w, HALF_RTOL, max(half_atol(w[np.isfinite(w)], bits), 6e-8), f"{name} log={log}")
        else:
            assert_close(g, w, F32_RTOL, F32_ATOL, f"{name} log={log}")


CHANNEL_CASES = [
    ("f32 [4, 21, 128, 128] axis 1", np.float32, [4, 21, 128, 128], 1),
    ("f16 [2, 3, 40000] axis 1", np.float16, [2, 3, 40000], 1),
    ("f32 [32, 70000] axis 0", np.float32, [32, 70000], 0),
    ("bf16 [3, 64, 30000] axis 1", "bf16", [3, 64, 30000], 1),
    ("f32 [2, 10, 33333] axis 1 (odd inner length)", np.float32, [2, 10, 33333], 1),
    ("f64 [2, 30, 40000] axis 1", np.float64, [2, 30, 40000], 1),
    # longer axes: 2 ... 16 thread rows share an inner position and meet in LDS
    ("f32 [24, 128, 56, 56] axis 1 (8 thread rows)", np.float32, [24, 128, 56, 56], 1),
    ("f16 [2, 300, 40000] axis 1 (16 thread rows)", np.float16, [2, 300, 40000], 1),
    ("f32 [600, 66001] axis 0 (single elements, 16 thread rows)", np.float32, [600, 66001], 0),
    ("f64 [3, 100, 30000] axis 1", np.float64, [3, 100, 30000], 1),
    # inner dims that are not whole vectors: unaligned vectors, the last one of a row from its end
    ("f16 [3, 7, 33, 1361] axis 1 (odd inner length 44913)", np.float16, [3, 7, 33, 1361], 1),
    ("bf16 [21, 33, 3631] axis 0 (two thread rows)", "bf16", [21, 33, 3631], 0),
    ("f32 [2, 21, 213, 211] axis 1", np.float32, [2, 21, 213, 211], 1),
    ("f64 [2, 9, 70001] axis 1", np.float64, [2, 9, 70001], 1),
    ("f16 [300, 70001] axis 0 (16 thread rows)", np.float16, [300, 70001], 0),
    # a narrow inner dim of whole PAIRS of two-byte elements: 64 four-byte loads per thread
    ("f16 [300, 300, 18] axis 1 (pairs, 8 thread rows)", np.float16, [300, 300, 18], 1),
    ("bf16 [200, 512, 10] axis 1 (single two-byte elements, 8 thread rows)", "bf16", [200, 512, 10], 1),
    ("f16 [500, 100, 14] axis 1 (single two-byte elements, 2 thread rows)", np.float16, [500, 100, 14], 1),
]


GROUP_CASES = [
    ("f32 [60000, 16, 2] axis 1", np.float32, [60000, 16, 2], 1),
    ("f16 [600, 128, 4, 64] axis 2 (heads)", np.float16, [600, 128, 4, 64], 2),
    ("f16 [3, 65537, 4, 12] axis 2", np.float16, [3, 65537, 4, 12], 2),
    ("bf16 [8191, 129, 8, 3] axis 2", "bf16", [8191, 129, 8, 3], 2),
    ("f32 [700001, 2, 3] axis 1", np.float32, [700001, 2, 3], 1),
    ("f16 [4097, 12, 96, 5] axis 2 (a long axis in a small group)", np.float16, [4097, 12, 96, 5], 2),
    ("f64 [90001, 5, 7] axis 1", np.float64, [90001, 5, 7], 1),
]


SLAB_CASES = [
    ("f16 [900, 1001, 3] axis 1", np.float16, [900, 1001, 3], 1),
    ("f32 [300, 1093, 5] axis 1 (slabs off 16-byte boundaries)", np.float32, [300, 1093, 5], 1),
    ("bf16 [260, 2730, 12] axis 1 (64 KiB slabs)", "bf16", [260, 2730, 12], 1),
    ("f32 [1200, 501, 2] axis 1 (slabs of half vectors)", np.float32, [1200, 501, 2], 1),
    ("f64 [300, 1101, 3] axis 1", np.float64, [300, 1101, 3], 1),
    ("f16 [2, 300, 2049, 7] axis 2 (odd slab size)", np.float16, [2, 300, 2049, 7], 2),
    # four-byte inner dims up to 11 elements that are not whole vectors
    ("f32 [600, 513, 7] axis 1", np.float32, [600, 513, 7], 1),
    ("f32 [500, 300, 11] axis 1", np.float32, [500, 300, 11], 1),
    ("f32 [8000, 101, 6] axis 1 (short axis)", np.float32, [8000, 101, 6], 1),
]


INTERLEAVED_SLAB_CASES = [  # an inner dim that divides the vector: the slab is a row in registers
    ("f32 [1200, 500, 2] axis 1", np.float32, [1200, 500, 2], 1),
    ("f16 [700, 900, 4] axis 1", np.float16, [700, 900, 4], 1),
    ("bf16 [2, 300, 2048, 8] axis 2", "bf16", [2, 300, 2048, 8], 2),
    ("f64 [300, 1100, 2] axis 1", np.float64, [300, 1100, 2], 1),
    ("bf16 [260, 2047, 16] axis 1 (64 KiB slabs, two vectors side by side)", "bf16", [260, 2047, 16], 1),
]


MODULAR_SLAB_CASES = [  # an inner dim of 3, 5, 6, 7 and slabs of whole vectors: the slab is a row held by lanes in multiples of the inner dim
    ("f16 [900, 1000, 3] axis 1", np.float16, [900, 1000, 3], 1),
    ("f32 [300, 1092, 5] axis 1", np.float32, [300, 1092, 5], 1),
    ("f64 [300, 1100, 3] axis 1", np.float64, [300, 1100, 3], 1),
    ("f32 [600, 512, 7] axis 1", np.float32, [600, 512, 7], 1),
    ("f32 [8000, 100, 6] axis 1 (short axis, 32 lanes per row)", np.float32, [8000, 100, 6], 1),
    ("bf16 [2, 300, 1024, 7] axis 2", "bf16", [2, 300, 1024, 7], 2),
    ("f32 [300, 8000, 3] axis 1 (rows of 1024 threads)", np.float32, [300, 8000, 3], 1),
    ("f16 [700, 4000, 6] axis 1", np.float16, [700, 4000, 6], 1),
    ("f32 [2000, 1000, 3] axis 1", np.float32, [2000, 1000, 3], 1),
    ("f64 [400, 1000, 6] axis 1 (three two-element vectors per inner row)", np.float64, [400, 1000, 6], 1),
]


ROW_SLAB_CASES = INTERLEAVED_SLAB_CASES + MODULAR_SLAB_CASES


@pytest.mark.parametrize("case", CHANNEL_CASES + GROUP_CASES + SLAB_CASES + ROW_SLAB_CASES,
                         ids=[c[0] for c in CHANNEL_CASES + GROUP_CASES + SLAB_CASES + ROW_SLAB_CASES])
def test_softmax_over_a_short_strided_axis_in_registers(hpt, orc, dev, case):
    """softmax over the channels of [B, C, H, W], C <= 64: every thread keeps the whole axis of its
    inner positions in registers (one read, one write). Small [C, L] groups laid back to back go
    through LDS tiles instead (one lane per inner position of a group), mid-sized slabs with a narrow
    inner dim one workgroup per slab (groups of lanes per column)."""
    name, npdt, shape, axis = case
    rng = np.random.default_rng(212)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    idx = [0] * len(shape)
    idx[axis], idx[-1] = slice(None), 1
    x[tuple(idx)] = -np.inf                      # one inner position without a finite entry
    if npdt == "bf16":
        cv, dt, odt, bits, tof, acc = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32, orc.ACC_F32
    elif npdt == np.float16:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(np.float16)), None, None, 11, (lambda v: v.astype(np.float32)), orc.ACC_F32
    else:
        cv, dt, odt, bits, tof, acc = (lambda v: v.astype(npdt)), None, None, 0, (lambda v: v), orc.ACC_F64
    a = cv(x)
    t = hpt.Tensor.from_numpy(a, dt).to_hip(dev)
    want_plan = ("col-group-tile" if case in GROUP_CASES else "col-slab" if case in SLAB_CASES else
                 "rowreg-interleaved" if case in INTERLEAVED_SLAB_CASES else "rowreg-modular" if case in MODULAR_SLAB_CASES else "col-reg")
    assert hpt.normalize_plan(t, axis).startswith(want_plan), hpt.normalize_plan(t, axis)
    for log in (False, True):
        got = tof((t.log_softmax(axis) if log else t.softmax(axis)).numpy())
        want = tof(orc.softmax(a, axis, log=log, acc=acc, dtype=odt))
        dead = np.isnan(want)
        assert dead.any() and np.all(np.isnan(got[dead])), f"{name}: no finite entry -> NaN"
        g, w = np.where(dead, 0, got), np.where(dead, 0, want)
        if bits:
            assert_close(g, w, HALF_RTOL, max(half_atol(w[np.isfinite(w)], bits), 6e-8), f"{name} log={log}")
        else:
            assert_close(g, w, F32_RTOL, F32_ATOL, f"{name} log={log}")


def test_special_values_on_the_large_shape_kernels(hpt, orc, dev):
    """+inf and NaN entries on the kernels only large shapes reach: a row / column with +inf or NaN
    comes out NaN where the oracle says so, everything else matches."""
    rng = np.random.default_rng(213)
    for shape, axis, plan in (((60001, 33), 1, "rowreg+tile"), ((1100, 8192), 1, "rowreg rows"), ((1100, 8200), 1, "rowreg-lds rows"), ((500001, 5), 0, "col-split-flat"),
                              ((4, 21, 128, 128), 1, "col-reg"), ((300, 70000), 1, "rowreg-lds rows"), ((300, 70001), 1, "rowreg-lds-shift"),
                              ((130, 140000), 1, "rowstream"), ((2100, 4097), 1, "rowreg-shift")):
        x = (rng.standard_normal(shape) * 2).astype(np.float32)
        flat = x.reshape(-1)
        flat[rng.integers(0, flat.size, 40)] = np.inf
        flat[rng.integers(0, flat.size, 40)] = np.nan
        flat[rng.integers(0, flat.size, flat.size // 100)] = -np.inf
        t = hpt.Tensor.from_numpy(x).to_hip(dev)
        assert hpt.normalize_plan(t, axis).startswith(plan), hpt.normalize_plan(t, axis)
        for log in (False, True):
            got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
            with np.errstate(invalid="ignore", over="ignore"):
                want = orc.softmax(x, axis, log=log, acc=orc.ACC_F64)
            assert np.array_equal(np.isnan(got), np.isnan(want)), f"{shape} axis={axis} log={log}: NaN pattern"
            assert_close(got, want, F32_RTOL, F32_ATOL, f"{shape} axis={axis} log={log}")


def test_half_rows_of_millions_of_elements_against_the_f64_truth(hpt, orc, dev):
    """f16 layernorm over all four dims of [63, 50, 53, 37] permuted (1, 2, 0, 3) — one strided row of
    6 177 150 elements, the case a randomised run once flagged — and its bf16 twin, plus softmax and a
    full sum of the same row. Rows this long are checked against the f64 accumulation rounded once:
    the sequential-f32 oracle mode is itself ~0.4 % off here (shown on the host in
    tests/test_oracle_numerics.py::test_sequential_f32_accumulation_is_no_truth_for_long_half_rows)."""
    from util import half_acc
    rng = np.random.default_rng(0)
    shape = [63, 50, 53, 37]
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    gf = rng.normal(1, 0.1, [50, 53, 63, 37]).astype(np.float32)
    bf = rng.normal(0, 0.1, [50, 53, 63, 37]).astype(np.float32)
    for bits in (11, 8):
        if bits == 8:
            cv, dt, odt, tof = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, hpt.bf16_bits_to_f32
        else:
            cv, dt, odt, tof = (lambda v: v.astype(np.float16)), None, None, (lambda v: v.astype(np.float32))
        base, g, b = cv(x), cv(gf), cv(bf)
        t = hpt.Tensor.from_numpy(base, dt).to_hip(dev).permute([1, 2, 0, 3])
        a = base.transpose(1, 2, 0, 3)
        acc = half_acc(orc, a.size)
        assert acc == orc.ACC_F64
        tg, tb = hpt.Tensor.from_numpy(g, dt).to_hip(dev), hpt.Tensor.from_numpy(b, dt).to_hip(dev)
        got = tof(t.layernorm(list(a.shape), tg, tb, 1e-5).numpy())
        want = tof(orc.layernorm(a, 4, g, b, 1e-5, acc=acc, dtype=odt))
        # one rounding of the result apart from the oracle: an ulp of the half type, nowhere more
        assert_close(got, want, 2.0 ** -(bits - 1), 2.0 ** -bits * 2.0 ** -6, f"layernorm of one 6M-element row, {bits} bits")
        # and the row's own statistics, which is where a drifting accumulation would show
        m = float(tof(t.mean([0, 1, 2, 3]).numpy())[0])
        xd = tof(a).astype(np.float64)
        assert abs(m - xd.mean()) < 2.0 ** -bits * max(abs(xd.mean()), 2.0 ** -14) + 1e-6
        if bits == 8:   # (2.5e7 is beyond f16's range)
            ss = float(tof(t.sum_square([0, 1, 2, 3]).numpy())[0])
            assert abs(ss / (xd * xd).sum() - 1) < 2.0 ** -bits
        got = tof(t.softmax(3).numpy())
        want = tof(orc.softmax(a, 3, acc=orc.ACC_F32, dtype=odt))
        assert_close(got, want, HALF_RTOL, max(half_atol(want, bits), 6e-8), f"softmax(3), {bits} bits")


@pytest.mark.parametrize("seed", range(4))
def test_long_rows_of_random_length_and_alignment(hpt, orc, dev, seed):
    """softmax / log_softmax over rows of 2049 ... 50000 vectors whose length, row pitch and first element
    are drawn at random: windows [r0:, c0:c1] of a parent matrix, so rows start anywhere on the 16-byte
    grid or off it, input and output rows are misaligned alike or not, and every plan of such rows is
    reached: registers + LDS (aligned and shifted, 256 and 512 threads), the raw-row kernel, the
    streaming kernel (aligned, shifted, element-wise)."""
    rng = np.random.default_rng(4200 + seed)
    seen = set()
    for it in range(14):
        kind = ("f32", "f16", "bf16")[int(rng.integers(0, 3))]
        vec = 4 if kind == "f32" else 8
        cols = int(rng.integers(2049 * vec, 50000 * vec // (2 if kind == "f32" else 3)))
        if rng.integers(0, 3) == 0:
            cols -= cols % vec                      # whole vectors
        rows = int(rng.integers(129, 150))     # (fewer rows are shared among workgroups: another plan)
        lead, tail = (int(rng.integers(0, 2 * vec)) if rng.integers(0, 2) else 0 for _ in range(2))
        if rng.integers(0, 3) == 0:
            tail += -(lead + cols + tail) % vec    # a pitch of whole vectors: every row misaligned alike
        x = (rng.standard_normal((rows + 1, lead + cols + tail)) * 2).astype(np.float32)
        if kind == "bf16":
            a, dt, odt, bits, tof = hpt.f32_to_bf16_bits(x), hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32
        elif kind == "f16":
            a, dt, odt, bits, tof = x.astype(np.float16), None, None, 11, (lambda v: v.astype(np.float32))
        else:
            a, dt, odt, bits, tof = x, None, None, 0, (lambda v: v)
        t = hpt.Tensor.from_numpy(a, dt).to_hip(dev)[1:, lead:lead + cols]
        view = a[1:, lead:lead + cols]
        plan = hpt.normalize_plan(t, 1).split(" ")[0]
        seen.add(plan)
        what = f"seed={seed} case={it} {kind} rows={rows} cols={cols} lead={lead} pitch={a.shape[1]} plan={plan}"
        acc = orc.ACC_F32 if bits else orc.ACC_F64
        for log in (False, True):
            got = tof((t.log_softmax(1) if log else t.softmax(1)).numpy())
            want = tof(orc.softmax(view, 1, log=log, acc=acc, dtype=odt))
            if bits:
                assert_close(got, want, HALF_RTOL, max(half_atol(want[np.isfinite(want)], bits), 6e-8), f"log={log} {what}")
            else:
                assert_close(got, want, F32_RTOL, 2 * F32_ATOL if log else F32_ATOL, f"log={log} {what}")
    assert any(p.startswith("rowreg-lds") for p in seen), seen


WIDE_AXIS_CASES = [
    # four-byte axes of 257 ... 512 elements with a wide inner dim: 128 registers of raw values per thread
    ([2, 512, 2048], 1), ([3, 257, 1024], 1), ([384, 8192], 0), ([1, 300, 4096], 1), ([5, 512, 64, 32], 1),
    # 129 ... 256 elements: the same registers over eight thread rows
    ([16, 200, 1024], 1), ([256, 8192], 0), ([2, 129, 4096], 1), ([64, 256, 16, 8], 1),
]


@pytest.mark.parametrize("case", WIDE_AXIS_CASES, ids=[str(c[0]) for c in WIDE_AXIS_CASES])
def test_softmax_over_a_strided_axis_of_up_to_512_in_registers(hpt, orc, dev, case):
    shape, axis = case
    rng = np.random.default_rng(611)
    x = (rng.standard_normal(shape) * 4).astype(np.float32)
    x[..., 0] += 30  # one inner position with a dominating band: the maximum matters
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    plan = hpt.normalize_plan(t, axis)
    assert plan.startswith("col-reg") and "nchunk=32" in plan, plan
    for log in (False, True):
        got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
        assert_close(got, orc.softmax(x, axis, log=log, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"{shape} axis={axis} log={log}")
    # -inf entries and a position whose whole axis is -inf (NaN, as the reference's x - max gives)
    x[..., 5] = -np.inf
    idx = [slice(None)] * len(shape)
    idx[axis] = slice(0, shape[axis] // 2)
    x[tuple(idx)][..., 7] = -np.inf
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    got = t.softmax(axis).numpy()
    want = orc.softmax(x, axis, acc=orc.ACC_F64)
    assert_close(got, want, F32_RTOL, F32_ATOL, f"{shape} axis={axis} with -inf")
    assert np.isnan(got[..., 5]).all()


DOMINANT_CASES = [
    # (shape, axis, transposed view, first word of the plan)
    ([4096, 4096], 1, False, "rowreg"), ([8192, 1000], 1, False, "rowreg"), ([1000000, 8], 1, False, "rowreg+tile"),
    ([64, 65536], 1, False, "rowsplit"), ([8, 400000], 1, False, "rowsplit"),
    ([17310, 256, 2], 1, False, "col-group-tile"), ([100000, 16, 2], 1, False, "col-group-tile"),
    ([2048, 2047, 2], 1, False, "col-slab"), ([512, 1001, 3], 1, False, "col-slab"), ([512, 1000, 3], 1, False, "rowreg-modular"), ([2048, 2048, 2], 1, False, "rowreg-interleaved"),
    ([8, 512, 4096], 1, False, "col-reg"), ([4, 128, 3136], 1, False, "col-reg"), ([64, 64, 3000], 1, False, "col-reg"),
    ([200000, 3], 0, False, "col-split"), ([100000, 33], 0, False, "col-split-flat"), ([32768, 1024], 0, False, "col-split-flat"),
    ([4096, 4096], 1, True, "transposed-tile"),
]


@pytest.mark.parametrize("case", DOMINANT_CASES, ids=[f"{c[3]}-{'x'.join(map(str, c[0]))}" for c in DOMINANT_CASES])
def test_log_softmax_with_a_dominating_first_element(hpt, orc, dev, case):
    """The FIRST element along the axis dominates (+14): the sum of exponentials is 1 + many tiny terms, so a
    running f32 sum sits just above 1 for the whole walk and loses up to 6e-8 per addition, and the entry at the
    maximum, -ln(sum), is close to zero where only the absolute tolerance helps. One case per kernel family."""
    shape, axis, transposed, family = case
    rng = np.random.default_rng(1)
    x = rng.standard_normal(shape).astype(np.float32)
    idx = [slice(None)] * len(shape)
    idx[axis] = 0
    x[tuple(idx)] += 14
    if transposed:
        t = hpt.Tensor.from_numpy(np.ascontiguousarray(x.T)).to_hip(dev).permute([1, 0])
    else:
        t = hpt.Tensor.from_numpy(x).to_hip(dev)
    assert hpt.normalize_plan(t, axis).split(" ")[0] == family, hpt.normalize_plan(t, axis)
    for log in (True, False):
        got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
        assert_close(got, orc.softmax(x, axis, log=log, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"{shape} axis={axis} log={log}")


OFFSET_CASES = [
    # (shape, view, first word of the plan)
    ([8192, 4096], None, "rowreg"), ([200001, 3], "drop", "rowreg"), ([1000000, 8], None, "rowreg+tile"), ([100000, 33], None, "rowreg+tile"),
    ([4096, 4096], "T", "transposed-tile"), ([64, 65536], None, "rowsplit"), ([640, 50304], None, "rowstream"),
    ([512, 4097], None, "rowreg-shift"), ([1024, 12288], None, "rowreg"),
]


@pytest.mark.parametrize("case", OFFSET_CASES, ids=[f"{c[2]}-{'x'.join(map(str, c[0]))}" for c in OFFSET_CASES])
def test_layernorm_of_rows_whose_offset_dwarfs_their_spread(hpt, orc, dev, case):
    """Rows of 1000 + N(0, 1): the mean must be right to a few 1e-6 of the SPREAD, i.e. 1e-9 of its own size,
    which needs the lanes' own sums in f64 as well as the sum across lanes. (Three-element rows also meet rows
    whose elements nearly coincide, where 1 / sqrt(var + eps) multiplies the mean's error by up to 316.)"""
    shape, view, family = case
    rng = np.random.default_rng(2)
    for off in (0.0, 1000.0):
        x = (rng.standard_normal(shape) * (3 if shape[-1] == 3 else 1) + off).astype(np.float32)
        if view == "T":
            t = hpt.Tensor.from_numpy(np.ascontiguousarray(x.T)).to_hip(dev).permute([1, 0])
            a = x
        elif view == "drop":  # rows that start off a 16-byte boundary: one lane per row
            t = hpt.Tensor.from_numpy(x).to_hip(dev)[1:, :]
            a = np.ascontiguousarray(x[1:])
        else:
            t = hpt.Tensor.from_numpy(x).to_hip(dev)
            a = x
        n = shape[-1]
        assert hpt.normalize_plan(t, 0, 1).split(" ")[0] == family, hpt.normalize_plan(t, 0, 1)
        got = t.layernorm([n], None, None, 1e-5).numpy()
        assert_close(got, orc.layernorm(a, 1, None, None, 1e-5, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, f"{shape} offset {off}")


L2GB_CASES = [
    # (dtype, shape, plan words) - layernorm rows too long for gamma / beta beside them in registers or LDS
    (np.float32, [300, 16388], "tpr=1024 rpb=1 nchunk=5 "), (np.float32, [600, 18944], "tpr=1024 rpb=1 nchunk=5 "), (np.float32, [520, 28672], "tpr=1024 rpb=1 nchunk=7 "),
    (np.float32, [257, 32768], "tpr=1024 rpb=1 nchunk=8 "), (np.float16, [600, 18944], "tpr=512 rpb=1 nchunk=5 "), ("bf16", [300, 25600], "tpr=1024 rpb=1 nchunk=4 "),
    (np.float16, [515, 49152], "tpr=1024 rpb=1 nchunk=6 "), (np.float64, [300, 8194], "tpr=1024 rpb=1 nchunk=5 "), (np.float64, [513, 16384], "tpr=1024 rpb=1 nchunk=8 "),
    (np.float32, [1100, 20480], "tpr=1024 rpb=1 nchunk=5 "),  # more rows than workgroups: they walk the rows and prefetch
]


@pytest.mark.parametrize("case", L2GB_CASES, ids=[f"{getattr(c[0], '__name__', c[0])}-{'x'.join(map(str, c[1]))}" for c in L2GB_CASES])
def test_layernorm_rows_with_gamma_beta_read_from_l2(hpt, orc, dev, case):
    npdt, shape, words = case
    rng = np.random.default_rng(811)
    x = (rng.standard_normal(shape) * 2 + 1).astype(np.float32)
    n = shape[-1]
    g32 = rng.normal(1, 0.2, n).astype(np.float32)
    b32 = rng.normal(0, 0.3, n).astype(np.float32)
    if npdt == "bf16":
        conv, dt, odt, bits, tof = hpt.f32_to_bf16_bits, hpt.bf16, orc.BF16, 8, hpt.bf16_bits_to_f32
    else:
        conv, dt, odt, bits, tof = (lambda v: v.astype(npdt)), None, None, 11, (lambda v: v)
    base, g, b = conv(x), conv(g32), conv(b32)
    t = hpt.Tensor.from_numpy(base, dt).to_hip(dev)
    plan = hpt.normalize_plan(t, 0, 1)
    assert plan.startswith("rowreg-l2gb ") and words in plan, plan
    tg, tb = hpt.Tensor.from_numpy(g, dt).to_hip(dev), hpt.Tensor.from_numpy(b, dt).to_hip(dev)
    half = npdt in ("bf16", np.float16)
    for gg, bb, tgg, tbb in ((g, b, tg, tb), (None, None, None, None), (g, None, tg, None), (None, b, None, tb)):
        got = t.layernorm([n], tgg, tbb, 1e-5).numpy()
        want = orc.layernorm(base, 1, gg, bb, 1e-5, acc=orc.ACC_F64, dtype=odt)
        if half:
            w = tof(want).astype(np.float32)
            assert_close(tof(got).astype(np.float32), w, HALF_RTOL, half_atol(w, bits), f"{npdt} {shape} g={gg is not None} b={bb is not None}")
        else:
            assert_close(got, want, F32_RTOL, F32_ATOL, f"{npdt} {shape} g={gg is not None} b={bb is not None}")


TILE_LENGTHS = [2, 3, 5, 7, 9, 15, 17, 24, 31, 33, 47, 63, 65, 97, 129, 161, 197, 225, 257, 321, 385, 449, 511]


@pytest.mark.parametrize("npdt", [np.float32, np.float16], ids=["f32", "f16"])
def test_short_rows_of_every_count_per_lane(hpt, orc, dev, npdt):
    """The tile kernel is compiled once per number of elements a lane holds (1 ... 8) and picks the lanes per row from the
    row length: row lengths on both sides of every boundary, softmax, log_softmax and layernorm."""
    rng = np.random.default_rng(907)
    half = npdt == np.float16
    acc = orc.ACC_F32 if half else orc.ACC_F64
    for n in TILE_LENGTHS:
        rows = (4 << 20) // (n * np.dtype(npdt).itemsize) + 37   # (at least 4 MiB, or the rows stay with the register kernel)
        x = (rng.standard_normal((rows, n)) * 2 + 0.5).astype(npdt)
        t = hpt.Tensor.from_numpy(x).to_hip(dev)
        assert "+tile" in hpt.normalize_plan(t, 1), (n, hpt.normalize_plan(t, 1))
        g = rng.normal(1, 0.1, n).astype(npdt)
        b = rng.normal(0, 0.1, n).astype(npdt)
        tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
        for what, got, want in (("softmax", t.softmax(1).numpy(), orc.softmax(x, 1, acc=acc)),
                                ("log_softmax", t.log_softmax(1).numpy(), orc.softmax(x, 1, log=True, acc=acc)),
                                ("layernorm", t.layernorm([n], tg, tb, 1e-5).numpy(), orc.layernorm(x, 1, g, b, 1e-5, acc=acc))):
            if half:
                w = want.astype(np.float32)
                assert_close(got.astype(np.float32), w, HALF_RTOL, max(half_atol(w[np.isfinite(w)], 11), 6e-8), f"f16 {what} rows of {n}")
            else:
                assert_close(got, want, F32_RTOL, F32_ATOL, f"f32 {what} rows of {n}")
