"""GPU parity of the steps either side of the path, through the C ABI: contiguous() of any view
(hpt/src/backends/cuda/tensor_internal/normal_out_unary.rs:286-310), full (set_val), and add / sub / mul /
div with broadcasting and in place (hpt-traits/src/ops/binary.rs:34-152). Every result is bit-exact against
oracle/elementwise.py."""
import numpy as np
import pytest

from oracle import elementwise as ew
from util import apply_view_np, apply_view_t, layouts_for

pytestmark = pytest.mark.gpu

NP_DTYPES = [np.bool_, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64,
             np.float16, np.float32, np.float64]


def rand(rng, shape, npdt):
    if npdt == np.bool_:
        return rng.integers(0, 2, shape).astype(np.bool_)
    if np.dtype(npdt).kind in "iu":
        info = np.iinfo(npdt)
        return rng.integers(info.min, info.max, shape, dtype=npdt, endpoint=True)
    return (rng.standard_normal(shape) * 4).astype(npdt)


def same_bits(got, want, msg):
    assert got.shape == want.shape and got.dtype == want.dtype, msg
    got, want = np.ascontiguousarray(got), np.ascontiguousarray(want)
    assert np.array_equal(got.view(np.uint8) if got.size else got, want.view(np.uint8) if want.size else want), msg


# ---- contiguous ------------------------------------------------------------------------------------

COPY_CASES = [
    # name, base shape, view ops, expected plan prefix
    ("2-D transpose, ragged tiles", [200, 136], (("permute", (1, 0)),), "transpose"),
    ("3-D rotate", [24, 40, 72], (("permute", (2, 0, 1)),), "transpose"),
    ("batched transpose", [3, 80, 48], (("permute", (0, 2, 1)),), "transpose"),
    # whole (16 vectors)^2 tiles in both dims for every element size, with ragged last tiles: staged through LDS
    ("2-D transpose through LDS, ragged tiles", [400, 304], (("permute", (1, 0)),), "transpose"),
    ("batched transpose through LDS", [3, 272, 400], (("permute", (0, 2, 1)),), "transpose"),
    ("3-D rotate through LDS", [272, 5, 288], (("permute", (2, 1, 0)),), "transpose"),
    ("4-D middle swap keeps inner rows", [4, 6, 10, 64], (("permute", (0, 2, 1, 3)),), "inner"),
    ("row slice", [50, 128], (("slice", ((3, 41, 1), (0, 128, 1))),), "inner"),
    ("column slice (unaligned rows)", [50, 128], (("slice", ((0, 50, 1), (5, 77, 1))),), "inner"),
    ("step 2 columns", [50, 128], (("slice", ((0, 50, 1), (0, 128, 2))),), "inner-step2"),
    ("step 2 columns, odd start", [50, 128], (("slice", ((0, 50, 1), (1, 128, 2))),), "inner vec=1"),
    ("step 2 rows and columns", [50, 128], (("slice", ((1, 50, 2), (0, 128, 2))),), "inner-step2"),
    ("negative steps", [9, 31], (("slice", ((8, None, -1), (30, None, -3))),), "inner"),
    ("transpose too small for tiles", [5, 7], (("permute", (1, 0)),), "inner"),
    ("5-D permute", [3, 4, 5, 6, 8], (("permute", (4, 2, 0, 3, 1)),), ""),
    ("one element", [1, 1], (), "inner"),
]


@pytest.mark.parametrize("case", COPY_CASES, ids=[c[0] for c in COPY_CASES])
def test_contiguous_all_dtypes(hpt, dev, case):
    name, shape, ops, plan = case
    rng = np.random.default_rng(300)
    for npdt in NP_DTYPES:
        base = rand(rng, shape, npdt)
        t = apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)
        a = apply_view_np(base, ops)
        if np.dtype(npdt).itemsize == 4 and plan:
            assert hpt.contiguous_plan(t).startswith(plan), hpt.contiguous_plan(t)
        c = t.contiguous()
        assert c.is_contiguous() and c.shape == list(a.shape)
        same_bits(c.numpy(), ew.contiguous(a), f"contiguous {name} {np.dtype(npdt).name}")
        # to_cpu of a view goes through the same device copy (tensor_impls.rs:154-160)
        same_bits(t.to_cpu().numpy(), ew.contiguous(a), f"to_cpu {name} {np.dtype(npdt).name}")


def test_contiguous_bf16_random_layouts_and_empty(hpt, dev):
    rng = np.random.default_rng(301)
    for shape in ([33, 129], [4, 18, 40], [2, 3, 4, 5]):
        base = rng.integers(0, 65536, shape).astype(np.uint16)
        for lname, ops in layouts_for(shape, rng):
            t = apply_view_t(hpt.Tensor.from_numpy(base, hpt.bf16).to_hip(dev), ops)
            same_bits(t.contiguous().numpy(), ew.contiguous(apply_view_np(base, ops)), f"bf16 {shape} {lname}")
    e = hpt.Tensor.from_numpy(np.zeros((4, 0, 3), np.float32)).to_hip(dev).permute([2, 1, 0]).contiguous()
    assert e.shape == [3, 0, 4] and e.numpy().size == 0


def test_contiguous_large_transpose_and_errors(hpt, dev):
    """f16 [4096, 2048] transposed: 16 MiB through the LDS-staged tile kernel; f64 [1024, 1536]; i8."""
    rng = np.random.default_rng(302)
    for npdt, shape in ((np.float16, [4096, 2048]), (np.float64, [1024, 1536]), (np.int8, [2048, 4096])):
        base = rand(rng, shape, npdt)
        t = hpt.Tensor.from_numpy(base).to_hip(dev).permute([1, 0])
        assert hpt.contiguous_plan(t).startswith("transpose") and hpt.contiguous_plan(t).endswith("lds")
        same_bits(t.contiguous().numpy(), ew.contiguous(base.T), f"large transpose {np.dtype(npdt).name}")
    from hpt_amd import _ffi
    import ctypes as C
    a = hpt.Tensor.from_numpy(np.zeros((4, 6), np.float32)).to_hip(dev)
    bad = hpt.Tensor.empty([6, 5], hpt.f32, dev)
    va, k1 = a.permute([1, 0])._c_view()
    vb, k2 = bad._c_view()
    with pytest.raises(hpt.ShapeError):
        _ffi.check(hpt.lib().hpt_hip_contiguous(dev, None, C.byref(va), C.byref(vb)))
    wrong = hpt.Tensor.empty([6, 4], hpt.i32, dev)
    vw, k3 = wrong._c_view()
    with pytest.raises(hpt.DTypeError):
        _ffi.check(hpt.lib().hpt_hip_contiguous(dev, None, C.byref(va), C.byref(vw)))


# ---- fill -------------------------------------------------------------------------------------------

def test_full_all_dtypes_and_unaligned_views(hpt, dev):
    vals = {np.bool_: True, np.int8: -7, np.int16: -1234, np.int32: -123456789, np.int64: -(1 << 40) - 3,
            np.uint8: 200, np.uint16: 54321, np.uint32: 4000000000, np.uint64: (1 << 63) + 5,
            np.float16: 1.5, np.float32: -2.25, np.float64: 3.141592653589793}
    for npdt, v in vals.items():
        t = hpt.Tensor.from_numpy(np.zeros(1, npdt))   # only to look the dtype up
        for shape in ([1], [5], [1000], [3, 7, 11], [0]):
            f = hpt.Tensor.full(v, shape, t.dtype, dev)
            same_bits(f.numpy(), ew.full(v, shape, npdt), f"full {np.dtype(npdt).name} {shape}")
    b = hpt.Tensor.full(1.0 / 3.0, [9], hpt.bf16, dev).numpy()
    assert np.all(b == ew.f32_to_bf16_bits(np.array([1.0 / 3.0], np.float32))[0])
    assert np.all(hpt.Tensor.zeros([4, 4], hpt.f32, dev).numpy() == 0)
    assert np.all(hpt.Tensor.ones([4, 4], hpt.i64, dev).numpy() == 1)
    # fill a contiguous tail that starts off a 16-byte boundary: the rest of the block must stay untouched
    from hpt_amd import _ffi
    import ctypes as C
    base = hpt.Tensor.from_numpy(np.arange(100, dtype=np.int16)).to_hip(dev)
    tail = base[3:90]
    val = np.array([-5], np.int16)
    v, k = tail._c_view()
    _ffi.check(hpt.lib().hpt_hip_fill(dev, None, C.byref(v), C.c_void_p(val.ctypes.data)))
    want = np.arange(100, dtype=np.int16)
    want[3:90] = -5
    same_bits(base.numpy(), want, "fill of an unaligned tail")


# ---- binary -----------------------------------------------------------------------------------------

OPS = (("add", ew.ADD), ("sub", ew.SUB), ("mul", ew.MUL), ("div", ew.DIV))


@pytest.mark.parametrize("npdt", NP_DTYPES, ids=[np.dtype(d).name for d in NP_DTYPES])
def test_binary_broadcast_patterns(hpt, dev, npdt):
    rng = np.random.default_rng(310)
    shapes = [([37, 64], [37, 64]),      # same shape: flat vectors
              ([37, 64], [64]),          # bias over rows (layernorm's add_ / mul_)
              ([37, 64], [37, 1]),       # per-row scalar: broadcast along the inner dim
              ([5, 1, 24], [1, 7, 24]),  # both sides broadcast
              ([6, 10], [1]),            # scalar tensor
              ([3, 5], [3, 5])]          # tiny, not vectorisable
    for sa, sb in shapes:
        a, b = rand(rng, sa, npdt), rand(rng, sb, npdt)
        if np.dtype(npdt).kind == "f":
            b = np.where(np.abs(b) < 0.25, npdt(1.0), b)   # keep quotients tame
        ta, tb = hpt.Tensor.from_numpy(a).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
        for name, op in OPS:
            ok = not (npdt == np.bool_ and op in (ew.SUB, ew.DIV)) and not (op == ew.DIV and np.dtype(npdt).kind != "f")
            if not ok:
                with pytest.raises(hpt.DTypeError):
                    getattr(ta, name)(tb)
                continue
            got = getattr(ta, name)(tb).numpy()
            same_bits(got, ew.binary(op, a, b), f"{name} {np.dtype(npdt).name} {sa} {sb}")


def test_binary_strided_operands_inplace_and_bf16(hpt, dev):
    rng = np.random.default_rng(311)
    base = rand(rng, [48, 80], np.float32)
    other = rand(rng, [80, 48], np.float32)
    ta, tb = hpt.Tensor.from_numpy(base).to_hip(dev), hpt.Tensor.from_numpy(other).to_hip(dev)
    same_bits(ta.add(tb.permute([1, 0])).numpy(), ew.binary(ew.ADD, base, other.T), "add of a transposed operand")
    same_bits(ta[:, ::2].mul(tb.permute([1, 0])[:, 1::2]).numpy(), ew.binary(ew.MUL, base[:, ::2], other.T[:, 1::2]),
              "mul of stepped views")
    # in place: res.add_(beta, res) / res.mul_(gamma, res), as normalization.rs:187-192
    res = hpt.Tensor.from_numpy(base).to_hip(dev)
    gamma = rand(rng, [80], np.float32)
    tg = hpt.Tensor.from_numpy(gamma).to_hip(dev)
    out = res.mul_(tg, res)
    assert out is res
    same_bits(res.numpy(), ew.binary(ew.MUL, base, gamma), "mul_ in place")
    res.add_(tg, res)
    same_bits(res.numpy(), ew.binary(ew.ADD, ew.binary(ew.MUL, base, gamma), gamma), "add_ in place")
    # out overlapping an operand without being it is refused
    with pytest.raises(hpt.ParamError):
        ta[1:].add_(ta[1:], ta[:-1])
    # bf16
    xa = ew.f32_to_bf16_bits(rand(rng, [33, 40], np.float32))
    xb = ew.f32_to_bf16_bits(rand(rng, [40], np.float32))
    t1, t2 = hpt.Tensor.from_numpy(xa, hpt.bf16).to_hip(dev), hpt.Tensor.from_numpy(xb, hpt.bf16).to_hip(dev)
    for name, op in OPS[:3]:
        same_bits(getattr(t1, name)(t2).numpy(), ew.binary(op, xa, xb, bf16=True), f"bf16 {name}")
    # dtype mismatch and shape mismatch
    with pytest.raises(hpt.DTypeError):
        ta.add(hpt.Tensor.from_numpy(np.zeros([48, 80], np.float64)).to_hip(dev))
    with pytest.raises(hpt.ShapeError):
        ta.add(hpt.Tensor.from_numpy(np.zeros([48, 81], np.float32)).to_hip(dev))


TRANSPOSED_OPERAND_CASES = [
    # (dtype, shape of the result, which operands are permuted views, the permutation)
    ("f32 a + b.t()", np.float32, [264, 136], "rhs", (1, 0)),
    ("f32 a.t() - b", np.float32, [264, 136], "lhs", (1, 0)),
    ("f32 a.t() * b.t()", np.float32, [200, 328], "both", (1, 0)),
    ("f16 both, tiles of 128", np.float16, [264, 392], "both", (1, 0)),
    ("f16 rhs", np.float16, [520, 136], "rhs", (1, 0)),
    ("f64", np.float64, [72, 104], "both", (1, 0)),
    ("i32 wraps", np.int32, [136, 200], "rhs", (1, 0)),
    ("u16", np.uint16, [264, 136], "lhs", (1, 0)),
    ("i64", np.int64, [40, 72], "both", (1, 0)),
    ("f32 3-D, batch outermost", np.float32, [5, 136, 72], "rhs", (0, 2, 1)),
    ("f32 3-D, the batch dim between", np.float32, [72, 3, 136], "both", (2, 1, 0)),
    ("f16 4-D", np.float16, [2, 3, 136, 264], "lhs", (0, 1, 3, 2)),
]


@pytest.mark.parametrize("case", TRANSPOSED_OPERAND_CASES, ids=[c[0] for c in TRANSPOSED_OPERAND_CASES])
def test_binary_with_transposed_operands(hpt, dev, case):
    """An operand whose contiguous dim is not the innermost one (a + b.t()) is transposed tile by tile
    through LDS inside the binary kernel; the other operand may lie like the result, be transposed too,
    or be broadcast; the result may overwrite an operand that lies like it."""
    name, npdt, shape, which, perm = case
    rng = np.random.default_rng(330)
    inv = list(np.argsort(perm))
    pshape = [shape[i] for i in inv]  # parent shape whose permutation by `perm` is `shape`

    def operand(transposed):
        if transposed:
            base = rand(rng, pshape, npdt)
            return base.transpose(perm), hpt.Tensor.from_numpy(base).to_hip(dev).permute(list(perm))
        base = rand(rng, shape, npdt)
        return base, hpt.Tensor.from_numpy(base).to_hip(dev)

    a, ta = operand(which in ("lhs", "both"))
    b, tb = operand(which in ("rhs", "both"))
    if np.dtype(npdt).kind == "f":
        b = np.where(np.abs(b) < 0.25, npdt(1.0), b)
        tb = hpt.Tensor.from_numpy(np.ascontiguousarray(b.transpose(inv) if which in ("rhs", "both") else b)).to_hip(dev)
        if which in ("rhs", "both"):
            tb = tb.permute(list(perm))
    plan = hpt.binary_plan(ta, tb)
    assert plan.startswith("transpose") and plan.endswith(f"{which} lds"), plan
    for opname, op in OPS:
        if op == ew.DIV and np.dtype(npdt).kind != "f":
            continue
        same_bits(getattr(ta, opname)(tb).numpy(), ew.binary(op, a, b), f"{opname} {name}")
    # broadcast partners of a transposed operand: a row, a column, a scalar
    if which != "both" and len(shape) == 2:
        t_op, n_np = (ta, a) if which == "lhs" else (tb, b)
        for bshape in ([shape[1]], [shape[0], 1], [1]):
            o = rand(rng, bshape, npdt)
            to = hpt.Tensor.from_numpy(o).to_hip(dev)
            assert hpt.binary_plan(t_op, to.expand(shape)).startswith("transpose"), hpt.binary_plan(t_op, to.expand(shape))
            same_bits(t_op.mul(to).numpy(), ew.binary(ew.MUL, n_np, o), f"mul by a broadcast {bshape} {name}")
            same_bits(to.sub(t_op).numpy(), ew.binary(ew.SUB, o, n_np), f"broadcast {bshape} minus {name}")
    # in place over the operand that lies like the result
    if which == "rhs":
        res = hpt.Tensor.from_numpy(np.ascontiguousarray(a)).to_hip(dev)
        assert res.add_(tb, res) is res
        same_bits(res.numpy(), ew.binary(ew.ADD, a, b), f"add_ in place {name}")


def test_binary_transposed_operands_large_and_refusals(hpt, dev):
    rng = np.random.default_rng(331)
    a = rand(rng, [2048, 3072], np.float32)
    b = rand(rng, [3072, 2048], np.float32)
    ta, tb = hpt.Tensor.from_numpy(a).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
    same_bits(ta.add(tb.permute([1, 0])).numpy(), a + b.T, "f32 [2048, 3072] a + b.t()")
    same_bits(ta.permute([1, 0]).mul(tb).numpy(), a.T * b, "f32 [3072, 2048] a.t() * b")
    # one-byte types, short dims and unaligned views keep the gathering kernel
    u = hpt.Tensor.from_numpy(rand(rng, [512, 256], np.uint8)).to_hip(dev)
    assert hpt.binary_plan(u.permute([1, 0]), u.permute([1, 0])).startswith("inner")
    s = hpt.Tensor.from_numpy(rand(rng, [48, 80], np.float32)).to_hip(dev)
    assert hpt.binary_plan(s, hpt.Tensor.from_numpy(rand(rng, [80, 48], np.float32)).to_hip(dev).permute([1, 0])).startswith("inner")
    odd = ta[:, 1:2049]  # rows start off the 16-byte grid
    assert hpt.binary_plan(odd, tb.permute([1, 0])[:, :2048]).startswith("inner")
    same_bits(odd.add(tb.permute([1, 0])[:, :2048]).numpy(), a[:, 1:2049] + b.T[:, :2048], "unaligned partner")
    # an output that overlaps the transposed operand without being it is refused
    sq = hpt.Tensor.from_numpy(rand(rng, [256, 256], np.float32)).to_hip(dev)
    with pytest.raises(hpt.ParamError):
        sq.permute([1, 0]).add_(sq, sq)


def test_layernorm_equals_normalise_then_affine_steps(hpt, orc, dev):
    """The reference applies gamma / beta as separate mul_ / add_ passes after normalising
    (normalization.rs:187-192); the fused kernel must agree with those steps done on the device."""
    rng = np.random.default_rng(312)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    g = rng.normal(1, 0.1, 256).astype(np.float32)
    b = rng.normal(0, 0.1, 256).astype(np.float32)
    tx, tg, tb = (hpt.Tensor.from_numpy(v).to_hip(dev) for v in (x, g, b))
    fused = tx.layernorm([256], tg, tb, 1e-5).numpy()
    steps = tx.layernorm([256], None, None, 1e-5)
    steps.mul_(tg, steps)
    steps.add_(tb, steps)
    np.testing.assert_allclose(steps.numpy(), fused, rtol=2e-6, atol=2e-7)


# ---- casts ------------------------------------------------------------------------------------------

def test_astype_to_float_dtypes_bit_exact(hpt, dev):
    rng = np.random.default_rng(320)
    targets = [(hpt.f16, np.float16), (hpt.f32, np.float32), (hpt.f64, np.float64), (hpt.bf16, "bf16")]
    for npdt in NP_DTYPES:
        for shape, ops in (([37, 64], ()), ([40, 24], (("permute", (1, 0)),)), ([5, 7, 3], (("slice", ((0, 5, 2), (1, 7, 1), (0, 3, 1))),))):
            base = rand(rng, shape, npdt)
            if np.dtype(npdt).kind == "f":
                base = (base.astype(np.float64) * rng.choice([1e-6, 1.0, 300.0, 7e4], shape)).astype(npdt)
            t = apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)
            a = apply_view_np(base, ops)
            for hdt, to in targets:
                got = t.astype(hdt).numpy()
                want = np.ascontiguousarray(ew.cast(a, to))
                same_bits(got, want, f"astype {np.dtype(npdt).name} -> {hdt.name} {shape} {ops}")
    # bf16 source
    xb = ew.f32_to_bf16_bits((rng.standard_normal((33, 16)) * 100).astype(np.float32))
    tb = hpt.Tensor.from_numpy(xb, hpt.bf16).to_hip(dev)
    for hdt, to in targets:
        same_bits(tb.astype(hdt).numpy(), np.ascontiguousarray(ew.cast(xb, to, bf16_in=True)), f"astype bf16 -> {hdt.name}")
    # the f64 -> half tie cases that a detour through f32 gets wrong
    d = np.array([1 + 2.0 ** -11 + 2.0 ** -40, 1 + 2.0 ** -11, 65519.999, 65520.0, 6e-8, -2.5e-8, np.nan, np.inf,
                  1 + 2.0 ** -8 + 2.0 ** -40, 3.4e38])
    td = hpt.Tensor.from_numpy(d).to_hip(dev)
    got = td.astype(hpt.f16).numpy()
    want = ew.cast(d, np.float16)
    assert np.array_equal(got.view(np.uint16)[~np.isnan(want)], want.view(np.uint16)[~np.isnan(want)]) and np.isnan(got[6])
    gb = td.astype(hpt.bf16).numpy()
    wb = ew.cast(d, "bf16")
    keep = ~np.isnan(d)
    assert np.array_equal(gb[keep], wb[keep]) and np.isnan(ew.bf16_bits_to_f32(gb)[6])
    with pytest.raises(hpt.DTypeError):
        td.astype(hpt.i32)
    same_bits(hpt.Tensor.from_numpy(np.arange(12, dtype=np.int32).reshape(3, 4)).to_hip(dev).permute([1, 0]).astype(hpt.i32).numpy(),
              np.ascontiguousarray(np.arange(12, dtype=np.int32).reshape(3, 4).T), "astype to the same dtype is a copy")


def test_integer_inputs_of_softmax_and_layernorm_promote(hpt, orc, dev):
    """NormalizationOps::Output = Tensor<FloatBinaryType<T>>: i32 -> f32, i16 -> f16, i64 -> f64."""
    from conftest import assert_close
    rng = np.random.default_rng(321)
    xi = rng.integers(-6, 7, (19, 200)).astype(np.int32)
    t = hpt.Tensor.from_numpy(xi).to_hip(dev)
    s = t.softmax(1)
    assert s.dtype is hpt.f32
    assert_close(s.numpy(), orc.softmax(xi.astype(np.float32), 1, acc=orc.ACC_F64), 1e-5, 1e-6, "softmax of i32")
    ln = t.layernorm([200])
    assert ln.dtype is hpt.f32
    assert_close(ln.numpy(), orc.layernorm(xi.astype(np.float32), 1, None, None, 1e-5, acc=orc.ACC_F64), 1e-5, 1e-6, "layernorm of i32")
    x16 = rng.integers(-5, 6, (7, 64)).astype(np.int16)
    s16 = hpt.Tensor.from_numpy(x16).to_hip(dev).log_softmax(-1)
    assert s16.dtype is hpt.f16
    want = orc.softmax(x16.astype(np.float16), 1, log=True, acc=orc.ACC_F32).astype(np.float32)
    assert_close(s16.numpy().astype(np.float32), want, 1e-2, 1e-3, "log_softmax of i16")
    x64 = rng.integers(-5, 6, (3, 5, 9)).astype(np.int64)
    s64 = hpt.Tensor.from_numpy(x64).to_hip(dev).permute([2, 0, 1]).softmax(0)
    assert s64.dtype is hpt.f64
    assert_close(s64.numpy(), orc.softmax(x64.astype(np.float64).transpose(2, 0, 1), 0, acc=orc.ACC_F64), 1e-12, 1e-14, "softmax of i64")


PROMOTED = [(np.bool_, np.float16), (np.int8, np.float16), (np.int16, np.float16), (np.uint8, np.float16), (np.uint16, np.float16),
            (np.int32, np.float32), (np.uint32, np.float32), (np.int64, np.float64), (np.uint64, np.float64)]


@pytest.mark.parametrize("npin,npout", PROMOTED, ids=[p[0].__name__ for p in PROMOTED])
def test_integer_inputs_are_promoted_inside_one_call(hpt, orc, dev, npin, npout):
    """softmax / log_softmax / layernorm of an integer tensor through ONE C-ABI call each (no astype
    first): the result must equal the op applied to the input cast to FloatBinaryType<T> - including
    values the cast rounds (i16 / u16 beyond 2048 in f16, i32 beyond 2^24 in f32, u16 beyond 65504 -> inf) -
    on contiguous rows (vector loads of the integer type), permuted, sliced and stepped views."""
    import ctypes as C
    from conftest import assert_close
    from util import layouts_for, upload
    rng = np.random.default_rng(77)
    half = npout == np.float16
    for shape in ([33, 256], [5, 6, 40], [260, 1024]):
        if npin == np.bool_:
            base = rng.random(shape) < 0.4
        else:
            info = np.iinfo(npin)
            base = rng.integers(max(info.min, -9), min(info.max, 9) + 1, shape).astype(npin)
            # a few values that do not survive the cast exactly
            flat = base.reshape(-1)
            big = {np.int16: [2049, -4099, 30001], np.uint16: [2051, 65519, 65535], np.int32: [(1 << 24) + 1, -(1 << 25) - 3],
                   np.uint32: [(1 << 24) + 1, 4294967295], np.int64: [(1 << 53) + 1], np.uint64: [(1 << 53) + 1]}.get(npin, [])
            for k, v in enumerate(big):
                flat[(k * 37) % flat.size] = v
        for lname, ops in layouts_for(shape, rng):
            t, a = upload(hpt, base, ops, dev=dev)
            if a.size == 0:
                continue
            with np.errstate(over="ignore"):
                af = a.astype(npout)      # what `astype` would have stored
            nd = a.ndim
            for axis in (nd - 1, 0):
                for log in (False, True):
                    # straight through the ABI: integer view in, float tensor out
                    res = hpt.Tensor.empty(a.shape, hpt.DTYPES[orc.reduce_out_dtype(orc.MEAN, t.dtype.code)], dev)
                    vin, k1 = t._c_view()
                    vout, k2 = res._c_view()
                    hpt._ffi.check(hpt.lib().hpt_hip_softmax(dev, None, int(log), C.byref(vin), axis, C.byref(vout)))
                    got = res.numpy()
                    assert got.dtype == npout
                    with np.errstate(invalid="ignore", over="ignore"):
                        want = orc.softmax(af, axis, log=log, acc=orc.ACC_F32 if half else orc.ACC_F64)
                    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{npin.__name__} {shape} {lname} axis={axis} log={log}: NaN pattern"
                    if half:
                        assert_close(got, want, 1e-2, 1e-3 if log else 6e-8 + 1e-3 * float(np.nanmax(want)), f"softmax {npin.__name__} {shape} {lname} axis={axis} log={log}")
                    elif npout == np.float32:
                        assert_close(got, want, 1e-5, 1e-6, f"softmax {npin.__name__} {shape} {lname} axis={axis} log={log}")
                    else:
                        assert_close(got, want, 1e-12, 1e-13, f"softmax {npin.__name__} {shape} {lname} axis={axis} log={log}")
            n = a.shape[-1]
            g = rng.normal(1, 0.1, n).astype(npout)
            b = rng.normal(0, 0.1, n).astype(npout)
            tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
            got = t.layernorm([n], tg, tb, 1e-5).numpy()
            assert got.dtype == npout
            fin = np.isfinite(af).all(axis=-1)
            with np.errstate(invalid="ignore", over="ignore"):
                want = orc.layernorm(af, 1, g, b, 1e-5, acc=orc.ACC_F32 if half else orc.ACC_F64)
            tol = (1e-2, 4e-3) if half else ((1e-5, 1e-6) if npout == np.float32 else (1e-12, 1e-12))
            assert_close(got[fin], want[fin], tol[0], tol[1], f"layernorm {npin.__name__} {shape} {lname}")
            # gamma / beta must have the OUTPUT's dtype
            if npin != np.bool_ and lname == "contiguous":
                wrong = hpt.Tensor.from_numpy(np.ones(n, npin)).to_hip(dev)
                with pytest.raises(hpt.DTypeError, match="gamma"):
                    t.layernorm([n], wrong, None, 1e-5)
    # the fused kinds take float tensors only
    ti = hpt.Tensor.from_numpy(np.ones((4, 8), npin)).to_hip(dev)
    with pytest.raises(hpt.DTypeError):
        ti.softmax_causal(1.0)
