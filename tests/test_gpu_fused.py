"""GPU parity of the fused forms, through the C ABI, against the UNFUSED sequences restated with the
oracle: softmax_causal == softmax(where(key > query + offset, -inf, round(scale * x))) and
add_layernorm == layernorm(round(x + residual)) (hpt-examples/examples/transformer/main.rs:87-91, 233-246).
The unfused sequences are also run on the device and must agree with the fused kernels."""
import numpy as np
import pytest

from conftest import assert_close
from oracle import elementwise as ew
from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol, apply_view_np, apply_view_t

pytestmark = pytest.mark.gpu


def causal_reference(orc, a, scale, offset, log, bf16=False, acc=None):
    """The unfused sequence on the host: mul_ by the scalar (rounded to the dtype), masked fill, softmax."""
    if bf16:
        xs = ew.binary(ew.MUL, a, ew.f32_to_bf16_bits(np.array([scale], np.float32)), bf16=True)
        neg = ew.f32_to_bf16_bits(np.array([-np.inf], np.float32))[0]
    else:
        xs = ew.binary(ew.MUL, a, np.array([scale], a.dtype))
        neg = a.dtype.type(-np.inf)
    q = np.arange(a.shape[-2])[:, None]
    k = np.arange(a.shape[-1])[None, :]
    xs = np.where(k > q + offset, neg, xs)
    return xs, orc.softmax(np.ascontiguousarray(xs), a.ndim - 1, log=log, acc=acc, dtype=orc.BF16 if bf16 else None)


CAUSAL_CASES = [
    # name, shape, view ops, scale, offset
    ("square f32", [64, 64], (), 0.125, 0),
    ("heads x queries x keys", [3, 40, 72], (), 0.25, 0),
    ("more keys than queries (offset = K - Q)", [2, 16, 48], (), 1.0, 32),
    ("negative offset: first rows have no key", [24, 24], (), 0.5, -3),
    ("long rows (streaming kernel would not be used, registers)", [5, 4096], (), 1.0, 0),
    ("rows beyond registers: 40000 keys", [3, 40000], (), 0.5, 39990),
    ("1536 keys: three vectors per thread", [2, 300, 1536], (), 0.5, 1236),
    ("2560 keys: five vectors per thread", [1, 200, 2560], (), 1.0, 2360),
    ("6144 keys: six vectors per thread", [1, 96, 6144], (), 1.0, 6048),
    ("sliced view", [4, 33, 70], (("slice", ((0, 4, 1), (1, 33, 1), (3, 67, 1))),), 2.0, 5),
    ("step-2 keys", [2, 32, 128], (("slice", ((0, 2, 1), (0, 32, 1), (0, 128, 2))),), 1.0, 0),
    ("permuted: keys not contiguous", [48, 2, 40], (("permute", (1, 2, 0)),), 0.5, 4),
]


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("case", CAUSAL_CASES, ids=[c[0] for c in CAUSAL_CASES])
def test_softmax_causal_f32_f64(hpt, orc, dev, case, log):
    name, shape, ops, scale, offset = case
    rng = np.random.default_rng(400)
    for npdt in (np.float32, np.float64):
        base = (rng.standard_normal(shape) * 3).astype(npdt)
        t = apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)
        a = apply_view_np(base, ops)
        got = t.softmax_causal(scale, offset, log=log).numpy()
        xs, want = causal_reference(orc, a, scale, offset, log, acc=orc.ACC_F64)
        dead = np.all(np.isneginf(xs), axis=-1)
        assert np.all(np.isnan(got[dead])), f"{name}: rows without keys must be NaN"
        assert_close(got[~dead], want[~dead], F32_RTOL, F32_ATOL, f"softmax_causal {name} log={log} {npdt.__name__}")
        # masked keys: exactly 0 (or -inf): nothing of the masked input leaks
        q = np.arange(a.shape[-2])[:, None]
        k = np.arange(a.shape[-1])[None, :]
        m = np.broadcast_to(k > q + offset, a.shape) & ~dead[..., None]
        assert np.all(np.isneginf(got[m]) if log else got[m] == 0)
        # the same sequence, unfused, on the device
        if not ops:
            sc = hpt.Tensor.from_numpy(np.array([scale], npdt)).to_hip(dev)
            scaled = t.mul(sc).numpy()
            masked = np.where(np.broadcast_to(k > q + offset, a.shape), npdt(-np.inf), scaled)
            unfused = hpt.Tensor.from_numpy(masked).to_hip(dev)
            u = (unfused.log_softmax(-1) if log else unfused.softmax(-1)).numpy()
            assert_close(got[~dead], u[~dead], 2e-6, 1e-7, f"fused vs unfused on device {name}")


@pytest.mark.parametrize("name", ["f16", "bf16"])
def test_softmax_causal_half_types_never_reads_the_masked_part(hpt, orc, dev, name):
    rng = np.random.default_rng(401)
    shape = [4, 96, 160]
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    # poison what the mask hides: NaN there must not reach any output
    q = np.arange(96)[:, None]
    k = np.arange(160)[None, :]
    hidden = np.broadcast_to(k > q + 64, shape)
    xp = np.where(hidden, np.float32(np.nan), x)
    if name == "f16":
        base, dt, bits, tof, bf = xp.astype(np.float16), None, 11, (lambda v: v.astype(np.float32)), False
    else:
        base, dt, bits, tof, bf = hpt.f32_to_bf16_bits(xp), hpt.bf16, 8, hpt.bf16_bits_to_f32, True
    t = hpt.Tensor.from_numpy(base, dt).to_hip(dev)
    for log in (False, True):
        got = tof(t.softmax_causal(0.3, 64, log=log).numpy())
        _, want = causal_reference(orc, base, 0.3, 64, log, bf16=bf, acc=orc.ACC_F32)
        want = tof(want)
        assert not np.isnan(got).any()
        atol = max(half_atol(want[np.isfinite(want)], bits), 6e-8 if name == "f16" else 0.0)
        assert_close(got, want, HALF_RTOL, atol, f"softmax_causal {name} log={log}")


ADD_LN_CASES = [
    ("rows in registers", [37, 1024], (), 1),
    ("two normalised dims", [6, 8, 96], (), 2),
    ("long rows: streaming", [3, 40000], (), 1),
    ("rows of 8192 (two-byte types keep gamma / beta in LDS)", [1300, 8192], (), 1),
    ("rows of 12288, more rows than workgroups", [1100, 12288], (), 1),
    ("rows of 20480: in registers with gamma / beta from L2 (f64: streaming)", [600, 20480], (), 1),
    ("rows of 10240 (f64: five vectors per thread, gamma / beta from L2)", [700, 10240], (), 1),
    ("sliced input", [20, 300], (("slice", ((2, 19, 1), (4, 260, 1))),), 1),
    ("step-2 input", [16, 512], (("slice", ((0, 16, 1), (0, 512, 2))),), 1),
    ("transposed input: demoted to the generic rows", [256, 4096], (("permute", (1, 0)),), 1),
]


@pytest.mark.parametrize("case", ADD_LN_CASES, ids=[c[0] for c in ADD_LN_CASES])
def test_add_layernorm(hpt, orc, dev, case):
    name, shape, ops, nn = case
    rng = np.random.default_rng(402)
    for npdt in (np.float32, np.float64, np.float16):
        base = (rng.standard_normal(shape) + 3).astype(npdt)
        t = apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)
        a = apply_view_np(base, ops)
        r = rng.standard_normal(a.shape).astype(npdt)
        ns = list(a.shape[a.ndim - nn:])
        g = rng.normal(1, 0.1, ns).astype(npdt)
        b = rng.normal(0, 0.1, ns).astype(npdt)
        tr, tg, tb = (hpt.Tensor.from_numpy(v).to_hip(dev) for v in (r, g, b))
        got = t.add_layernorm(tr, ns, tg, tb, 1e-5).numpy()
        summed = ew.binary(ew.ADD, a, r)
        if npdt == np.float16:
            want = orc.layernorm(np.ascontiguousarray(summed), nn, g, b, 1e-5, acc=orc.ACC_F32)
            assert_close(got.astype(np.float32), want.astype(np.float32), HALF_RTOL, half_atol(want, 11),
                         f"add_layernorm f16 {name}")
        else:
            want = orc.layernorm(np.ascontiguousarray(summed), nn, g, b, 1e-5, acc=orc.ACC_F64)
            assert_close(got, want, F32_RTOL, F32_ATOL, f"add_layernorm {npdt.__name__} {name}")
            # unfused on the device: (x + r) then layernorm
            u = t.add(tr).layernorm(ns, tg, tb, 1e-5).numpy()
            assert_close(got, u, 2e-6, 2e-7, f"fused vs unfused on device {name}")
        # without gamma / beta
        got2 = t.add_layernorm(tr, ns, None, None, 1e-5).numpy()
        want2 = orc.layernorm(np.ascontiguousarray(summed), nn, None, None, 1e-5,
                              acc=orc.ACC_F32 if npdt == np.float16 else orc.ACC_F64)
        if npdt == np.float16:
            assert_close(got2.astype(np.float32), want2.astype(np.float32), HALF_RTOL, half_atol(want2, 11), "no affine")
        else:
            assert_close(got2, want2, F32_RTOL, F32_ATOL, f"add_layernorm no affine {name}")


def test_fused_argument_errors(hpt, dev):
    x = hpt.Tensor.from_numpy(np.zeros((4, 8), np.float32)).to_hip(dev)
    with pytest.raises(hpt.ShapeError):
        x.add_layernorm(hpt.Tensor.from_numpy(np.zeros((4, 9), np.float32)).to_hip(dev), [8])
    with pytest.raises(hpt.DTypeError):
        x.add_layernorm(hpt.Tensor.from_numpy(np.zeros((4, 8), np.float64)).to_hip(dev), [8])
    with pytest.raises(hpt.ShapeError):
        x.add_layernorm(hpt.Tensor.from_numpy(np.zeros((8, 4), np.float32)).to_hip(dev).permute([1, 0]), [8])
    with pytest.raises(hpt.ShapeError):
        hpt.Tensor.from_numpy(np.zeros(8, np.float32)).to_hip(dev).softmax_causal()
    with pytest.raises(hpt.DTypeError):
        hpt.Tensor.from_numpy(np.zeros((4, 8), np.int32)).to_hip(dev).softmax_causal()


CHUNK_CASES = [
    # every row length from 1 to K: each chunk of a row (the vectors its lanes hold side by side) is met wholly
    # below the diagonal, wholly above it and cut by it, at every position of the cut
    ("f32 2048 keys, one wavefront per row", np.float32, [2, 2048, 2048], 1.0, 0),
    ("f32 2048 keys, diagonal shifted by one", np.float32, [1, 2048, 2048], 0.5, 1),
    ("f32 2048 keys, first row without keys", np.float32, [1, 2048, 2048], 0.5, -1),
    ("f32 256 keys, several rows per wavefront", np.float32, [3, 512, 256], 0.25, -100),
    ("f32 1000 keys (not a power of two), more queries than keys", np.float32, [2, 1500, 1000], 1.0, 0),
    ("f16 2048 keys", np.float16, [2, 2048, 2048], 0.125, 0),
    ("bf16 2048 keys", "bf16", [2, 2048, 2048], 0.125, 0),
    ("bf16 4096 keys, two wavefronts per row", "bf16", [1, 1024, 4096], 0.125, 3072),
    ("f16 320 keys, several rows per wavefront", np.float16, [4, 320, 320], 1.0, 0),
    # rows dealt out by live length (one wavefront per full row): every class boundary, offsets either way,
    # more queries than keys, a query count that no class divides
    ("f32 1024 keys, 1024 queries", np.float32, [3, 1024, 1024], 1.0, 0),
    ("f32 1024 keys, offset -5", np.float32, [2, 1024, 1024], 0.5, -5),
    ("f32 1024 keys, offset 300", np.float32, [2, 1024, 1024], 0.5, 300),
    ("f32 768 keys (three vectors per thread), 1000 queries", np.float32, [2, 1000, 768], 1.0, -232),
    ("bf16 2048 keys, offset -100", "bf16", [2, 2048, 2048], 0.125, -100),
    ("bf16 2048 keys, offset 700", "bf16", [2, 2048, 2048], 0.125, 700),
    ("f16 2048 keys, 512 queries at the end (offset K - Q)", np.float16, [3, 512, 2048], 0.25, 1536),
    ("f16 2048 keys, 2101 queries", np.float16, [1, 2101, 2048], 1.0, 0),
    ("bf16 2048 keys, nothing kept in most rows", "bf16", [2, 2048, 2048], 1.0, -1900),
]


@pytest.mark.parametrize("log", [False, True])
@pytest.mark.parametrize("case", CHUNK_CASES, ids=[c[0] for c in CHUNK_CASES])
def test_softmax_causal_every_row_length(hpt, orc, dev, case, log):
    name, npdt, shape, scale, offset = case
    rng = np.random.default_rng(402)
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    if npdt == "bf16":
        base, dt, bits, tof, bf, acc = hpt.f32_to_bf16_bits(x), hpt.bf16, 8, hpt.bf16_bits_to_f32, True, orc.ACC_F32
    elif npdt == np.float16:
        base, dt, bits, tof, bf, acc = x.astype(np.float16), None, 11, (lambda v: v.astype(np.float32)), False, orc.ACC_F32
    else:
        base, dt, bits, tof, bf, acc = x, None, 0, (lambda v: v), False, orc.ACC_F64
    t = hpt.Tensor.from_numpy(base, dt).to_hip(dev)
    got = tof(t.softmax_causal(scale, offset, log=log).numpy())
    xs, want = causal_reference(orc, base, scale, offset, log, bf16=bf, acc=acc)
    want = tof(want)
    xs = tof(xs) if bf or bits else xs
    dead = np.all(np.isneginf(xs), axis=-1)
    assert np.all(np.isnan(got[dead])), f"{name}: rows without keys must be NaN"
    if bits:
        atol = max(half_atol(want[~dead][np.isfinite(want[~dead])], bits), 6e-8 if npdt == np.float16 else 0.0)
        assert_close(got[~dead], want[~dead], HALF_RTOL, atol, f"{name} log={log}")
    else:
        assert_close(got[~dead], want[~dead], F32_RTOL, F32_ATOL, f"{name} log={log}")
    q = np.arange(shape[-2])[:, None]
    k = np.arange(shape[-1])[None, :]
    m = np.broadcast_to(k > q + offset, shape) & ~dead[..., None]
    assert np.all(np.isneginf(got[m]) if log else got[m] == 0), f"{name}: masked keys must come out exactly 0 / -inf"
    if not log:
        assert_close(got[~dead].astype(np.float64).sum(-1), np.ones(int((~dead).sum())), 2 ** -bits if bits else 2e-6, 0, f"{name}: rows sum to one")
