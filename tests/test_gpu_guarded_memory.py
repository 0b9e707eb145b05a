"""Nothing is written outside the output, and nothing at all into the input: every op of the path on
random views whose parent and whose result both sit inside one arena of foreign memory filled with a
byte pattern, a few bytes off the 16-byte grid. After each op the whole arena is read back; the bytes
of the result's slot must agree with the same op writing into memory of the library's own, and every
other byte (the guards either side, the parent with the elements a view skips) must be as uploaded.
The kernels read and write whole 128-bit vectors over rows that start and end anywhere, and several
walk tiles that overhang the view: this is the test that an overhang is never stored."""
import ctypes as C
import os

import numpy as np
import pytest

from conftest import assert_close
from test_gpu_random_views import layernorm_floor, rand_base, rand_shape, rand_view
from util import apply_view_np, apply_view_t

pytestmark = pytest.mark.gpu

GUARD = 4096
PATTERN = 0xA5


@pytest.fixture(scope="module")
def hip():
    h = C.CDLL("libamdhip64.so")
    h.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    h.hipFree.argtypes = [C.c_void_p]
    h.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    return h


class Arena:
    """[guard | pad | parent | guard | pad | result | guard] in one hipMalloc block."""

    def __init__(self, hip, base, in_pad, out_bytes, out_pad):
        self.hip = hip
        self.in_off = GUARD + in_pad
        self.out_off = self.in_off + base.nbytes + GUARD
        self.out_off += -self.out_off % 16 + out_pad
        self.out_bytes = out_bytes
        self.host = np.full(self.out_off + out_bytes + GUARD, PATTERN, np.uint8)
        self.host[self.in_off:self.in_off + base.nbytes] = np.ascontiguousarray(base).view(np.uint8).reshape(-1)
        p = C.c_void_p()
        assert hip.hipMalloc(C.byref(p), self.host.nbytes) == 0
        self.ptr = p.value
        self.upload()

    def upload(self):
        assert self.hip.hipMemcpy(C.c_void_p(self.ptr), C.c_void_p(self.host.ctypes.data), self.host.nbytes, 1) == 0

    def check(self, what):
        """Returns the result slot's bytes; everything else must be as uploaded."""
        back = np.empty_like(self.host)
        assert self.hip.hipMemcpy(C.c_void_p(back.ctypes.data), C.c_void_p(self.ptr), back.nbytes, 2) == 0
        lo, hi = self.out_off, self.out_off + self.out_bytes
        for name, a, b in (("before", 0, lo), ("after", hi, back.size)):
            bad = np.nonzero(back[a:b] != self.host[a:b])[0]
            assert bad.size == 0, (f"{what}: {bad.size} bytes changed {name} the result, first at arena offset "
                                   f"{a + int(bad[0])} (parent at {self.in_off}, result at {lo}..{hi})")
        return back[lo:hi].copy()

    def free(self):
        assert self.hip.hipFree(C.c_void_p(self.ptr)) == 0


def raw_view(hpt, arena, base, a, dev):
    """The device tensor over the arena's copy of `base` that has the layout of the numpy view `a`."""
    off = a.__array_interface__["data"][0] - base.__array_interface__["data"][0]
    strides = [s // a.itemsize for s in a.strides]
    return hpt.Tensor.from_raw(arena.ptr + arena.in_off + off, a.shape, hpt.tensor._BY_NP[np.dtype(a.dtype)], dev,
                               strides=strides)


def same(got, want, floor, what):
    """The two results come from the same library on the same view; the alignment of parent and result
    differs, which may pick other vector widths and with them another order of the additions."""
    if want.dtype.kind != "f":
        assert np.array_equal(got, want), what
        return
    rtol = 2e-3 if want.dtype == np.float16 else (1e-12 if want.dtype == np.float64 else 1e-5)
    assert_close(got, want, rtol, floor, what)


def run_guarded(hpt, hip, dev, rng, base, ops, names, axes, pads, what):
    """Each op in `names` on the view `ops` of `base`, once into library memory and once inside an arena."""
    from util import apply_view_t
    a = apply_view_np(base, ops)
    nd = a.ndim
    is_float = base.dtype.kind == "f"
    t_probe = apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)
    acc_ulp = 2.0 ** -52 if base.dtype == np.float64 else 2.0 ** -23
    in_pad, out_pad_units = pads
    for name in names:
        floor = 0.0
        extra = ()
        if name == "sum":
            want_t = t_probe.sum(axes)
            if is_float:  # the additions' rounding scales with the sum of magnitudes, not with the result
                floor = 8 * acc_ulp * np.abs(a.astype(np.float64)).sum(tuple(axes))
        elif name == "max":
            want_t = t_probe.max(axes)
        elif name in ("softmax", "log_softmax"):
            ax = axes[0]
            want_t = getattr(t_probe, name)(ax)
            floor = 16 * acc_ulp * (8 if name == "log_softmax" else 1)
        elif name == "mul":
            g = rng.normal(1, 0.1, a.shape[-1:]).astype(base.dtype)
            tg = hpt.Tensor.from_numpy(g).to_hip(dev)
            want_t = t_probe.mul(tg)
        else:
            nn = len(axes)  # layernorm over the trailing len(axes) dims
            ns = list(a.shape[nd - nn:])
            if int(np.prod(ns)) < 2:
                continue
            g = rng.normal(1, 0.1, ns).astype(base.dtype)
            b = rng.normal(0, 0.1, ns).astype(base.dtype)
            tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
            want_t = t_probe.layernorm(ns, tg, tb, 1e-5)
            floor = 64 * acc_ulp + layernorm_floor(a, nn, g, acc_ulp)
        want = want_t.numpy()
        osz = want.dtype.itemsize
        out_pad = (out_pad_units * osz) % 16
        arena = Arena(hip, base, in_pad, max(want.nbytes, osz), out_pad)
        try:
            t = raw_view(hpt, arena, base, a, dev)
            o = hpt.Tensor.from_raw(arena.ptr + arena.out_off, want.shape if want.ndim else [1],
                                    hpt.tensor._BY_NP[np.dtype(want.dtype)], dev)
            w = f"{name} out_pad={out_pad} {what}"
            if name == "sum":
                t.sum_(axes, False, True, o)
            elif name == "max":
                t._reduce(hpt.tensor.MAX, axes, False, out=o)
            elif name in ("softmax", "log_softmax"):
                getattr(t, name)(ax, out=o)
            elif name == "mul":
                t.mul_(tg, o)
            else:
                t.layernorm(ns, tg, tb, 1e-5, out=o)
            hpt.synchronize(dev)
            got = arena.check(w)[:want.nbytes].view(want.dtype).reshape(want.shape)
            same(got, want, floor, w)
        finally:
            hpt.synchronize(dev)
            arena.free()


# (HPT_GUARDED_SEEDS=100 widens the search on a machine with time to spare)
@pytest.mark.parametrize("seed", range(int(os.environ.get("HPT_GUARDED_SEEDS", "8"))))
def test_ops_write_only_their_result(hpt, dev, hip, seed):
    rng = np.random.default_rng(77000 + seed)
    done = 0
    for it in range(40):
        shape = rand_shape(rng)
        ops = rand_view(rng, shape)
        base = rand_base(rng, shape)
        a = apply_view_np(base, ops)
        if a.size == 0:
            continue
        nd = a.ndim
        isz = base.itemsize
        pads = (int(rng.integers(0, 16 // isz)) * isz if rng.integers(0, 2) else 0,
                int(rng.integers(0, 16)) if rng.integers(0, 2) else 0)
        axes = sorted(int(x) for x in rng.choice(nd, int(rng.integers(1, nd + 1)), replace=False))
        what = f"seed={seed} case={it} shape={shape} view={ops} dtype={base.dtype} axes={axes} pads={pads}"
        run_guarded(hpt, hip, dev, rng, base, ops, ("sum", "max", "mul"), axes, pads, what)
        if base.dtype.kind == "f":
            run_guarded(hpt, hip, dev, rng, base, ops, ("softmax", "log_softmax"), [int(rng.integers(0, nd))], pads, what)
            run_guarded(hpt, hip, dev, rng, base, ops, ("layernorm",), list(range(nd - int(rng.integers(1, nd + 1)), nd)),
                        pads, what)
        done += 1
    assert done >= 20


F16, F32, F64, I32 = np.float16, np.float32, np.float64, np.int32
T = (("permute", (1, 0)),)
STEP2 = (("slice", ((0, None, 1), (0, None, 2))),)
# (parent shape, dtype, view, ops, axes): one case per kernel family and per row shape the planners tell
# apart, few rows each (the families are chosen by the row, not by the row count)
DIRECTED = [
    # rows in registers: short rows through LDS tiles, whole vectors, shifted, with an LDS half, streamed, split
    ((300, 33), F32, (), ("softmax", "layernorm", "sum", "max"), [1]),
    ((263, 128), F32, (), ("softmax", "layernorm", "sum"), [1]),
    ((37, 4097), F32, (), ("softmax", "layernorm", "sum"), [1]),
    ((9, 50257), F32, (), ("softmax", "log_softmax"), [1]),
    ((5, 70001), F32, (), ("softmax", "layernorm"), [1]),
    ((5, 65536), F32, (), ("softmax",), [1]),
    ((3, 65540), F32, (), ("softmax",), [1]),
    ((2, 1048576), F32, (), ("softmax", "layernorm", "sum"), [1]),
    ((35, 131072), F16, (), ("softmax",), [1]),
    ((5, 30522), F32, (), ("softmax", "log_softmax"), [1]),
    ((3, 128256), F32, (), ("softmax",), [1]),
    ((3, 100277), F32, (), ("log_softmax",), [1]),
    ((3, 151936), F16, (), ("softmax",), [1]),
    ((5, 32001), F16, (), ("softmax", "log_softmax"), [1]),
    ((5, 16392), F16, (), ("softmax",), [1]),
    # 3, 5, 6, 7 vectors per thread; gamma / beta through LDS for the two-byte types
    ((67, 768), F16, (), ("layernorm", "softmax"), [1]),
    ((67, 5120), F16, (), ("layernorm", "softmax"), [1]),
    ((67, 384), F16, (), ("layernorm",), [1]),
    ((67, 1024), F16, (), ("layernorm",), [1]),
    ((67, 1536), F32, (), ("softmax", "layernorm"), [1]),
    ((67, 2560), F32, (), ("softmax", "layernorm"), [1]),
    ((67, 6144), F32, (), ("softmax", "layernorm"), [1]),
    ((67, 7168), F32, (), ("softmax",), [1]),
    ((35, 10000), F32, (), ("softmax",), [1]),
    ((35, 12000), F32, (), ("softmax",), [1]),
    ((67, 16384), F32, (), ("log_softmax", "layernorm"), [1]),
    ((67, 4096), F64, (), ("softmax", "layernorm", "sum"), [1]),
    # every second element of a row
    ((67, 8192), F16, STEP2, ("softmax", "layernorm", "sum"), [1]),
    ((67, 8192), F16, STEP2, ("sum", "max"), [0]),
    # the axis strided: channels, a flat walk, column statistics, slabs, small groups
    ((3, 21, 50, 52), F32, (), ("softmax", "sum", "max"), [1]),
    ((1000, 3), F32, (), ("softmax", "sum"), [0]),
    ((517, 1024), F32, (), ("softmax", "sum"), [0]),
    ((512, 1000), F32, (), ("softmax", "sum"), [0]),
    ((9, 2048, 2), F32, (), ("softmax", "sum"), [1]),
    ((1000, 8, 32), F32, (), ("softmax", "sum"), [1]),
    # input contiguous along the rows (transposed), whole tiles and ragged ones
    ((264, 136), F16, T, ("softmax", "layernorm", "sum"), [1]),
    ((1024, 512), F16, T, ("softmax", "layernorm"), [1]),
    ((259, 131), F32, T, ("softmax", "layernorm", "sum"), [1]),
    # reductions: flat column walks, unaligned columns, narrow whole vectors, ragged and general rows
    ((10168, 33), F32, (), ("sum", "max"), [0]),
    ((819, 4097), F32, (), ("sum",), [0]),
    ((300, 257), F32, (), ("sum",), [0]),
    ((100, 33), I32, (), ("sum", "max"), [0]),
    ((40000, 8), F32, (), ("sum",), [0]),
    ((3355, 100), F32, (), ("sum",), [1]),
    ((1315, 257), F32, (), ("sum", "max"), [1]),
    ((7, 1023), F32, (), ("sum",), [1]),
    ((16, 8, 7, 7), F32, (), ("sum",), [0, 2, 3]),
    ((64, 32, 14, 14), F32, (), ("sum", "max"), [2, 3]),
    ((33554403 // 64,), F32, (), ("sum", "max"), [0]),
]


@pytest.mark.parametrize("case", range(len(DIRECTED)))
def test_each_kernel_family_writes_only_its_result(hpt, dev, hip, case):
    shape, dt, ops, names, axes = DIRECTED[case]
    rng = np.random.default_rng(500 + case)
    if np.dtype(dt).kind == "f":
        base = (rng.standard_normal(shape) * 2).astype(dt)
    else:
        base = rng.integers(-1000, 1000, shape).astype(dt)
    isz = base.itemsize
    for pads in ((0, 0), (isz, 1), (16 - isz, 3)):
        what = f"case={case} shape={shape} dtype={np.dtype(dt)} view={ops} axes={axes} pads={pads}"
        run_guarded(hpt, hip, dev, rng, base, ops, names, axes, pads, what)
