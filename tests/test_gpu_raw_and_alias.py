"""Memory the library did not allocate, tensors given up to the caller, and outputs that share
memory with an input.

  * Tensor::from_raw / forget / allclose (hpt/src/backends/cpu/tensor_impls.rs:123-147, 218-248, 320;
    hpt/src/backends/cuda/tensor_impls.rs:259-306): every entry point must take a device pointer from
    a plain hipMalloc at any element-aligned address, and dropping the adopting tensor frees nothing.
  * `out` may be the input itself for the normalisations (one contiguous tensor, in place).
  * The stream a result was produced on is waited for before the result is copied or its block reused.
"""
import ctypes as C
import threading

import numpy as np
import pytest

from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol
from conftest import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    h = C.CDLL("libamdhip64.so")
    h.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    h.hipFree.argtypes = [C.c_void_p]
    h.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    h.hipStreamCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
    h.hipStreamDestroy.argtypes = [C.c_void_p]
    h.hipDeviceSynchronize.argtypes = []
    return h


def stats(hpt, dev):
    a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
    assert hpt.lib().hpt_hip_alloc_stats(dev, C.byref(a), C.byref(b), C.byref(c)) == 0
    return a.value, b.value, c.value


def raw_upload(hip, arr, offset_bytes):
    """hipMalloc a buffer, place `arr` at `offset_bytes` inside it; returns (base pointer, data pointer)."""
    p = C.c_void_p()
    assert hip.hipMalloc(C.byref(p), arr.nbytes + offset_bytes + 256) == 0
    arr = np.ascontiguousarray(arr)
    assert hip.hipMemcpy(C.c_void_p(p.value + offset_bytes), C.c_void_p(arr.ctypes.data), arr.nbytes, 1) == 0
    return p.value, p.value + offset_bytes


@pytest.mark.parametrize("np_dt,off", [(np.float16, 2), (np.float16, 6), (np.float32, 4), (np.float32, 36)],
                         ids=["f16+2", "f16+6", "f32+4", "f32+36"])
def test_from_raw_on_an_interior_odd_aligned_pointer(hpt, orc, dev, hip, np_dt, off):
    import gc
    rng = np.random.default_rng(31)
    shape = (257, 1000)
    x = (rng.standard_normal(shape) * 2).astype(np_dt)
    g = rng.normal(1, 0.1, shape[1]).astype(np_dt)
    b = rng.normal(0, 0.1, shape[1]).astype(np_dt)
    base, ptr = raw_upload(hip, x, off)
    gbase, gptr = raw_upload(hip, g, off)
    bbase, bptr = raw_upload(hip, b, off)
    dt = hpt.f16 if np_dt == np.float16 else hpt.f32
    gc.collect()
    before = stats(hpt, dev)
    t = hpt.Tensor.from_raw(ptr, shape, dt, dev)
    tg = hpt.Tensor.from_raw(gptr, (shape[1],), dt, dev)
    tb = hpt.Tensor.from_raw(bptr, (shape[1],), dt, dev)
    assert ptr % 16 != 0 and t.is_contiguous()
    half = np_dt == np.float16
    acc = orc.ACC_F32 if half else orc.ACC_F64
    rtol = HALF_RTOL if half else F32_RTOL

    def tol(want):
        return half_atol(want, 11) if half else F32_ATOL

    for axes in ([1], [0], [0, 1]):
        want = orc.reduce(orc.SUM, x, axes, acc=acc)
        assert_close(t.sum(axes).numpy(), want, rtol, tol(want) * (4 if half else 30), f"sum{axes}")
        assert np.array_equal(t.max(axes).numpy().reshape(-1), x.max(tuple(axes)).reshape(-1))
    for axis in (0, 1):
        assert np.array_equal(t.argmax(axis).numpy(), orc.argreduce(True, x, axis)), f"argmax({axis})"
        want = orc.softmax(x, axis, acc=acc)
        assert_close(t.softmax(axis).numpy(), want, rtol, tol(want), f"softmax({axis})")
    want = orc.layernorm(x, 1, g, b, 1e-5, acc=acc)
    assert_close(t.layernorm([shape[1]], tg, tb, 1e-5).numpy(), want, rtol, 2 * tol(want), "layernorm")
    # a strided view of foreign memory: every second column, and the transposed matrix
    v = hpt.Tensor.from_raw(ptr, (shape[0], shape[1] // 2), dt, dev, strides=[shape[1], 2])
    want = orc.softmax(x[:, ::2], 1, acc=acc)
    assert_close(v.softmax(1).numpy(), want, rtol, tol(want), "softmax of a stepped raw view")
    vt = hpt.Tensor.from_raw(ptr, (shape[1], shape[0]), dt, dev, strides=[1, shape[1]])
    assert np.array_equal(vt.contiguous().numpy(), x.T)
    assert np.array_equal(vt.numpy(), x.T)
    # results written INTO foreign memory
    obase, optr = raw_upload(hip, np.zeros(shape, np_dt), off)
    o = hpt.Tensor.from_raw(optr, shape, dt, dev)
    t.softmax(1, out=o)
    want = orc.softmax(x, 1, acc=acc)
    assert_close(o.numpy(), want, rtol, tol(want), "softmax into raw memory")
    # dropping the adopting tensors frees nothing: no live block appears or disappears
    hpt.synchronize(dev)
    del t, tg, tb, v, vt, o
    gc.collect()
    after = stats(hpt, dev)
    assert after[0] == before[0], "live blocks changed by tensors over foreign memory"
    # the memory is still the caller's: reading it back gives the input
    back = np.empty(shape, np_dt)
    assert hip.hipMemcpy(C.c_void_p(back.ctypes.data), C.c_void_p(ptr), back.nbytes, 2) == 0
    assert np.array_equal(back, x)
    for p in (base, gbase, bbase, obase):
        assert hip.hipFree(C.c_void_p(p)) == 0


def test_from_raw_argument_errors(hpt, dev):
    with pytest.raises(hpt.ParamError, match="data is null"):
        hpt.Tensor.from_raw(0, (4,), hpt.f32, dev)
    with pytest.raises(hpt.ParamError, match="not aligned"):
        hpt.Tensor.from_raw(4098, (4,), hpt.f32, dev)
    with pytest.raises(hpt.ShapeError):
        hpt.Tensor.from_raw(4096, (4, 4), hpt.f32, dev, strides=[1])


def test_forget_hands_the_block_to_the_caller(hpt, dev, hip):
    import gc
    gc.collect()
    x = np.arange(4096, dtype=np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    live0, cached0, _ = stats(hpt, dev)
    with pytest.raises(hpt.ParamError, match="tensor is a view"):
        t[1:].forget()
    alias = hpt.Tensor(t._storage, t.ptr, t.shape, t.strides, t.dtype, "hip", dev)
    with pytest.raises(hpt.ParamError, match="ref_count: 2"):
        t.forget()
    del alias
    ptr, (nbytes, align) = t.forget()
    assert (nbytes, align) == (x.nbytes, 64) and ptr % 64 == 0
    assert t.size() == 0
    live1, cached1, _ = stats(hpt, dev)
    assert (live1, cached1) == (live0 - 1, cached0), "forget must neither cache nor keep tracking the block"
    del t
    gc.collect()
    assert stats(hpt, dev)[:2] == (live1, cached1)
    # the allocator no longer knows the pointer: freeing it through the library is an error ...
    assert hpt.lib().hpt_hip_free(dev, C.c_void_p(ptr), nbytes, align) == hpt._ffi.ERR_MEMORY
    # ... the data is intact, usable through from_raw, and the caller's to release
    r = hpt.Tensor.from_raw(ptr, (4096,), hpt.f32, dev)
    assert float(r.sum([0]).numpy()[0]) == float(x.astype(np.float64).sum())
    del r
    assert hip.hipFree(C.c_void_p(ptr)) == 0
    # forgetting a pointer the allocator never had is a no-op, as in the reference
    assert hpt.lib().hpt_hip_forget(dev, C.c_void_p(12345 * 64)) == 0


def test_allclose_follows_the_reference(hpt, dev):
    a = np.array([[1.0, np.nan, np.inf, -np.inf, 100.0, 0.0]], np.float32)
    ta = hpt.Tensor.from_numpy(a).to_hip(dev)
    assert ta.allclose(ta, 0.0, 0.0)
    b = a.copy()
    b[0, 4] = 100.5
    tb = hpt.Tensor.from_numpy(b).to_hip(dev)
    assert not ta.allclose(tb, 1e-3, 0.0)       # 0.5 > 1e-3 * 100.5
    assert ta.allclose(tb, 1e-2, 0.0)           # tolerance scales with |other|
    assert ta.allclose(tb, 0.0, 0.6)
    c = a.copy()
    c[0, 2] = -np.inf                           # infinities of opposite sign
    assert not ta.allclose(hpt.Tensor.from_numpy(c).to_hip(dev), 1.0, 1.0)
    d = a.copy()
    d[0, 1] = 3.0                               # NaN against a number
    assert not ta.allclose(hpt.Tensor.from_numpy(d).to_hip(dev), 1.0, 1.0)
    assert not ta.allclose(hpt.Tensor.from_numpy(a.reshape(6, 1)).to_hip(dev), 1.0, 1.0)   # shapes differ
    # views and half types go through to_cpu like any other
    h = np.linspace(-4, 4, 64, dtype=np.float16).reshape(8, 8)
    th = hpt.Tensor.from_numpy(h).to_hip(dev)
    assert th.permute([1, 0]).allclose(hpt.Tensor.from_numpy(np.ascontiguousarray(h.T)).to_hip(dev), 0.0, 0.0)


IN_PLACE = [
    # (name, np dtype, shape, what)
    ("rows in registers f32", np.float32, (1024, 4096)),
    ("odd rows f32", np.float32, (2051, 257)),
    ("short rows through LDS f32", np.float32, (150000, 33)),
    ("long rows streamed f32", np.float32, (24, 70001)),
    ("few long rows split f32", np.float32, (8, 600000)),
    ("rows in registers f16", np.float16, (4096, 2048)),
    ("vocabulary rows f16", np.float16, (64, 50257)),
]


@pytest.mark.parametrize("name,np_dt,shape", IN_PLACE, ids=[c[0] for c in IN_PLACE])
def test_normalisations_in_place_over_one_contiguous_tensor(hpt, dev, name, np_dt, shape):
    rng = np.random.default_rng(77)
    x = (rng.standard_normal(shape) * 3).astype(np_dt)
    g = rng.normal(1, 0.1, shape[-1]).astype(np_dt)
    b = rng.normal(0, 0.1, shape[-1]).astype(np_dt)
    tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
    src = hpt.Tensor.from_numpy(x).to_hip(dev)
    for what in ("softmax", "log_softmax", "layernorm", "softmax0"):
        if what == "softmax0" and shape[0] * shape[1] > 30_000_000:
            continue
        t = src.contiguous()
        if what == "layernorm":
            want = src.layernorm([shape[-1]], tg, tb, 1e-5).numpy()
            got = t.layernorm([shape[-1]], tg, tb, 1e-5, out=t)
        elif what == "softmax0":
            want = src.softmax(0).numpy()
            got = t.softmax(0, out=t)
        else:
            want = getattr(src, what)(1).numpy()
            got = getattr(t, what)(1, out=t)
        assert got is t
        assert t.numpy().tobytes() == want.tobytes(), f"{name}: {what} in place differs from out of place"
    # in place over a view of the same buffer is refused (here: the transposed matrix into itself)
    if shape[0] == shape[1]:
        return
    t = src.contiguous()
    flat = hpt.Tensor(t._storage, t.ptr, [shape[1], shape[0]], [shape[0], 1], t.dtype, "hip", dev)
    with pytest.raises(hpt.ParamError, match="overlaps"):
        t.permute([1, 0]).softmax(1, out=flat)


def test_results_on_a_callers_stream_are_waited_for(hpt, orc, dev, hip):
    """Integer inputs of softmax / layernorm go through a promoted temporary; on a non-blocking caller
    stream nothing but the host mirror's own bookkeeping keeps that temporary (and the result) from
    being reused or read early while another thread allocates the very same layouts."""
    st = C.c_void_p()
    assert hip.hipStreamCreateWithFlags(C.byref(st), 1) == 0  # hipStreamNonBlocking
    rng = np.random.default_rng(5)
    shape = (2048, 4096)
    xi = rng.integers(-8, 9, shape).astype(np.int32)
    want_s = orc.softmax(xi.astype(np.float32), 1, acc=orc.ACC_F64)
    want_l = orc.layernorm(xi.astype(np.float32), 1, None, None, 1e-5, acc=orc.ACC_F64)
    ti = hpt.Tensor.from_numpy(xi).to_hip(dev)
    stop = threading.Event()
    errors = []

    def churn():
        # same (bytes, align) layouts as the promoted temporary and the result, refilled at once
        try:
            while not stop.is_set():
                z = hpt.Tensor.full(1e30, shape, hpt.f32, dev)
                del z
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    th = threading.Thread(target=churn)
    th.start()
    try:
        for _ in range(25):
            got = ti.softmax(1, stream=st)
            assert_close(got.numpy(), want_s, F32_RTOL, F32_ATOL, "i32 softmax on a caller stream")
            got = ti.layernorm([shape[1]], stream=st)
            assert_close(got.numpy(), want_l, F32_RTOL, 2 * F32_ATOL, "i32 layernorm on a caller stream")
            got = ti.permute([1, 0]).sum([0], stream=st)
            assert np.array_equal(got.to_cpu().numpy(), xi.sum(1, dtype=np.int32))
    finally:
        stop.set()
        th.join()
        hpt.synchronize(dev, st)
        hpt.synchronize(dev)
        hip.hipStreamDestroy(st)
    assert not errors, errors[0]


def test_split_reductions_on_two_streams_at_once(hpt, dev, hip):
    """Each stream has its own scratch buffer and lock: two threads running full reductions (partials
    in scratch) of different sizes on their own streams, one growing its scratch on the way."""
    rng = np.random.default_rng(9)
    sizes = [[1 << 20, 3_000_001, 12_582_912], [5_000_003, 1 << 22, 20_000_000]]
    data, want = [], []
    for k in range(2):
        row = []
        for n in sizes[k]:
            x = rng.standard_normal(n).astype(np.float32)
            t = hpt.Tensor.from_numpy(x).to_hip(dev)
            cols = hpt.Tensor.from_numpy(x[: (n // 4096) * 4096].reshape(-1, 4096)).to_hip(dev)
            row.append((t, cols))
        data.append(row)
        want.append([(t.sum([0]).numpy(), t.max([0]).numpy(), c.sum([0]).numpy()) for t, c in row])
    streams = []
    for k in range(2):
        s = C.c_void_p()
        assert hip.hipStreamCreateWithFlags(C.byref(s), 1) == 0
        streams.append(s)
    errors = []

    def work(k):
        try:
            for it in range(30):
                for (t, c), w in zip(data[k], want[k]):
                    got = (t.sum([0], stream=streams[k]), t.max([0], stream=streams[k]), c.sum([0], stream=streams[k]))
                    for g, ww in zip(got, w):
                        if g.numpy().tobytes() != ww.tobytes():
                            raise AssertionError(f"stream {k} iteration {it}: split reduction differs from the single run")
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    ths = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for th in ths:
        th.start()
    for th in ths:
        th.join()
    hpt.synchronize(dev)
    for s in streams:
        hip.hipStreamDestroy(s)
    assert not errors, errors[0]
    # the scratch buffers came from the caching allocator: a caller never sees them as live blocks,
    # and cache_clear releases them with everything else
    import gc
    del data, row, t, cols
    gc.collect()
    live = stats(hpt, dev)[0]
    assert hpt.lib().hpt_hip_cache_clear(dev) == 0
    assert stats(hpt, dev)[:2] == (live, 0)
    # and the next split reduction simply takes a new one
    x = rng.standard_normal(1 << 20).astype(np.float32)
    got = hpt.Tensor.from_numpy(x).to_hip(dev).sum([0]).numpy()
    import math
    want = float(np.float32(math.fsum(x.astype(np.float64))))
    assert abs(float(got[0]) - want) <= 1e-6 + 1e-5 * abs(want)
