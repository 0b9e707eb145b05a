"""The device caching allocator and the transfers behind to_hip / to_cpu (through the C ABI).

Behaviour under test follows hpt-allocator: blocks keyed by (size, align), freed blocks cached
in an LRU of layouts, eviction releases a layout's blocks (allocators/cuda.rs:41-322,
utils/allocate.rs:15-130, utils/deallocate.rs:11-32)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def stats(hpt, dev):
    a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
    assert hpt.lib().hpt_hip_alloc_stats(dev, C.byref(a), C.byref(b), C.byref(c)) == 0
    return a.value, b.value, c.value


def alloc(hpt, dev, n, align=64, zeroed=0):
    from hpt_amd import _ffi
    p = C.c_void_p()
    _ffi.check(hpt.lib().hpt_hip_alloc(dev, n, align, zeroed, C.byref(p)))
    return p.value


def free(hpt, dev, p, n, align=64):
    from hpt_amd import _ffi
    _ffi.check(hpt.lib().hpt_hip_free(dev, C.c_void_p(p), n, align))


def test_cache_hit_reuses_the_block(hpt, dev):
    import gc
    gc.collect()
    l = hpt.lib()
    assert l.hpt_hip_cache_clear(dev) == 0
    live0, cached0, mallocs0 = stats(hpt, dev)
    assert cached0 == 0
    p = alloc(hpt, dev, 1 << 20)
    assert p % 64 == 0
    assert stats(hpt, dev) == (live0 + 1, 0, mallocs0 + 1)
    free(hpt, dev, p, 1 << 20)
    assert stats(hpt, dev) == (live0, 1, mallocs0 + 1)
    q = alloc(hpt, dev, 1 << 20)
    assert q == p                                   # same layout -> the cached block, no hipMalloc
    assert stats(hpt, dev) == (live0 + 1, 0, mallocs0 + 1)
    r = alloc(hpt, dev, (1 << 20) + 64)             # another layout -> a fresh block
    assert r != p and stats(hpt, dev)[2] == mallocs0 + 2
    free(hpt, dev, q, 1 << 20)
    free(hpt, dev, r, (1 << 20) + 64)
    assert l.hpt_hip_cache_clear(dev) == 0
    assert stats(hpt, dev)[:2] == (live0, 0)


def test_lru_eviction_and_resize(hpt, dev):
    l = hpt.lib()
    assert l.hpt_hip_cache_clear(dev) == 0
    assert l.hpt_hip_cache_resize(dev, 2) == 0
    sizes = [4096, 8192, 12288]
    ptrs = [alloc(hpt, dev, s) for s in sizes]
    for p, s in zip(ptrs, sizes):
        free(hpt, dev, p, s)                         # third layout evicts the least recently used (4096)
    assert stats(hpt, dev)[1] == 2
    m0 = stats(hpt, dev)[2]
    a = alloc(hpt, dev, 8192)
    b = alloc(hpt, dev, 12288)
    assert stats(hpt, dev)[2] == m0                  # both still cached
    c = alloc(hpt, dev, 4096)
    assert stats(hpt, dev)[2] == m0 + 1              # evicted earlier -> hipMalloc again
    for p, s in ((a, 8192), (b, 12288), (c, 4096)):
        free(hpt, dev, p, s)
    assert l.hpt_hip_cache_resize(dev, 0) == 0       # capacity 0: nothing stays cached
    assert stats(hpt, dev)[1] == 0
    assert l.hpt_hip_cache_resize(dev, 100) == 0


def test_zeroed_and_errors(hpt, dev):
    from hpt_amd import _ffi
    p = alloc(hpt, dev, 4096)
    junk = np.full(4096, 0xAB, np.uint8)
    _ffi.check(hpt.lib().hpt_hip_memcpy_h2d_sync(dev, C.c_void_p(p), C.c_void_p(junk.ctypes.data), 4096))
    free(hpt, dev, p, 4096)
    q = alloc(hpt, dev, 4096, zeroed=1)              # the recycled block must come back zeroed
    back = np.empty(4096, np.uint8)
    _ffi.check(hpt.lib().hpt_hip_memcpy_d2h_sync(dev, C.c_void_p(back.ctypes.data), C.c_void_p(q), 4096))
    assert not back.any()
    with pytest.raises(hpt.MemoryError_, match="layout mismatch"):
        free(hpt, dev, q, 8192)
    free(hpt, dev, q, 4096)
    with pytest.raises(hpt.MemoryError_, match="was not allocated"):
        free(hpt, dev, q, 4096)                      # double free
    with pytest.raises(hpt.ParamError):
        alloc(hpt, dev, 64, align=48)
    with pytest.raises(hpt.DeviceError):
        alloc(hpt, 1 << 10, 64)
    with pytest.raises(hpt.MemoryError_, match="Failed to allocate"):
        alloc(hpt, dev, 1 << 50)                     # 1 PiB: must fail cleanly after emptying the cache


def test_round_trip_and_tensor_lifetime(hpt, dev):
    import gc
    rng = np.random.default_rng(300)
    for d in hpt.DTYPES:
        a = rng.integers(0, 200, (13, 7, 5)).astype(d.np_dtype)
        t = hpt.Tensor.from_numpy(a, d).to_hip(dev)
        assert np.array_equal(t.to_cpu().numpy(), a)
        assert np.array_equal(t.permute([2, 0, 1])[1:, ::2].numpy(), a.transpose(2, 0, 1)[1:, ::2])
    del t
    gc.collect()
    live0 = stats(hpt, dev)[0]
    t = hpt.Tensor.from_numpy(np.ones((64, 64), np.float32)).to_hip(dev)
    v = t.permute([1, 0])[::2]
    assert stats(hpt, dev)[0] == live0 + 1
    del t
    gc.collect()
    assert stats(hpt, dev)[0] == live0 + 1           # the view keeps the storage alive
    assert v.sum([0, 1]).numpy()[0] == 64 * 32
    del v
    gc.collect()
    assert stats(hpt, dev)[0] == live0


def test_storage_is_freed_after_its_stream_is_gone(hpt, dev):
    """A tensor used on a caller's stream that the caller destroys before the tensor dies: the per-stream wait
    can fail, the whole device is waited for instead, and the block still goes back to the allocator."""
    import gc
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    gc.collect()
    live0 = stats(hpt, dev)[0]
    s = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(s)) == 0
    x = np.random.default_rng(3).standard_normal((64, 4096)).astype(np.float32)
    t = hpt.Tensor.from_numpy(x).to_hip(dev)
    y = t.softmax(1, stream=s)
    z = t.sum([0, 1], stream=s)     # a split reduction: per-stream scratch as well
    assert hip.hipStreamSynchronize(s) == 0
    got = y.numpy()
    assert abs(float(got.sum()) - 64.0) < 1e-3
    assert hip.hipStreamDestroy(s) == 0
    assert stats(hpt, dev)[0] >= live0 + 3
    del t, y, z
    gc.collect()
    assert stats(hpt, dev)[0] == live0, "blocks used on a destroyed stream were not returned"


def test_device_synchronize_and_device_checks(hpt, dev):
    l = hpt.lib()
    assert l.hpt_hip_device_synchronize(dev) == 0
    n = hpt.device_count()
    for bad in (-1, n, n + 7):
        assert l.hpt_hip_device_synchronize(bad) != 0
        assert b"does not exist" in l.hpt_hip_last_error()
        # forget validates the device like free does (a foreign pointer is otherwise left alone)
        assert l.hpt_hip_forget(bad, C.c_void_p(0x1000)) != 0
    assert l.hpt_hip_forget(dev, C.c_void_p(0x1000)) == 0


def test_cache_clear_while_other_threads_reduce(hpt, orc, dev):
    """cache_clear hands the scratch buffers back while other host threads keep running split reductions (which use
    them): every result stays right, and nothing is handed out twice."""
    import threading
    rng = np.random.default_rng(5)
    xs = [rng.integers(-1000, 1001, (3, 1 << 18)).astype(np.int32) for _ in range(3)]
    want = [x.sum(dtype=np.int32) for x in xs]
    errors, stop = [], threading.Event()

    def worker(k):
        try:
            t = hpt.Tensor.from_numpy(xs[k]).to_hip(dev)
            while not stop.is_set():
                got = t.sum([0, 1]).numpy()
                if int(got[0]) != int(want[k]):
                    errors.append((k, int(got[0]), int(want[k])))
                    return
        except Exception as e:  # noqa: BLE001
            errors.append((k, repr(e)))

    th = [threading.Thread(target=worker, args=(k,)) for k in range(3)]
    for t in th:
        t.start()
    try:
        for _ in range(40):
            assert hpt.lib().hpt_hip_cache_clear(dev) == 0
    finally:
        stop.set()
        for t in th:
            t.join()
    assert not errors, errors[:3]
