"""The C ABI from several host threads at once, on the default stream and on caller-made streams: every
entry must be callable concurrently (Hpt calls it from rayon workers), launches on one stream stay ordered,
and each stream has its own scratch for the split reductions."""
import ctypes as C
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_concurrent_callers_and_streams(hpt, dev):
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    rng = np.random.default_rng(600)
    nthreads, iters = 8, 40
    data, want = [], []
    for k in range(nthreads):
        x = rng.standard_normal((257 + k, 1536)).astype(np.float32)
        xi = rng.integers(-1000, 1000, (64, 33 + k, 49)).astype(np.int32)
        t, ti = hpt.Tensor.from_numpy(x).to_hip(dev), hpt.Tensor.from_numpy(xi).to_hip(dev)
        data.append((t, ti))
        # single-threaded results first: the kernels are deterministic, so concurrent runs must repeat them bit for bit
        want.append((t.sum([0, 1]).numpy(), t.softmax(1).numpy(), t.layernorm([1536]).numpy(),
                     ti.sum([1]).numpy(), ti.argmax(1).numpy(), t.permute([1, 0]).contiguous().numpy(),
                     t.permute([1, 0]).softmax(1).numpy()))
    assert np.array_equal(want[0][3], np.asarray(data[0][1].numpy()).sum(1, dtype=np.int32))
    streams = []
    for k in range(nthreads):
        s = C.c_void_p()
        if k % 2:
            assert hip.hipStreamCreate(C.byref(s)) == 0
        streams.append(s if k % 2 else None)
    errors = []

    def work(k):
        try:
            t, ti = data[k]
            st = streams[k]
            for it in range(iters):
                got = (t.sum([0, 1], stream=st), t.softmax(1, stream=st), t.layernorm([1536], stream=st),
                       ti.sum([1], stream=st), ti.argmax(1, stream=st), t.permute([1, 0]).contiguous(stream=st),
                       t.permute([1, 0]).softmax(1, stream=st))
                hpt.synchronize(dev, st)
                for g, w in zip(got, want[k]):
                    if not np.array_equal(g.numpy(), w, equal_nan=True):
                        raise AssertionError(f"thread {k} iteration {it}: result differs from the single-threaded run")
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append(e)

    threads = [threading.Thread(target=work, args=(k,)) for k in range(nthreads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    hpt.synchronize(dev)
    for s in streams:
        if s is not None:
            hip.hipStreamDestroy(s)
    assert not errors, errors[0]
