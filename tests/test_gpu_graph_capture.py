"""Entry points that allocate nothing under HIP graph capture: a layernorm (rows in registers: no scratch)
and a full sum through hpt_hip_reduce_static (two kernels, partials in the static device array) are captured
once on a caller's stream and replayed with new inputs. Between replays the program does ordinary eager work
and synchronises; every replay is checked against the oracle and against the same calls made eagerly."""
import ctypes as C

import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL

pytestmark = pytest.mark.gpu

HIP_STREAM_NON_BLOCKING = 1
HIP_STREAM_CAPTURE_MODE_RELAXED = 2


def test_layernorm_and_static_sum_replayed_from_a_graph(hpt, orc, dev):
    from hpt_amd import _ffi
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreateWithFlags.argtypes = [C.POINTER(C.c_void_p), C.c_uint]
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    l = hpt.lib()

    rng = np.random.default_rng(77)
    rows, cols = 512, 1024
    host = [(rng.standard_normal((rows, cols)) * 2 + k).astype(np.float32) for k in range(4)]
    g = rng.normal(1, 0.1, cols).astype(np.float32)
    b = rng.normal(0, 0.1, cols).astype(np.float32)
    x = hpt.Tensor.from_numpy(host[0]).to_hip(dev)
    tg, tb = hpt.Tensor.from_numpy(g).to_hip(dev), hpt.Tensor.from_numpy(b).to_hip(dev)
    y = hpt.Tensor.empty([rows, cols], hpt.f32, dev)
    z = hpt.Tensor.empty([1], hpt.f32, dev)

    s = C.c_void_p()
    assert hip.hipStreamCreateWithFlags(C.byref(s), HIP_STREAM_NON_BLOCKING) == 0

    def enqueue():
        x.layernorm([cols], tg, tb, 1e-5, stream=s, out=y)
        y._reduce(hpt.SUM if hasattr(hpt, "SUM") else 0, [0, 1], False, out=z, stream=s, static_scratch=True)

    # eagerly once: the static array's address is looked up on the first call on a device
    enqueue()
    assert hip.hipStreamSynchronize(s) == 0
    eager_y, eager_z = y.numpy().copy(), z.numpy().copy()
    assert "split=" in hpt.reduce_plan(y, 0, [0, 1]) and "split=1(" not in hpt.reduce_plan(y, 0, [0, 1]), \
        "the captured sum is meant to be a two-kernel reduction with partials in scratch"

    assert hip.hipStreamBeginCapture(s, HIP_STREAM_CAPTURE_MODE_RELAXED) == 0
    try:
        enqueue()
    finally:
        graph = C.c_void_p()
        rc = hip.hipStreamEndCapture(s, C.byref(graph))
    assert rc == 0 and graph.value, f"hipStreamEndCapture failed ({rc})"
    gexec = C.c_void_p()
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0

    try:
        for k in (1, 2, 3, 0):
            # eager work between the replays: a new input into the captured buffer, outputs cleared, an
            # unrelated split reduction on the default stream (it takes the ordinary, per-stream scratch)
            _ffi.check(l.hpt_hip_memcpy_h2d_sync(dev, C.c_void_p(x.ptr), C.c_void_p(host[k].ctypes.data), host[k].nbytes))
            junk = np.full((rows, cols), np.nan, np.float32)
            _ffi.check(l.hpt_hip_memcpy_h2d_sync(dev, C.c_void_p(y.ptr), C.c_void_p(junk.ctypes.data), junk.nbytes))
            other = hpt.Tensor.from_numpy(host[(k + 1) % 4]).to_hip(dev)
            assert_close(other.sum([0, 1]).numpy(), orc.reduce(orc.SUM, host[(k + 1) % 4], [0, 1], acc=orc.ACC_EXACT),
                         F32_RTOL, F32_ATOL, "eager sum between replays")
            hpt.synchronize(dev)
            assert hip.hipGraphLaunch(gexec, s) == 0
            assert hip.hipStreamSynchronize(s) == 0
            want_y = orc.layernorm(host[k], 1, g, b, 1e-5, acc=orc.ACC_F64)
            got_y, got_z = y.numpy(), z.numpy()
            assert_close(got_y, want_y, F32_RTOL, F32_ATOL, f"replayed layernorm, input {k}")
            # (the sum is taken of the f32 values the layernorm stored: that is its truth)
            assert_close(got_z, np.array([got_y.astype(np.float64).sum()], np.float32), F32_RTOL, F32_ATOL, f"replayed sum, input {k}")
            # the eager calls on the same input give the same bits
            enqueue()
            assert hip.hipStreamSynchronize(s) == 0
            assert np.array_equal(y.numpy(), got_y) and np.array_equal(z.numpy(), got_z), f"replay and eager differ, input {k}"
            if k == 0:
                assert np.array_equal(got_y, eager_y) and np.array_equal(got_z, eager_z)
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(s)
