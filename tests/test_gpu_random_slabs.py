"""Randomised parity over contiguous [B, C, L] tensors reduced or normalised over the middle axis: random inner dims
(2 ... 8, 12, 16), axis lengths from just over a wavefront to thousands, batch counts that put every case above the
size where the planner leaves the general kernels, random dtypes. The seeds are fixed; a failure names its case. The
shapes land on the interleaved and modular rows, the LDS slabs and group tiles, the register columns and the flat
walks, whichever the planner picks - the test only fixes the family of shapes, and checks every result against the
oracle."""
import numpy as np
import pytest

from conftest import assert_close
from util import F32_ATOL, F32_RTOL, HALF_RTOL, half_atol, upload

pytestmark = pytest.mark.gpu

CASES_PER_SEED = 12


def rand_case(rng):
    L = int(rng.choice([2, 2, 3, 3, 4, 4, 5, 6, 7, 8, 8, 12, 16]))
    C = int(rng.choice([int(rng.integers(65, 400)), int(rng.integers(400, 2100)), int(rng.integers(2100, 9000))]))
    if rng.integers(0, 2):  # slabs of whole vectors
        C = max(72, C // 8 * 8)
    npdt = [np.float32, np.float32, np.float16, np.float64, np.int32, np.uint8][int(rng.integers(0, 6))]
    elem = np.dtype(npdt).itemsize
    lo = (4 << 20) // (C * L * elem) + 1
    B = int(max(lo, 256, min(4 * lo, (48 << 20) // (C * L * elem))) * (1 + 0.3 * rng.random()))
    if rng.integers(0, 4) == 0:  # an outer batch dim that merges with the next
        return npdt, (2, (B + 1) // 2, C, L), 2
    return npdt, (B, C, L), 1


@pytest.mark.parametrize("seed", [7001, 7002, 7003, 7004, 7005, 7006])
def test_random_slabs(hpt, orc, dev, seed):
    rng = np.random.default_rng(seed)
    plans = set()
    for case in range(CASES_PER_SEED):
        npdt, shape, axis = rand_case(rng)
        L, C = shape[-1], shape[axis]
        tag = f"seed {seed} case {case}: {np.dtype(npdt).name} {list(shape)} axis {axis}"
        print(tag, flush=True)
        if np.issubdtype(npdt, np.floating):
            base = (rng.standard_normal(shape) * 2 + (np.arange(L) * 5.0 - 7.0)).astype(npdt)
        else:
            info = np.iinfo(npdt)
            base = rng.integers(max(info.min, -90), min(info.max, 90) + 1, shape).astype(npdt)
        # ties for the arg-reductions at both ends of the axis
        first = tuple(0 if i == axis else slice(None) for i in range(len(shape)))
        last = tuple(C - 1 if i == axis else slice(None) for i in range(len(shape)))
        top = np.asarray(base.max() + 1, dtype=np.float64).astype(npdt)
        base[first] = top
        base[last] = top
        t, a = upload(hpt, base, dev=dev)
        plans.add(hpt.reduce_plan(t, hpt.SUM, [axis]).split(" ")[0])
        assert np.array_equal(t.max([axis]).numpy(), a.max(axis)), tag
        assert np.array_equal(t.min([axis]).numpy(), a.min(axis)), tag
        assert np.array_equal(t.argmax(axis).numpy(), orc.argreduce(True, a, axis)), tag
        assert np.array_equal(t.argmin(axis).numpy(), orc.argreduce(False, a, axis)), tag
        if npdt == np.float16:
            want = orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F32).astype(np.float32)
            assert_close(t.sum([axis]).numpy().astype(np.float32), want, HALF_RTOL, half_atol(want, 11), tag + " sum")
        elif np.issubdtype(npdt, np.floating):
            rtol, atol = (F32_RTOL, 4 * F32_ATOL) if npdt == np.float32 else (1e-12, 1e-11)
            assert_close(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis], acc=orc.ACC_F64), rtol, atol, tag + " sum")
        else:
            assert np.array_equal(t.sum([axis]).numpy(), orc.reduce(orc.SUM, a, [axis])), tag
            continue
        plans.add(hpt.normalize_plan(t, axis).split(" ")[0])
        for log in (False, True):
            got = (t.log_softmax(axis) if log else t.softmax(axis)).numpy()
            if npdt == np.float16:
                want = orc.softmax(a, axis, log=log, acc=orc.ACC_F32).astype(np.float32)
                assert_close(got.astype(np.float32), want, HALF_RTOL, max(half_atol(want, 11), 6e-8), tag + f" softmax log={log}")
            elif npdt == np.float32:
                assert_close(got, orc.softmax(a, axis, log=log, acc=orc.ACC_F64), F32_RTOL, F32_ATOL, tag + f" softmax log={log}")
            else:
                assert_close(got, orc.softmax(a, axis, log=log, acc=orc.ACC_F64), 1e-12, 1e-14, tag + f" softmax log={log}")
        del t
    print(f"seed {seed}: plans {sorted(plans)}", flush=True)
