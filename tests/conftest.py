"""Shared pytest set-up: the `gpu` marker, import paths, and built libraries.

CPU tests (`-m "not gpu"`) check the oracle against golden vectors and the host
logic of libhpt_hip.so; GPU tests (`-m gpu`) are the parity tests and go through
the C ABI. Libraries are loaded as built; they are compiled here only when
nothing has been built yet.
"""
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def hpt():
    import hpt_amd
    from hpt_amd import _ffi, build
    if not _ffi.LIB_PATH.exists():
        build.build()
    hpt_amd.lib()
    return hpt_amd


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def dev(hpt):
    """Device 0 of a GPU box; GPU tests must fail, not skip, when the library cannot see it."""
    n = hpt.device_count()
    assert n >= 1, "no HIP device visible"
    return 0


def assert_close(got, want, rtol, atol, what=""):
    """|got - want| <= atol + rtol*|want|, NaN == NaN, inf by sign: the reference's allclose
    (hpt/src/backends/cpu/tensor_impls.rs:218-248)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} != {want.shape}"
    both_nan = np.isnan(got) & np.isnan(want)
    same_inf = np.isinf(got) & np.isinf(want) & (np.sign(got) == np.sign(want))
    with np.errstate(invalid="ignore"):
        ok = np.abs(got - want) <= atol + rtol * np.abs(want)
    ok = ok | both_nan | same_inf
    if not ok.all():
        bad = np.argwhere(~ok)
        i = tuple(bad[0])
        with np.errstate(invalid="ignore"):
            err = np.nanmax(np.abs(got - want)[~ok])
        raise AssertionError(f"{what}: {len(bad)} of {got.size} differ; first at {i}: got {got[i]!r}, "
                             f"want {want[i]!r}; max abs err {err:g} (rtol {rtol}, atol {atol})")
