"""The GPU path against the committed golden vectors (torch float64 results, tests/golden)."""
import numpy as np
import pytest

from conftest import assert_close
from test_oracle_numerics import cases, gold, load_case
from util import apply_view_t

pytestmark = pytest.mark.gpu


def dev_view(hpt, dev, base, ops):
    return apply_view_t(hpt.Tensor.from_numpy(base).to_hip(dev), ops)


@pytest.mark.parametrize("name", cases("softmax/"))
def test_softmax_golden(hpt, dev, name):
    base, ops, v = load_case(name)
    axis = int(gold()[name + "/axis"])
    t = dev_view(hpt, dev, base, ops)
    assert_close(t.softmax(axis).numpy(), gold()[name + "/softmax"], 1e-5, 1e-6, name)
    assert_close(t.log_softmax(axis).numpy(), gold()[name + "/log_softmax"], 1e-5, 1e-6, name + " log")


@pytest.mark.parametrize("name", cases("layernorm/"))
def test_layernorm_golden(hpt, dev, name):
    base, ops, v = load_case(name)
    g = gold()
    nn = int(g[name + "/n_norm"])
    t = dev_view(hpt, dev, base, ops)
    ns = t.shape[t.ndim - nn:]
    tg = hpt.Tensor.from_numpy(g[name + "/gamma"]).to_hip(dev)
    tb = hpt.Tensor.from_numpy(g[name + "/beta"]).to_hip(dev)
    assert_close(t.layernorm(ns, tg, tb, 1e-5).numpy(), g[name + "/out"], 1e-5, 1e-6, name)
    assert_close(t.layernorm(ns, None, None, 1e-5).numpy(), g[name + "/out_plain"], 1e-5, 1e-6, name + " plain")


@pytest.mark.parametrize("name", cases("reduce/"))
def test_reduce_golden(hpt, dev, name):
    base, ops, v = load_case(name)
    g = gold()
    axes = [int(a) for a in g[name + "/axes"]]
    t = dev_view(hpt, dev, base, ops)
    for op in ("sum", "mean", "max", "min", "sum_square", "reducel1", "reducel2", "reducel3"):
        want = np.atleast_1d(g[f"{name}/{op}"]).reshape(-1)
        got = getattr(t, op)(axes).numpy().reshape(-1)
        assert_close(got, want, 1e-5, 1e-6, f"{name} {op}")


@pytest.mark.parametrize("name", cases("argreduce"))
def test_argreduce_golden(hpt, dev, name):
    base, ops, v = load_case(name)
    axis = int(gold()[name + "/axis"])
    t = dev_view(hpt, dev, base, ops)
    assert np.array_equal(t.argmax(axis).numpy(), gold()[name + "/argmax"])
    assert np.array_equal(t.argmin(axis).numpy(), gold()[name + "/argmin"])


@pytest.mark.parametrize("name", cases("reduce_i32/"))
def test_reduce_i32_golden(hpt, dev, name):
    base, ops, v = load_case(name)
    axes = [int(a) for a in gold()[name + "/axes"]]
    t = dev_view(hpt, dev, base, ops)
    assert np.array_equal(t.sum(axes).numpy().reshape(-1), np.atleast_1d(gold()[name + "/sum"]).reshape(-1))
    assert np.array_equal(t.max(axes).numpy().reshape(-1), np.atleast_1d(gold()[name + "/max"]).reshape(-1))
