"""Pins the softmax-family oracle (oracle/softmax_family_oracle.c) with the values the reference's
docstrings and tests hold, with closed forms evaluated independently in numpy, and with finite
differences for the two gradients."""
import numpy as np
import pytest

import reference_cases as R

G = R.softmax_family_gold()


def _np_softmax(x, axes):
    e = np.exp(x - x.max(axis=axes, keepdims=True))
    return e / e.sum(axis=axes, keepdims=True)


def test_doctest_and_inf_tables(oracle):
    d = G["doctest_matrix_dims2"]
    assert np.allclose(oracle.softmax(R.rows(d["x_rows"]), dims=2), R.rows(d["y_rows"]), atol=1e-6)
    t = G["inf_table_other_dims"]                                     # test/softmax.jl:68-70
    x = R.rows(t["x_rows"])
    for dt in (np.float32, np.float64):
        assert np.allclose(oracle.softmax(x, dims=2, dtype=dt), R.rows(t["dims2"]), atol=1e-6)
        assert np.allclose(oracle.softmax(x, dims=None, dtype=dt), R.rows(t["dims_all"]))
        assert np.allclose(oracle.softmax(x, dims=(1, 2), dtype=dt), R.rows(t["dims_1_2"]))


def test_logsoftmax_known_answers(oracle):
    d = G["logsoftmax_vector"]
    assert np.allclose(oracle.logsoftmax(np.array(d["x"], dtype=np.float32), dtype=np.float32), d["y"])
    d = G["logsoftmax_matrix"]
    assert np.allclose(oracle.logsoftmax(R.rows(d["x_rows"]), dtype=np.float32), R.rows(d["y_rows"]))
    d = G["logsoftmax_large_negative"]
    assert np.allclose(oracle.logsoftmax(np.array(d["x"])), d["y"])
    # test/softmax.jl:72-74: exp(logsoftmax(x)) == softmax(x) also for +-Inf entries
    for rows in ([[1, 2], [3, "Inf"]], [[1, "-Inf"], [3, "Inf"]], [[1, "Inf"], [3, "Inf"]]):
        x = R.rows(rows)
        assert np.allclose(np.exp(oracle.logsoftmax(x, dtype=np.float32)), oracle.softmax(x, dtype=np.float32))


def test_gradient_known_answers(oracle):
    x = R.rows(G["logsoftmax_matrix"]["x_rows"])
    ones = np.ones_like(x)
    y = oracle.logsoftmax(x, dtype=np.float32)
    assert np.allclose(oracle.grad_logsoftmax(ones, y, dtype=np.float32), R.rows(G["grad_logsoftmax_ones"]["dx_rows"]))
    y = oracle.softmax(x, dtype=np.float32)
    assert np.allclose(oracle.grad_softmax(ones, y, dtype=np.float32), R.rows(G["grad_softmax_ones"]["dx_rows"]))
    t = G["pytorch_logsoftmax_table"]                                  # values from PyTorch's LogSoftmax
    x = R.rows(t["x_rows"], np.float64)
    ones = np.ones_like(x)
    assert np.allclose(oracle.grad_logsoftmax(ones, oracle.logsoftmax(x)), R.rows(t["dx_rows"], np.float64), rtol=1e-5)
    assert np.allclose(oracle.grad_softmax(ones, oracle.softmax(x)), 0, atol=1e-6)


@pytest.mark.parametrize("dims,axes", [(1, (0,)), (2, (1,)), (3, (2,)), ((1, 2), (0, 1)), ((2, 3), (1, 2)), (None, (0, 1, 2))])
def test_closed_forms_on_every_dims(oracle, dims, axes):
    """test/softmax.jl:8-21,27-28: exp(x)/sum(exp(x)), log of it, and logsumexp, along every axis."""
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 5, 3))
    sm = _np_softmax(x, axes)
    assert np.allclose(oracle.softmax(x, dims), sm, atol=1e-12)
    assert np.allclose(oracle.logsoftmax(x, dims), np.log(sm), atol=1e-12)
    lse = oracle.logsumexp(x, dims)
    ref = np.log(np.exp(x).sum(axis=axes, keepdims=dims is not None))
    assert np.allclose(lse.reshape(ref.shape), ref, atol=1e-12)
    assert np.abs(oracle.softmax(x, dims, np.float32) - sm).max() < 1e-6
    # test/softmax.jl:100-106: logsumexp == mean(x - logsoftmax(x))
    assert np.allclose(lse.reshape(ref.shape), (x - oracle.logsoftmax(x, dims)).mean(axis=axes, keepdims=dims is not None))


@pytest.mark.parametrize("dims", [1, 2, None])
@pytest.mark.parametrize("log", [False, True])
def test_gradients_by_finite_differences(oracle, dims, log):
    """test/softmax.jl:108-123 checks the rrules numerically; same here with central differences."""
    rng = np.random.default_rng(4)
    x = rng.standard_normal((3, 4))
    dy = rng.standard_normal((3, 4))
    f = (lambda z: oracle.logsoftmax(z, dims)) if log else (lambda z: oracle.softmax(z, dims))
    dx = oracle.grad_softmax(dy, f(x), dims, log=log)
    num = np.zeros_like(x)
    h = 1e-6
    for idx in np.ndindex(x.shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        num[idx] = ((f(xp) - f(xm)) * dy).sum() / (2 * h)
    assert np.abs(dx - num).max() < 1e-7


@pytest.mark.parametrize("dims", [None, 1, 2])
def test_logsumexp_pullback_against_finite_differences(oracle, dims):
    """test/softmax.jl:126-128: gradtest(logsumexp, (3,4); dims = d) compares the rrule (src/softmax.jl:205-212)
    with finite differences; here the finite differences are those of the forward oracle."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal((3, 4))
    y = oracle.logsumexp(x, dims)
    dy = rng.standard_normal(y.shape if y.shape else (1,))
    got = oracle.grad_logsumexp(dy, x, dims)
    fd = np.zeros_like(x)
    h = 1e-6
    for idx in np.ndindex(x.shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        fd[idx] = ((oracle.logsumexp(xp, dims) - oracle.logsumexp(xm, dims)).reshape(dy.shape) * dy).sum() / (2 * h)
    assert np.abs(got - fd).max() < 1e-8
    # the gradient is softmax scaled by dy (the comment at src/softmax.jl:206)
    scale = dy.reshape(y.shape) if y.shape else dy.reshape(())
    assert np.abs(got - oracle.softmax(x, dims) * scale).max() < 1e-12
