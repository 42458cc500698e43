"""GPU parity of softmax(dims=1) / softmax! against the reference's own values and the CPU oracle
(test/softmax.jl, test/ext_amdgpu/softmax.jl, test/ext_cuda/softmax.jl)."""
import numpy as np
import pytest

import reference_cases as R
from conftest import round_to

pytestmark = pytest.mark.gpu


def _sm(nn, x, dtype="f32"):
    return nn.softmax(nn.DeviceArray.from_numpy(np.asarray(x, dtype=np.float32), dtype)).to_numpy()


def test_reference_values(nn):
    g = R.softmax_gold()
    d = g["doctest_vector"]
    assert np.allclose(_sm(nn, d["x"]), d["y"], atol=1e-6)
    d = g["doctest_matrix_dims1"]
    assert np.allclose(_sm(nn, R.rows(d["x_rows"])), R.rows(d["y_rows"]), atol=1e-6)
    for key in ("int_zeros", "large_negative"):
        assert np.allclose(_sm(nn, g[key]["x"]), g[key]["y"])
    for case in g["inf_nan_table"]["cases"]:          # test/softmax.jl:63-66
        y = _sm(nn, R.rows(case["x_rows"]))
        assert np.allclose(y, R.rows(case["y_rows"]), atol=1e-6, equal_nan=True), case


@pytest.mark.parametrize("dtype,atol", [("f32", 1e-6), ("f16", 1e-3), ("bf16", 1e-2)])
@pytest.mark.parametrize("shape", [(5,), (5, 5), (5, 5, 5, 5), (128, 384, 8), (1000, 7), (4096, 33), (4097, 3),
                                   (32768, 5), (40000, 2), (1, 9), (257, 64)])
def test_against_oracle(nn, oracle, dtype, atol, shape):
    """Sizes from test/ext_amdgpu/softmax.jl:1-17 and benchmark/benchmarks.jl:22-48, plus column
    lengths on both sides of every kernel boundary (one wave, registers, re-read)."""
    rng = np.random.default_rng(sum(shape))
    x = round_to(rng.standard_normal(shape) * 3, dtype)
    y = _sm(nn, x, dtype)
    ref = oracle.softmax_dim1(x.astype(np.float64), np.float64)
    assert y.shape == ref.shape
    assert np.abs(y - ref).max() <= atol
    if dtype == "f32":
        assert np.abs(y.sum(axis=0) - 1).max() < 1e-5


def test_float16_ones(nn):
    """test/ext_amdgpu/softmax.jl:9-10 uses ones for Float16."""
    y = _sm(nn, np.ones((5, 5)), "f16")
    assert np.abs(y - 0.2).max() < 1e-2


def test_in_place_and_out_of_place_agree(nn):
    """test/softmax.jl:8-14,77-103: softmax!(out, x) == softmax(x), softmax!(x) overwrites x."""
    rng = np.random.default_rng(0)
    x = rng.random((2, 2, 2, 2, 2)).astype(np.float32)
    dx = nn.DeviceArray.from_numpy(x)
    out = nn.DeviceArray.zeros(x.shape)
    nn.softmax_(out, dx)
    assert np.array_equal(out.to_numpy(), nn.softmax(dx).to_numpy())
    y = nn.softmax(dx).to_numpy()
    nn.softmax_(dx)
    assert np.array_equal(dx.to_numpy(), y)


def test_masked_inputs(nn, oracle):
    """test/ext_cuda/softmax.jl:34-78: a -1e3 fill stays finite; a hard -Inf fill gives exact zeros."""
    rng = np.random.default_rng(1)
    x = rng.standard_normal((128, 32)).astype(np.float32)
    x[:64] = -1e3
    y = _sm(nn, x)
    assert np.isfinite(y).all() and np.abs(y - oracle.softmax_dim1(x)).max() < 1e-4
    x[:64] = -np.inf
    y = _sm(nn, x)
    assert np.isfinite(y).all() and np.all(y[:64] == 0)
    assert np.abs(y - oracle.softmax_dim1(x)).max() < 1e-4
    # an all -Inf column is NaN (src/softmax.jl:73-75); its neighbours are untouched
    x[:, 3] = -np.inf
    y = _sm(nn, x)
    assert np.isnan(y[:, 3]).all() and np.isfinite(np.delete(y, 3, axis=1)).all()


def test_errors_and_empty(nn):
    with pytest.raises(nn.ArgumentError, match="expects an array"):
        nn.softmax(3.0)                                         # src/softmax.jl:215-218
    with pytest.raises(nn.DimensionMismatch):
        nn.softmax_(nn.DeviceArray.zeros((3, 2)), nn.DeviceArray.zeros((2, 3)))
    assert nn.softmax(nn.DeviceArray.zeros((0, 4))).dims == (0, 4)
