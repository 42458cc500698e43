"""GPU parity of softmax over any dims, logsoftmax, logsumexp and the two gradients, through the C ABI,
against the reference's own values (test/softmax.jl) and the CPU oracle."""
import numpy as np
import pytest

import reference_cases as R
from conftest import round_to

pytestmark = pytest.mark.gpu
G = R.softmax_family_gold()
TOL = {"f32": 2e-6, "f16": 2e-3, "bf16": 2e-2}


def _seed(*key):
    """A seed that is the same in every process (str hashes are salted per process)."""
    import zlib
    return zlib.crc32(repr(key).encode())


def _dev(nn, x, dtype="f32"):
    return nn.DeviceArray.from_numpy(np.asarray(x, dtype=np.float32), dtype)


def test_reference_values(nn):
    d = G["doctest_matrix_dims2"]
    assert np.allclose(nn.softmax(_dev(nn, R.rows(d["x_rows"])), dims=2).to_numpy(), R.rows(d["y_rows"]), atol=1e-6)
    t = G["inf_table_other_dims"]
    x = _dev(nn, R.rows(t["x_rows"]))
    assert np.allclose(nn.softmax(x, dims=2).to_numpy(), R.rows(t["dims2"]), atol=1e-6)
    assert np.allclose(nn.softmax(x, dims=None).to_numpy(), R.rows(t["dims_all"]))
    assert np.allclose(nn.softmax(x, dims=(1, 2)).to_numpy(), R.rows(t["dims_1_2"]))
    d = G["logsoftmax_vector"]
    assert np.allclose(nn.logsoftmax(_dev(nn, d["x"])).to_numpy(), d["y"])
    d = G["logsoftmax_matrix"]
    x = _dev(nn, R.rows(d["x_rows"]))
    assert np.allclose(nn.logsoftmax(x).to_numpy(), R.rows(d["y_rows"]))
    ones = _dev(nn, np.ones((2, 3)))
    assert np.allclose(nn.grad_logsoftmax(ones, nn.logsoftmax(x)).to_numpy(), R.rows(G["grad_logsoftmax_ones"]["dx_rows"]))
    assert np.allclose(nn.grad_softmax(ones, nn.softmax(x)).to_numpy(), 0)
    t = G["pytorch_logsoftmax_table"]
    x = _dev(nn, R.rows(t["x_rows"]))
    ones = _dev(nn, np.ones((3, 6)))
    assert np.allclose(nn.grad_logsoftmax(ones, nn.logsoftmax(x)).to_numpy(), R.rows(t["dx_rows"]), rtol=1e-4, atol=1e-6)
    assert np.allclose(nn.grad_softmax(ones, nn.softmax(x)).to_numpy(), 0, atol=1e-6)
    for rows in ([[1, 2], [3, "Inf"]], [[1, "-Inf"], [3, "Inf"]], [[1, "Inf"], [3, "Inf"]]):   # test/softmax.jl:72-74
        x = _dev(nn, R.rows(rows))
        assert np.allclose(np.exp(nn.logsoftmax(x).to_numpy()), nn.softmax(x).to_numpy())
    x = _dev(nn, R.rows([[1, 2], [3, "NaN"]]))
    y = nn.logsoftmax(x).to_numpy()
    assert np.isnan(y[:, 1]).all() and np.isfinite(y[:, 0]).all()


SHAPES = [((2, 2, 2, 2, 2), d) for d in (1, 2, 3, 4, 5)] + [
    ((5, 7), 2), ((3, 4), None), ((33, 65, 3), 2), ((64, 100, 5), 2), ((130, 17, 2), (2, 3)), ((7, 3000, 2), 2),
    ((1, 5000, 3), 2), ((300, 70, 2), 2), ((5000,), 1), ((70000,), None), ((4, 9, 6), (1, 2)), ((128, 40), 1),
    ((9, 5), 3), ((256, 1000, 3), 2), ((96, 129, 2), 2), ((32, 70, 2, 2), (2, 3)), ((1024, 65), 2),
    ((64, 9000, 2), 2), ((32, 5000, 2), 2), ((8, 8192, 1), 2), ((520, 300, 1), 2),
    # columns that exactly fill the register cache (straight-line kernels): 4096 for the gradients, 8192 and 16384
    ((32, 4096, 2), 2), ((32, 8192, 2), 2), ((32, 16384, 2), 2), ((64, 12000, 1), 2)]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape,dims", SHAPES)
def test_forward_against_oracle(nn, oracle, dtype, shape, dims):
    """Every dims of test/softmax.jl:8-14's 2^5 array, plus shapes on both sides of each kernel
    boundary (inner below / above 64, columns that fit registers or are re-read)."""
    rng = np.random.default_rng(_seed(shape, dims, 0))
    x = round_to(rng.standard_normal(shape) * 2, dtype)
    dx = _dev(nn, x, dtype)
    tol = TOL[dtype]
    sm = nn.softmax(dx, dims=dims).to_numpy()
    assert np.abs(sm - oracle.softmax(x, dims)).max() <= tol
    ls_ref = oracle.logsoftmax(x, dims)
    ls = nn.logsoftmax(dx, dims=dims).to_numpy()
    assert np.abs(ls - ls_ref).max() <= tol * max(1.0, np.abs(ls_ref).max())
    lse_ref = oracle.logsumexp(x, dims)
    lse = nn.logsumexp(dx, dims=dims)
    assert lse.dims == lse_ref.shape
    assert np.abs(lse.to_numpy() - lse_ref).max() <= tol * max(1.0, np.abs(lse_ref).max())
    # in place (softmax!(x), logsoftmax!(x)): test/softmax.jl:8-14
    d2 = _dev(nn, x, dtype)
    nn.logsoftmax_(d2, dims=dims)
    assert np.array_equal(d2.to_numpy(), ls)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape,dims", SHAPES)
def test_gradients_against_oracle(nn, oracle, dtype, shape, dims):
    rng = np.random.default_rng(_seed(shape, dims, 1))
    x = rng.standard_normal(shape) * 2
    dy = round_to(rng.standard_normal(shape), dtype)
    tol = TOL[dtype] * 4
    for log in (False, True):
        y = round_to(oracle.softmax(x, dims, log=log), dtype)
        ref = oracle.grad_softmax(dy, y, dims, log=log)
        fn = nn.grad_logsoftmax if log else nn.grad_softmax
        got = fn(_dev(nn, dy, dtype), _dev(nn, y, dtype), dims=dims).to_numpy()
        assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max()), (log, np.abs(got - ref).max())
    # ∇softmax!(dx, dy, y) writing over dy
    y = round_to(oracle.softmax(x, dims), dtype)
    ddy = _dev(nn, dy, dtype)
    nn.grad_softmax_(ddy, ddy, _dev(nn, y, dtype), dims=dims)
    assert np.abs(ddy.to_numpy() - oracle.grad_softmax(dy, y, dims)).max() <= tol


def test_errors(nn):
    with pytest.raises(nn.ArgumentError, match="expects an array"):
        nn.logsoftmax(1.0)
    with pytest.raises(nn.ArgumentError, match="expects an array"):
        nn.logsumexp(1.0)
    with pytest.raises(nn.DimensionMismatch):
        nn.grad_softmax_(nn.DeviceArray.zeros((3, 2)), nn.DeviceArray.zeros((2, 3)), nn.DeviceArray.zeros((2, 3)))


@pytest.mark.parametrize("length", [200, 8192, 9000, 16384, 20000],
                         ids=["register-cached", "cache-filled", "register-cached-32-pieces", "cache-filled-32-pieces", "streamed"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_special_values_on_the_wide_row_kernel(nn, oracle, dtype, length):
    """Both strided kernels (columns held in registers, with and without the straight-line variant for columns
    that fill the cache exactly; longer columns with a one-pass maximum-and-sum) keep the +-Inf / NaN rules of
    src/softmax.jl:72-75, 140-144 wherever the special entry sits."""
    rng = np.random.default_rng(11)
    x = round_to(rng.standard_normal((64, length, 2)), dtype)
    x[0, :, 0] = -np.inf                      # all -Inf: NaN
    x[1, 5, 0] = np.inf                       # one +Inf
    x[2, [3, 150], 0] = np.inf                # two +Inf: 0.5 each
    x[3, 0, 0] = -np.inf                      # -Inf first, finite later
    x[4, 199, 0] = -np.inf
    x[5, 77, 0] = np.nan                      # NaN poisons its column only
    x[6, :100, 1] = -np.inf                   # a long run of -Inf before the first finite entry
    x[7, 0, 1] = np.inf
    x[7, 1:, 1] = -np.inf
    d = _dev(nn, x, dtype)
    tol = TOL[dtype]
    with np.errstate(invalid="ignore"):
        for fn, ref in ((nn.softmax, oracle.softmax(x, 2)), (nn.logsoftmax, oracle.logsoftmax(x, 2))):
            got = fn(d, dims=2).to_numpy()
            assert np.array_equal(np.isnan(got), np.isnan(ref))
            assert np.array_equal(np.isinf(got), np.isinf(ref))
            fin = np.isfinite(ref)
            assert np.abs(got[fin] - ref[fin]).max() <= tol * max(1.0, np.abs(ref[fin]).max())
        got, ref = nn.logsumexp(d, dims=2).to_numpy(), oracle.logsumexp(x, 2)
        assert np.array_equal(np.isnan(got), np.isnan(ref)) and np.array_equal(np.isinf(got), np.isinf(ref))
        fin = np.isfinite(ref)
        assert np.abs(got[fin] - ref[fin]).max() <= tol * 10


@pytest.mark.parametrize("length", [200, 8192, 9000, 20000], ids=["register-cached", "cache-filled", "register-cached-32-pieces", "streamed"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_nan_poisons_its_whole_column_wherever_it_sits(nn, oracle, dtype, length):
    """src/softmax.jl:69-70: a NaN becomes the column maximum, so the whole column is NaN.  In the streamed kernel
    every thread keeps a running (maximum, sum) of its own rows: the NaN is put in a thread's very first row, right
    after a run of -Inf entries, in the middle, and in the last row."""
    rng = np.random.default_rng(12)
    x = round_to(rng.standard_normal((64, length, 2)), dtype)
    x[0, 0, 0] = np.nan                        # first row of the first slice
    x[1, 1, 0] = np.nan                        # first row of the second slice
    run = min(300, length // 2)
    x[2, :run, 0] = -np.inf
    x[2, run, 0] = np.nan                      # after a leading run of -Inf
    x[3, length // 2 + 7, 0] = np.nan
    x[4, length - 1, 0] = np.nan
    x[5, 63, 1] = np.nan
    x[5, 64:128, 1] = -np.inf
    x[6, :, 1] = -np.inf
    x[6, 17, 1] = np.nan                       # NaN among nothing but -Inf
    d = _dev(nn, x, dtype)
    poisoned = np.zeros((64, 2), bool)
    poisoned[[0, 1, 2, 3, 4], 0] = True
    poisoned[[5, 6], 1] = True
    with np.errstate(invalid="ignore"):
        for fn, ref in ((nn.softmax, oracle.softmax(x, 2)), (nn.logsoftmax, oracle.logsoftmax(x, 2))):
            got = fn(d, dims=2).to_numpy()
            assert np.array_equal(np.isnan(ref), np.broadcast_to(poisoned[:, None, :], ref.shape))   # the oracle agrees
            assert np.array_equal(np.isnan(got), np.isnan(ref))
            fin = np.isfinite(ref)
            assert np.abs(got[fin] - ref[fin]).max() <= TOL[dtype] * max(1.0, np.abs(ref[fin]).max())
        got, ref = nn.logsumexp(d, dims=2).to_numpy(), oracle.logsumexp(x, 2)
        assert np.array_equal(np.isnan(got).reshape(64, 2), poisoned) and np.array_equal(np.isnan(ref).reshape(64, 2), poisoned)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape,dims", [((3, 4), None), ((3, 4), 1), ((3, 4), 2), ((64, 100, 5), 2), ((33, 65, 3), (2, 3)),
                                        ((5000,), 1), ((128, 40), 1)])
def test_logsumexp_pullback(nn, oracle, dtype, shape, dims):
    """Pullback of logsumexp (rrule at src/softmax.jl:205-212; the reference checks it with gradtest,
    test/softmax.jl:126-128) against the oracle, with and without the saved forward result."""
    rng = np.random.default_rng(_seed(shape, dims, 2))
    x = round_to(rng.standard_normal(shape) * 2, dtype)
    ref_y = oracle.logsumexp(x, dims)
    dy = round_to(rng.standard_normal(ref_y.shape if ref_y.shape else (1,)), dtype)
    ref = oracle.grad_logsumexp(dy, x, dims)
    dx_, dy_ = _dev(nn, x, dtype), _dev(nn, dy.reshape(ref_y.shape) if ref_y.shape else dy.reshape(()), dtype)
    got = nn.grad_logsumexp(dy_, dx_, dims=dims).to_numpy()
    assert got.shape == x.shape
    # the forward result is handed over in the array's element type: a 16-bit logsumexp of size ~8 carries a
    # rounding error of 2^-9 (f16) / 2^-6 (bf16) relative to its exponent, which is the error of every exp(x - lse)
    tol = {"f32": 1e-5, "f16": 5e-3, "bf16": 3e-2}[dtype]
    assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max())
    lse = nn.logsumexp(dx_, dims=dims)
    got2 = nn.grad_logsumexp(dy_, dx_, dims=dims, lse=lse).to_numpy()
    assert np.array_equal(got, got2)


def test_logsumexp_pullback_of_infinite_columns_is_nan(nn, oracle):
    x = np.zeros((4, 3), dtype=np.float32)
    x[:, 0] = -np.inf
    x[1, 1] = np.inf
    dy = np.ones((1, 3), dtype=np.float32)
    with np.errstate(invalid="ignore"):
        ref = oracle.grad_logsumexp(dy, x, 1)
    got = nn.grad_logsumexp(_dev(nn, dy), _dev(nn, x), dims=1).to_numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.isnan(got[:, :2]).all() and np.allclose(got[:, 2], 0.25)


@pytest.mark.parametrize("shape,dims", [((2, 3, 4), (1, 3)), ((3, 2, 4, 5), (2, 4)), ((3, 2, 4, 5), (1, 3, 4)), ((2, 2, 2, 2, 2), (1, 5))])
def test_dims_that_are_not_neighbours(nn, oracle, shape, dims):
    """Base's reductions take any dims tuple (src/softmax.jl:69-79 reduces with maximum / sum over dims); sets that
    are not a run go through permutedims on the device.  Checked against the closed forms of test/softmax.jl:27-28
    and against the adjacent-dims path on a host-permuted copy."""
    rng = np.random.default_rng(len(shape) * 10 + len(dims))
    x = rng.standard_normal(shape).astype(np.float32)
    ax = tuple(d - 1 for d in dims)
    e = np.exp(x.astype(np.float64))
    sm = e / e.sum(axis=ax, keepdims=True)
    d = _dev(nn, x)
    assert np.abs(nn.softmax(d, dims=dims).to_numpy() - sm).max() < 1e-6
    assert np.abs(nn.logsoftmax(d, dims=dims).to_numpy() - np.log(sm)).max() < 1e-5
    lse = nn.logsumexp(d, dims=dims)
    assert lse.dims == tuple(1 if i in ax else n for i, n in enumerate(shape))
    assert np.abs(lse.to_numpy() - np.log(e.sum(axis=ax, keepdims=True))).max() < 1e-5
    # gradients: against the oracle on a host-permuted copy whose reduced dims are the leading run
    perm = list(ax) + [i for i in range(len(shape)) if i not in ax]
    inv = np.argsort(perm)
    front = tuple(range(1, len(dims) + 1))
    dy = rng.standard_normal(shape).astype(np.float32)
    y = sm.astype(np.float32)
    ref = np.transpose(oracle.grad_softmax(np.transpose(dy, perm), np.transpose(y, perm), front), inv)
    assert np.abs(nn.grad_softmax(_dev(nn, dy), _dev(nn, y), dims=dims).to_numpy() - ref).max() < 1e-5
    ly = np.log(sm).astype(np.float32)
    ref = np.transpose(oracle.grad_logsoftmax(np.transpose(dy, perm), np.transpose(ly, perm), front), inv)
    assert np.abs(nn.grad_logsoftmax(_dev(nn, dy), _dev(nn, ly), dims=dims).to_numpy() - ref).max() < 1e-5
    dl = rng.standard_normal(lse.dims).astype(np.float32)
    assert np.abs(nn.grad_logsumexp(_dev(nn, dl), d, dims=dims).to_numpy() - dl * sm).max() < 1e-5
    # in-place forms
    out = nn.DeviceArray.zeros(shape)
    assert nn.softmax_(out, d, dims=dims) is out
    assert np.abs(out.to_numpy() - sm).max() < 1e-6


@pytest.mark.parametrize("outer", [64, 128], ids=["16-pieces", "32-pieces"])
def test_strided_softmax_at_the_benchmark_shape(nn, oracle, outer):
    """bench.py's `softmax_dims2` array (256 x 4096 x 128 bf16, dims = 2) and its half: the straight-line
    register-cached kernels with 32- and 64-byte row pieces.  The oracle is run on three of the outer slices;
    every column of every slice must sum to one."""
    rng = np.random.default_rng(outer)
    x = round_to(rng.standard_normal((256, 4096, outer), dtype=np.float32) * 2, "bf16")
    d = _dev(nn, x, "bf16")
    sm = nn.softmax(d, dims=2).to_numpy()
    ls = nn.logsoftmax(d, dims=2).to_numpy()
    lse = nn.logsumexp(d, dims=2).to_numpy()
    assert np.abs(sm.sum(axis=1, dtype=np.float64) - 1.0).max() <= 2.0 ** -8   # every term is rounded to bf16
    for o in (0, outer // 2 - 1, outer - 1):
        xs = x[:, :, o:o + 1]
        assert np.abs(sm[:, :, o:o + 1] - oracle.softmax(xs, 2)).max() <= TOL["bf16"]
        ref = oracle.logsoftmax(xs, 2)
        assert np.abs(ls[:, :, o:o + 1] - ref).max() <= TOL["bf16"] * np.abs(ref).max()
        ref = oracle.logsumexp(xs, 2)
        assert np.abs(lse[:, :, o:o + 1] - ref).max() <= TOL["bf16"] * np.abs(ref).max()
    y = round_to(sm, "bf16")
    dy = round_to(rng.standard_normal(x.shape, dtype=np.float32), "bf16")
    g = nn.grad_softmax(_dev(nn, dy, "bf16"), _dev(nn, y, "bf16"), dims=2).to_numpy()
    for o in (0, outer - 1):
        ref = oracle.grad_softmax(dy[:, :, o:o + 1], y[:, :, o:o + 1], 2)
        assert np.abs(g[:, :, o:o + 1] - ref).max() <= 4 * TOL["bf16"] * max(1.0, np.abs(ref).max())
