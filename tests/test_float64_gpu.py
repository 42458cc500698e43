"""GPU parity of the Float64 (and integer-input) calls the reference makes: the softmax family
(src/softmax.jl:56 `similar(x, float(T))`, test/softmax.jl:4-29, 63-74) and dot_product_attention on Float64 arrays
(the element type of the reference's own golden vectors, test/attention.jl:17-34).  Nothing is down-cast: inputs,
kernels and results are Float64, compared with the Float64 oracle at 1e-12 and with the values the reference's tests
and docstrings hold at the precision they are written to."""
import numpy as np
import pytest

import reference_cases as R

pytestmark = pytest.mark.gpu

TOL = 1e-12


def _dev(nn, x, dtype="f64"):
    return nn.DeviceArray.from_numpy(np.asarray(x), dtype)


def _close(y, ref, tol=TOL):
    y, ref = np.asarray(y, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert y.shape == ref.shape
    same_nan = np.array_equal(np.isnan(y), np.isnan(ref))
    fin = np.isfinite(ref)
    same_inf = np.array_equal(y[~fin & ~np.isnan(ref)], ref[~fin & ~np.isnan(ref)])
    return same_nan and same_inf and (not fin.any() or np.abs(y[fin] - ref[fin]).max() <= tol * max(1.0, np.abs(ref[fin]).max()))


def test_softmax_reference_values_in_float64(nn):
    g = R.softmax_gold()
    d = g["doctest_vector"]
    y = nn.softmax(_dev(nn, np.array(d["x"], dtype=np.float64)))
    assert y.dtype == "f64"
    assert np.abs(y.to_numpy() - np.array(d["y"])).max() < 1e-15       # written to 16 digits in src/softmax.jl:20-24
    d = g["doctest_matrix_dims1"]
    assert np.allclose(nn.softmax(_dev(nn, R.rows(d["x_rows"], np.float64))).to_numpy(), R.rows(d["y_rows"], np.float64), atol=1e-6)
    y = nn.softmax(_dev(nn, np.array(g["large_negative"]["x"], dtype=np.float64))).to_numpy()   # test/softmax.jl:23-24
    assert np.array_equal(y, [0.5, 0.5])
    for case in g["inf_nan_table"]["cases"]:          # test/softmax.jl:63-66: written to 6-8 digits
        x = R.rows(case["x_rows"], np.float64)
        y = nn.softmax(_dev(nn, x)).to_numpy()
        assert np.allclose(y, R.rows(case["y_rows"], np.float64), atol=1e-6, equal_nan=True), case
        with np.errstate(invalid="ignore"):          # and to 1e-12 against the closed form where the input is finite
            if np.isfinite(x).all():
                assert _close(y, np.exp(x) / np.exp(x).sum(axis=0))


@pytest.mark.parametrize("itype", ["i32", "i64"])
def test_integer_input_gives_float64(nn, itype):
    """softmax(Int[0, 0]) == [0.5, 0.5] (test/softmax.jl:5): the result type of an integer array is Float64."""
    x = _dev(nn, np.array([0, 0], dtype=np.int64), itype)
    y = nn.softmax(x)
    assert y.dtype == "f64" and np.array_equal(y.to_numpy(), [0.5, 0.5])
    xi = np.arange(-6, 6, dtype=np.int64).reshape(3, 4, order="F")
    for dims in (1, 2):
        y = nn.softmax(_dev(nn, xi, itype), dims=dims)
        e = np.exp(xi.astype(np.float64))
        assert y.dtype == "f64" and _close(y.to_numpy(), e / e.sum(axis=dims - 1, keepdims=True))
        ls = nn.logsoftmax(_dev(nn, xi, itype), dims=dims)
        assert ls.dtype == "f64" and _close(ls.to_numpy(), np.log(e / e.sum(axis=dims - 1, keepdims=True)))
    lse = nn.logsumexp(_dev(nn, xi, itype))
    assert lse.dtype == "f64" and _close(lse.to_numpy().reshape(()), np.log(np.exp(xi.astype(np.float64)).sum()))


@pytest.mark.parametrize("shape,dims", [((5,), 1), ((5, 5), 1), ((5, 5), 2), ((7, 6, 5), 2), ((7, 6, 5), (1, 2)), ((7, 6, 5), (2, 3)),
                                        ((7, 6, 5), None), ((7, 6, 5), (1, 3)), ((1024, 3), 1), ((1025, 3), 1), ((5000, 2), 1),
                                        ((3, 3000), 2), ((130, 70, 3), 2), ((2, 3, 4, 5), (2, 4)), ((1, 9), 1), ((9, 1), 1)])
def test_family_against_float64_oracle(nn, oracle, shape, dims):
    """Every member of the family on Float64 arrays against the Float64 oracle: column lengths on both sides of the
    register-cached kernel's limit (1024), strided reductions, runs of dims, dims = :, and sets that are not adjacent."""
    rng = np.random.default_rng(1000 * sum(shape) + len(str(dims)))
    x = np.asfortranarray(rng.standard_normal(shape) * 4)
    dy = np.asfortranarray(rng.standard_normal(shape))
    adjacent = dims is None or isinstance(dims, int) or list(dims) == list(range(dims[0], dims[-1] + 1))

    def ref_over(fn, *arrs):
        """the oracle takes runs of adjacent dims: move a non-adjacent set to the front first"""
        if adjacent:
            return fn(*arrs, dims=dims)
        ds = [d - 1 for d in dims]
        rest = [d for d in range(len(shape)) if d not in ds]
        perm = ds + rest
        moved = [np.asfortranarray(np.transpose(a, perm)) for a in arrs]
        out = fn(*moved, dims=tuple(range(1, len(ds) + 1)))
        return np.transpose(out, np.argsort(perm))

    y = nn.softmax(_dev(nn, x), dims=dims)
    assert y.dtype == "f64"
    yref = ref_over(lambda a, dims: oracle.softmax(a, dims, np.float64), x)
    assert _close(y.to_numpy(), yref)
    ly = nn.logsoftmax(_dev(nn, x), dims=dims)
    lref = ref_over(lambda a, dims: oracle.logsoftmax(a, dims, np.float64), x)
    assert _close(ly.to_numpy(), lref)
    g = nn.grad_softmax(_dev(nn, dy), y, dims=dims)
    assert _close(g.to_numpy(), ref_over(lambda a, b, dims: oracle.grad_softmax(a, b, dims, np.float64), dy, yref))
    gl = nn.grad_logsoftmax(_dev(nn, dy), ly, dims=dims)
    assert _close(gl.to_numpy(), ref_over(lambda a, b, dims: oracle.grad_logsoftmax(a, b, dims, np.float64), dy, lref))
    if adjacent:
        lse = nn.logsumexp(_dev(nn, x), dims=dims)
        lse_ref = oracle.logsumexp(x, dims, np.float64)
        assert lse.dtype == "f64" and _close(lse.to_numpy().reshape(np.shape(lse_ref)), lse_ref)
        dl = rng.standard_normal(lse_ref.shape if lse_ref.shape else (1,))
        gx = nn.grad_logsumexp(_dev(nn, dl.reshape(lse_ref.shape) if lse_ref.shape else dl.reshape(())), _dev(nn, x), dims=dims, lse=lse)
        assert _close(gx.to_numpy(), oracle.grad_logsumexp(dl, x, dims, np.float64))


def test_inf_and_nan_columns_in_float64(nn, oracle):
    """The +-Inf rules of src/softmax.jl:73-75 and NaN propagation on every kernel of the Float64 family (cached column,
    streamed column, strided)."""
    t = R.softmax_family_gold()["inf_table_other_dims"]          # test/softmax.jl:68-70
    x = R.rows(t["x_rows"], np.float64)
    for dims, key in ((2, "dims2"), (None, "dims_all"), ((1, 2), "dims_1_2")):
        assert np.allclose(nn.softmax(_dev(nn, x), dims=dims).to_numpy(), R.rows(t[key], np.float64), atol=1e-6), key
    rng = np.random.default_rng(3)
    for shape, dims in (((40, 6), 1), ((3000, 6), 1), ((6, 40), 2)):
        x = np.asfortranarray(rng.standard_normal(shape))
        cols = x if dims == 1 else x.T
        cols[3, 0] = np.inf                      # one +Inf: indicator
        cols[5, 1] = cols[9, 1] = np.inf         # two +Inf: halves
        cols[:, 2] = -np.inf                     # nothing but -Inf: NaN (exp(-Inf - -Inf))
        cols[7, 3] = np.nan                      # a NaN poisons its column
        cols[2, 4] = -np.inf                     # a -Inf entry gets weight 0
        with np.errstate(invalid="ignore"):
            for fn, ref in ((nn.softmax, oracle.softmax), (nn.logsoftmax, oracle.logsoftmax)):
                y = fn(_dev(nn, x), dims=dims).to_numpy()
                assert _close(y, ref(x, dims, np.float64)), (shape, dims, fn.__name__)
            assert _close(nn.logsumexp(_dev(nn, x), dims=dims).to_numpy().ravel(), np.ravel(oracle.logsumexp(x, dims, np.float64)))


def test_attention_golden_vectors_in_float64(nn, oracle):
    """test/attention.jl:25-34 as the reference runs it: Float64 q = k = v, nheads = 2; `ytrue` and `αtrue` are written to
    seven digits (atol 1e-5 there); against the Float64 oracle the device result agrees to 1e-12."""
    q, ytrue, atrue = R.attention_gold()
    dq = _dev(nn, q)
    y, a = nn.dot_product_attention(dq, dq, dq, nheads=2)
    assert y.dtype == "f64" and a.dtype == "f64"
    assert np.abs(y.to_numpy() - ytrue).max() < 1e-6 and np.abs(a.to_numpy() - atrue).max() < 1e-6
    yo, ao = oracle.attention_f64(q, q, q, nheads=2)
    assert _close(y.to_numpy(), yo) and _close(a.to_numpy(), ao)
    # test/attention.jl:17-23: the scores of the 4-D call are the weights of the 3-D call
    q4 = (np.arange(1, 25, dtype=np.float64) / 24).reshape(4, 2, 3, 1, order="F")
    s = nn.dot_product_attention_scores(_dev(nn, q4), _dev(nn, q4))
    _, a3 = nn.dot_product_attention(_dev(nn, q4.reshape(8, 3, 1, order="F")), _dev(nn, q4.reshape(8, 3, 1, order="F")),
                                     _dev(nn, q4.reshape(8, 3, 1, order="F")), nheads=2)
    assert s.dtype == "f64" and np.array_equal(s.to_numpy(), a3.to_numpy())


@pytest.mark.parametrize("case", ["plain", "causal", "mask", "bias", "bias_mask", "long", "dv", "dropout"])
def test_attention_float64_against_oracle(nn, oracle, case):
    rng = np.random.default_rng(len(case) + 17)
    E, Ev, Lq, Lkv, H, B = 24, 24, 9, 13, 3, 2
    if case == "long":
        Lkv = 5000        # past the row that the kernel keeps in LDS
    if case == "dv":
        Ev = 36
    if case == "causal":
        Lq = Lkv
    q = np.asfortranarray(rng.standard_normal((E, Lq, B)))
    k = np.asfortranarray(rng.standard_normal((E, Lkv, B)))
    v = np.asfortranarray(rng.standard_normal((Ev, Lkv, B)))
    bias = np.asfortranarray(rng.standard_normal((Lkv, Lq, H, 1)) * 0.5) if "bias" in case else None
    mask = None
    if "mask" in case:
        mask = np.asfortranarray(rng.random((Lkv, Lq, 1, B)) < 0.8)
        mask[0] = True
    dmask = nn.make_causal_mask(nn.DeviceArray.from_numpy(q, "f64")) if case == "causal" else (
        nn.DeviceArray.from_numpy(mask, "bool") if mask is not None else None)
    omask = oracle.make_causal_mask(Lq) if case == "causal" else mask
    fdrop = nn.Dropout(0.3, seed=11) if case == "dropout" else nn.identity
    y, a = nn.dot_product_attention(_dev(nn, q), _dev(nn, k), _dev(nn, v), None if bias is None else _dev(nn, bias),
                                    mask=dmask, nheads=H, fdrop=fdrop)
    assert nn.last_attention_kernel() == "generic" and y.dtype == "f64" and a.dtype == "f64"
    yo, ao = oracle.attention_f64(q, k, v, bias=bias, mask=omask, nheads=H)
    if case == "dropout":
        keep = oracle.dropout_keep_mask((Lkv, Lq, H, B), 0.3, 11)
        ao = ao * keep / 0.7
        D = Ev // H
        yo = np.einsum("jihb,dhjb->dhib", ao, v.reshape(D, H, Lkv, B, order="F")).reshape(Ev, Lq, B, order="F")
        assert np.abs(a.to_numpy() - ao).max() < 1e-6      # the scale 1 / (1 - p) is a Float32 in the descriptor
        assert np.abs(y.to_numpy() - yo).max() < 1e-6
        return
    assert _close(a.to_numpy(), ao) and _close(y.to_numpy(), yo)
    assert np.abs(a.to_numpy().sum(axis=0) - 1).max() < 1e-13


def test_float64_gradient_is_refused(nn):
    """The gradient entry point takes Float32 and 16-bit arrays only."""
    q = _dev(nn, np.ones((4, 3, 1)))
    with pytest.raises(Exception):
        nn.dot_product_attention_grad(q, q, q, q, nheads=2)
