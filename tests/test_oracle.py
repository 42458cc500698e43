"""Pins the CPU oracle (oracle/nnlib_oracle.c and its numpy twin) before anything is compared to it.

Every check here is either a value the reference's own tests/docstrings hold, or something the
mathematics fixes independently of the oracle's code (closed forms, brute force, invariants)."""
import numpy as np
import pytest

import reference_cases as R

IMPLS = ["nnlib_attention_f32", "attention_f64", "numpy_attention"]


@pytest.mark.parametrize("impl", IMPLS)
def test_attention_specific_results(oracle, impl):
    """test/attention.jl:25-34.  Fails under a wrong head/feature interleave, a missing 1/sqrt(D),
    a softmax over the wrong axis or a transposed value product."""
    q, ytrue, atrue = R.attention_gold()
    y, a = getattr(oracle, impl)(q, q, q, nheads=2)
    assert np.abs(y - ytrue).max() < 1e-5
    assert np.abs(a - atrue).max() < 1e-5


def test_scores_equal_attention_weights(oracle):
    """test/attention.jl:17-23: 4-D scores of (D,H,L,B) inputs equal the weights of the 3-D call."""
    q = (np.arange(1, 25, dtype=np.float64) / 24).reshape(4, 2, 3, 1, order="F")
    a = oracle.scores4_f64(q, q)
    q2 = q.reshape(8, 3, 1, order="F")
    _, a2 = oracle.attention_f64(q2, q2, q2, nheads=2)
    assert np.allclose(a, a2, atol=1e-12)
    _, a3 = oracle.nnlib_attention_f32(q2, q2, q2, nheads=2)
    assert np.allclose(a, a3, atol=1e-6)


@pytest.mark.parametrize("batch_shape", [(), (1,), (2,), (2, 1, 3)])
@pytest.mark.parametrize("nheads", [1, 3, 5])
def test_shapes_and_unit_column_sums(oracle, batch_shape, nheads):
    """test/attention.jl:1-15."""
    rng = np.random.default_rng(0)
    n, lenq, lenkv = 15, 3, 4
    q = rng.random((n, lenq) + batch_shape, dtype=np.float32)
    k = rng.random((n, lenkv) + batch_shape, dtype=np.float32)
    v = rng.random((n, lenkv) + batch_shape, dtype=np.float32)
    y, a = oracle.nnlib_attention_f32(q, k, v, nheads=nheads)
    assert y.shape == (n, lenq) + batch_shape and y.dtype == np.float32
    assert a.shape == (lenkv, lenq, nheads) + batch_shape
    assert np.allclose(a.sum(axis=0), 1, atol=1e-6)
    y64, a64 = oracle.numpy_attention(q, k, v, nheads=nheads)     # independent einsum statement
    assert np.abs(y - y64).max() < 1e-5 and np.abs(a - a64).max() < 1e-6


def test_mask_zero_pattern_and_causal(oracle):
    """test/attention.jl:36-52: alpha > 0 exactly where the mask is true (true = keep); the causal
    mask is m[i, j] = i <= j (src/attention.jl:145)."""
    rng = np.random.default_rng(1)
    q = rng.random((8, 3, 1))
    k = rng.random((8, 5, 1))
    mask = rng.random((5, 3)) < 0.5
    mask[0] = True
    for impl in IMPLS:
        _, a = getattr(oracle, impl)(q, k, k, mask=mask, nheads=2)
        assert np.all((a[:, :, 0, 0] > 0) == mask) and np.all((a[:, :, 1, 0] > 0) == mask)
    cm = oracle.make_causal_mask(3)
    assert cm.dtype == bool and np.array_equal(cm, np.triu(np.ones((3, 3), bool)))
    assert np.array_equal(cm, np.fromfunction(lambda i, j: i <= j, (3, 3)))
    x = rng.random((8, 3, 1))
    _, a = oracle.nnlib_attention_f32(x, x, x, mask=cm, nheads=2)
    assert np.all((a[:, :, 0, 0] > 0) == cm)


def test_bias_broadcast_and_order(oracle):
    """test/attention.jl:61-68 (a (kv, q) bias broadcasts over heads and batch), and bias is added
    BEFORE the mask (src/attention.jl:122-123): a +1e4 bias on a dropped entry must not resurrect it."""
    rng = np.random.default_rng(2)
    q = rng.random((4, 5, 1))
    k = rng.random((4, 3, 1))
    bias = rng.standard_normal((3, 5))
    y, a = oracle.nnlib_attention_f32(q, k, k, bias=bias, nheads=2)
    assert a.shape == (3, 5, 2, 1) and y.shape == (4, 5, 1)
    y2, a2 = oracle.numpy_attention(q, k, k, bias=bias, nheads=2)
    assert np.abs(a - a2).max() < 1e-6
    # closed form for one column: softmax(k.q/sqrt(D) + bias)
    D = 2
    s = (k[:D, :, 0] * (q[:D, 1, 0] / np.sqrt(D))[:, None]).sum(axis=0) + bias[:, 1]
    e = np.exp(s - s.max())
    assert np.allclose(a[:, 1, 0, 0], e / e.sum(), atol=1e-6)
    mask = np.ones((3, 5), bool)
    mask[2, :] = False
    big = bias.copy()
    big[2, :] = 1e4
    for impl in IMPLS:
        _, am = getattr(oracle, impl)(q, k, k, bias=big, mask=mask, nheads=2)
        assert np.all(am[2] == 0) and np.allclose(am.sum(axis=0), 1, atol=1e-6)


def test_fully_masked_column_is_nan(oracle):
    """Not pinned by any reference test ("parity unpinned"): follows src/softmax.jl:73-75 by reading,
    exp(-Inf - -Inf) = NaN.  Recorded here so that all implementations at least agree."""
    rng = np.random.default_rng(3)
    q, k = rng.random((4, 3, 1)), rng.random((4, 5, 1))
    mask = np.ones((5, 3), bool)
    mask[:, 1] = False
    for impl in IMPLS:
        with np.errstate(invalid="ignore"):
            y, a = getattr(oracle, impl)(q, k, k, mask=mask, nheads=2)
        assert np.isnan(a[:, 1]).all() and np.isnan(y[:, 1]).all()
        assert np.isfinite(a[:, [0, 2]]).all() and np.isfinite(y[:, [0, 2]]).all()


# ---- softmax --------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_softmax_reference_values(oracle, dtype):
    g = R.softmax_gold()
    d = g["doctest_vector"]
    assert np.allclose(oracle.softmax_dim1(np.array(d["x"], dtype=dtype), dtype), d["y"], atol=1e-7)
    d = g["doctest_matrix_dims1"]
    assert np.allclose(oracle.softmax_dim1(R.rows(d["x_rows"], dtype), dtype), R.rows(d["y_rows"]), atol=d["atol"])
    for key in ("int_zeros", "large_negative"):
        assert np.allclose(oracle.softmax_dim1(np.array(g[key]["x"], dtype=dtype), dtype), g[key]["y"])
    for case in g["inf_nan_table"]["cases"]:
        with np.errstate(invalid="ignore"):
            y = oracle.softmax_dim1(R.rows(case["x_rows"], dtype), dtype)
        assert np.allclose(y, R.rows(case["y_rows"]), atol=1e-6, equal_nan=True), case


def test_softmax_closed_form_and_masked_inputs(oracle):
    """test/softmax.jl:27-28 (exp.(x)./sum(exp.(x))) and test/ext_cuda/softmax.jl:34-78 (a -1e3 fill
    stays finite; a hard -Inf fill gives exact zeros and no NaN)."""
    rng = np.random.default_rng(4)
    x = rng.random(5)
    assert np.allclose(oracle.softmax_dim1(x, np.float64), np.exp(x) / np.exp(x).sum(), atol=1e-15)
    x = rng.standard_normal((128, 32)).astype(np.float32)
    x[:64] = -1e3
    y = oracle.softmax_dim1(x)
    assert np.isfinite(y).all() and np.allclose(y.sum(axis=0), 1, atol=1e-6) and np.all(y[:64] < 1e-30)
    x[:64] = -np.inf
    y = oracle.softmax_dim1(x)
    assert np.isfinite(y).all() and np.all(y[:64] == 0)
    e = np.exp(x[64:].astype(np.float64) - x[64:].max(axis=0))
    assert np.allclose(y[64:], e / e.sum(axis=0), atol=1e-6)


# ---- batched GEMM ---------------------------------------------------------------------------------

def _bmm(a, b, ta=False, tb=False):
    """test/batchedmul.jl:6-16: per-slice product with numpy's own matmul."""
    out = []
    for i in range(max(a.shape[2], b.shape[2])):
        ai = a[:, :, i if a.shape[2] > 1 else 0]
        bi = b[:, :, i if b.shape[2] > 1 else 0]
        out.append((ai.T if ta else ai) @ (bi.T if tb else bi))
    return np.stack(out, axis=2)


@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-4), (np.float64, 1e-12)])
def test_batched_gemm_against_per_slice_products(oracle, dtype, tol):
    """test/batchedmul.jl:46-49,99-106: N/T combinations, alpha/beta, batch-1 broadcast."""
    rng = np.random.default_rng(5)
    A, B, C = rng.standard_normal((7, 5, 3)), rng.standard_normal((5, 7, 3)), rng.standard_normal((7, 6, 3))
    assert np.allclose(oracle.batched_gemm(A, B, dtype=dtype), _bmm(A, B), atol=tol)
    assert np.allclose(oracle.batched_gemm(A, B, True, True, dtype=dtype), _bmm(A, B, True, True), atol=tol)
    assert np.allclose(oracle.batched_gemm(A, C, True, False, dtype=dtype), _bmm(A, C, True), atol=tol)
    assert np.allclose(oracle.batched_gemm(A, A, False, True, dtype=dtype), _bmm(A, A, False, True), atol=tol)
    C1 = _bmm(A, B)
    assert np.allclose(oracle.batched_gemm(A, B, alpha=10, dtype=dtype), 10 * C1, atol=10 * tol)
    C2 = np.full((7, 7, 3), 10.0)
    assert np.allclose(oracle.batched_gemm(A, B, alpha=1, beta=10, C=C2, dtype=dtype), C1 + 100, atol=100 * tol)
    Cpi = np.full((7, 7, 3), np.pi)     # test/ext_amdgpu/batched_mul.jl:15-19
    assert np.allclose(oracle.batched_gemm(A, B, alpha=2, beta=3, C=Cpi, dtype=dtype), 2 * C1 + 3 * np.pi, atol=10 * tol)
    D1 = rng.standard_normal((5, 4, 1))
    assert np.allclose(oracle.batched_gemm(A, D1, dtype=dtype), _bmm(A, D1), atol=tol)
    # beta = 0 must overwrite NaN garbage, as BLAS does
    Cn = np.full((7, 7, 3), np.nan)
    assert np.isfinite(oracle.batched_gemm(A, B, beta=0, C=Cn, dtype=dtype)).all()


def test_batched_gemm_threaded_matches_serial(oracle):
    """test/batchedmul.jl:109-119 (N = 50 is large enough for the threaded branch of src/gemm.jl:121-123);
    odd sizes exercise every edge of the blocked kernel."""
    rng = np.random.default_rng(6)
    A, B = rng.random((50, 50, 50), dtype=np.float32), rng.random((50, 50, 50), dtype=np.float32)
    ref = _bmm(A.astype(np.float64), B.astype(np.float64))
    for nt in (1, 3, 8):
        assert np.allclose(oracle.batched_gemm(A, B, nthreads=nt), ref, rtol=1e-5)
    A, B = rng.standard_normal((131, 263, 2)).astype(np.float32), rng.standard_normal((263, 77, 2)).astype(np.float32)
    assert np.allclose(oracle.batched_gemm(A, B, nthreads=2), _bmm(A.astype(np.float64), B.astype(np.float64)),
                       atol=2e-4)


def test_nnlib_shaped_f32_matches_f64_on_moderate_sizes(oracle):
    """The op-by-op Float32 restatement against the direct double-precision formula with every
    feature on: several heads and batches, 4-D bias, broadcast mask."""
    rng = np.random.default_rng(7)
    E, Lq, Lkv, H, B = 48, 37, 75, 3, 2
    q, k = rng.standard_normal((E, Lq, B)), rng.standard_normal((E, Lkv, B))
    v = rng.standard_normal((30, Lkv, B))
    bias = 0.5 * rng.standard_normal((Lkv, Lq, H, 1))
    mask = rng.random((Lkv, Lq)) < 0.9
    mask[0] = True
    y32, a32 = oracle.nnlib_attention_f32(q, k, v, bias, mask, H, nthreads=4)
    y64, a64 = oracle.attention_f64(q, k, v, bias, mask, H)
    yn, an = oracle.numpy_attention(q, k, v, bias, mask, H)
    assert np.abs(y64 - yn).max() < 1e-12 and np.abs(a64 - an).max() < 1e-13
    assert np.abs(y32 - y64).max() < 2e-5 and np.abs(a32 - a64).max() < 2e-6
