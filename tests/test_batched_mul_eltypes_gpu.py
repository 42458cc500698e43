"""batched_mul on the element types of the reference's own test file: Float64, mixed Float64 x Float32,
ComplexF64 (and mixed complex), Int64 / Int32 and integer x float / complex.

Replays test/batchedmul.jl:41-137 ("batched_mul: Float64 * $TB" for TB in [Float64, Float32]) against per-slice
NumPy products evaluated in the promoted element type.  Bounds: Float64 / ComplexF64 results within 1e-12 of the
largest entry (Julia's isapprox default is sqrt(eps) = 1.5e-8 relative; the device path accumulates in Float64),
integer results bit-exact.  The result's element type is Julia's promote_type of the operands' (src/batched/
batchedmul.jl:65).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

NP = {"f64": np.float64, "f32": np.float32, "c128": np.complex128, "c64": np.complex64, "i64": np.int64, "i32": np.int32}
REAL_OF = {"c128": "f64", "c64": "f32"}


def D(nn, a, dtype):
    return nn.DeviceArray.from_numpy(np.asarray(a).astype(NP[dtype]), dtype)


def per_slice(a, b, adj_a=False, adj_b=False, out=np.float64):
    """bmm_test / bmm_adjtest of test/batchedmul.jl:6-28, in the promoted element type."""
    nb = max(a.shape[2], b.shape[2])
    res = []
    for i in range(nb):
        ai = a[:, :, i if a.shape[2] > 1 else 0].astype(out)
        bi = b[:, :, i if b.shape[2] > 1 else 0].astype(out)
        res.append((ai.conj().T if adj_a else ai) @ (bi.conj().T if adj_b else bi))
    return np.stack(res, axis=2)


def close(x, ref, tol=1e-12):
    x, ref = np.asarray(x), np.asarray(ref)
    assert x.shape == ref.shape, (x.shape, ref.shape)
    return np.abs(x - ref).max() <= tol * max(np.abs(ref).max(), 1e-300)


def randn(rng, *shape, cplx=False):
    a = rng.standard_normal(shape)
    return a + 1j * rng.standard_normal(shape) if cplx else a


@pytest.mark.parametrize("TB", ["f64", "f32"])
def test_real_products_and_transposes(nn, TB):
    """test/batchedmul.jl:43-49."""
    rng = np.random.default_rng(0)
    A, C = randn(rng, 7, 5, 3), randn(rng, 7, 6, 3)
    B = randn(rng, 5, 7, 3).astype(NP[TB])
    dA, dB, dC = D(nn, A, "f64"), D(nn, B, TB), D(nn, C, "f64")
    T = nn.batched_transpose
    r = nn.batched_mul(dA, dB)
    assert r.dtype == "f64" and r.dims == (7, 7, 3)
    tol = 1e-12
    assert close(r.to_numpy(), per_slice(A, B), tol)
    assert close(nn.batched_mul(T(dA), T(dB)).to_numpy(), per_slice(A.transpose(1, 0, 2), B.transpose(1, 0, 2)), tol)
    assert close(nn.batched_mul(T(dA), dC).to_numpy(), per_slice(A.transpose(1, 0, 2), C), tol)
    assert close(nn.batched_mul(dA, T(dA)).to_numpy(), per_slice(A, A.transpose(1, 0, 2)), tol)


@pytest.mark.parametrize("TB", ["c128", "c64"])
def test_complex_products_and_adjoints(nn, TB):
    """test/batchedmul.jl:51-59."""
    rng = np.random.default_rng(1)
    cA, cC = randn(rng, 7, 5, 3, cplx=True), randn(rng, 7, 6, 3, cplx=True)
    cB = randn(rng, 5, 7, 3, cplx=True).astype(NP[TB])
    dA, dB, dC = D(nn, cA, "c128"), D(nn, cB, TB), D(nn, cC, "c128")
    adj = nn.batched_adjoint
    c = np.complex128
    r = nn.batched_mul(dA, dB)
    assert r.dtype == "c128"
    assert close(r.to_numpy(), per_slice(cA, cB, out=c))
    assert close(nn.batched_mul(adj(dA), adj(dB)).to_numpy(), per_slice(cA, cB, True, True, out=c))
    assert close(nn.batched_mul(adj(dA), dC).to_numpy(), per_slice(cA, cC, True, out=c))
    assert close(nn.batched_mul(dA, adj(dA)).to_numpy(), per_slice(cA, cA, False, True, out=c))
    # wrappers which cancel (test/batchedmul.jl:61-65)
    assert adj(adj(dA)) is dA
    assert isinstance(nn.batched_transpose(adj(dA)), nn.BatchedTranspose)


@pytest.mark.parametrize("TB", ["f64", "f32"])
def test_integers_and_mixed(nn, TB):
    """test/batchedmul.jl:67-73: Int64 x (Float64 | Float32 converted from integers), complex x real."""
    rng = np.random.default_rng(2)
    iA = rng.integers(1, 100, (7, 5, 3))
    iBv = rng.integers(1, 100, (5, 7, 3))
    iB = iBv.astype(NP[TB])
    r = nn.batched_mul(D(nn, iA, "i64"), D(nn, iB, TB))
    assert r.dtype == TB                                   # promote_type(Int64, Float64 | Float32)
    assert np.array_equal(r.to_numpy(), per_slice(iA, iB, out=NP[TB]))      # small integers: exact in either float type
    cA = randn(rng, 7, 5, 3, cplx=True)
    r = nn.batched_mul(D(nn, cA, "c128"), D(nn, iB, TB))
    assert r.dtype == "c128"
    assert close(r.to_numpy(), per_slice(cA, iB, out=np.complex128))


@pytest.mark.parametrize("ta,tb", [("i64", "i64"), ("i64", "i32"), ("i32", "i32")])
def test_integer_products_are_bit_exact(nn, ta, tb):
    """Integer batched_mul (the generic fallback, src/batched/batchedmul.jl:306-325): exact, and wrapping on
    overflow like Julia's integer arithmetic."""
    rng = np.random.default_rng(3)
    A = rng.integers(-99, 100, (33, 70, 5)).astype(NP[ta])
    B = rng.integers(-99, 100, (70, 41, 5)).astype(NP[tb])
    out = "i64" if "i64" in (ta, tb) else "i32"
    r = nn.batched_mul(D(nn, A, ta), D(nn, B, tb))
    assert r.dtype == out
    assert np.array_equal(r.to_numpy(), per_slice(A, B, out=NP[out]))
    big = np.full((3, 4, 2), np.iinfo(NP[out]).max, NP[out])
    with np.errstate(over="ignore"):
        want = per_slice(big, big.transpose(1, 0, 2).copy(), out=NP[out])
    got = nn.batched_mul(D(nn, big, out), nn.batched_transpose(D(nn, big, out))).to_numpy()
    assert np.array_equal(got, want)
    # five-argument form with integer alpha, beta; a fractional alpha is Julia's InexactError
    C = rng.integers(-9, 10, (33, 41, 5)).astype(NP[out])
    dC = D(nn, C, out)
    nn.batched_mul_(dC, D(nn, A, ta), D(nn, B, tb), 3, -2)
    assert np.array_equal(dC.to_numpy(), 3 * per_slice(A, B, out=NP[out]) - 2 * C)
    with pytest.raises(nn.ArgumentError):
        nn.batched_mul_(dC, D(nn, A, ta), D(nn, B, tb), 0.5, 0)


@pytest.mark.parametrize("TB", ["f64", "f32"])
def test_errors(nn, TB):
    """test/batchedmul.jl:75-78."""
    z = lambda dt, *d: nn.DeviceArray.zeros(d, dt)
    with pytest.raises(nn.DimensionMismatch):
        nn.batched_mul(z("f64", 2, 2, 2), z(TB, 2, 2, 10))
    with pytest.raises(nn.DimensionMismatch):
        nn.batched_mul(z("f64", 2, 2, 2), z(TB, 10, 2, 2))
    with pytest.raises(Exception):
        nn.batched_mul_(z("f64", 2, 2, 10), z("f64", 2, 2, 2), z(TB, 2, 2, 2))
    with pytest.raises(nn.ArgumentError):                   # a Float64 product does not fit a Float32 C
        nn.batched_mul_(z("f32", 2, 2, 2), z("f64", 2, 2, 2), z("f64", 2, 2, 2))


@pytest.mark.parametrize("TB", ["f64", "f32"])
@pytest.mark.parametrize("perm", [(1, 3, 2), (2, 1, 3), (3, 2, 1)])
@pytest.mark.parametrize("adj", [False, True], ids=["identity", "batched_adjoint"])
@pytest.mark.parametrize("cplx", [False, True], ids=["real", "complex"])
def test_permuted_dims_inputs(nn, TB, perm, adj, cplx):
    """test/batchedmul.jl:80-88: lazily permuted operands equal their materialised permutations."""
    rng = np.random.default_rng(4)
    ta = "c128" if cplx else "f64"
    tb = {"f64": "c128", "f32": "c64"}[TB] if cplx else TB
    A, B = randn(rng, 4, 4, 4, cplx=cplx), randn(rng, 4, 4, 4, cplx=cplx).astype(NP[tb])
    dA, dB = D(nn, A, ta), D(nn, B, tb)
    fun = nn.batched_adjoint if adj else (lambda x: x)
    p0 = tuple(p - 1 for p in perm)
    out = np.complex128 if cplx else np.float64
    Af = A.conj().transpose(1, 0, 2) if adj else A
    assert close(nn.batched_mul(fun(dA), dB.permuted(perm)).to_numpy(), per_slice(Af, B.transpose(p0), out=out))
    Ap = A.transpose(p0)
    Apf = Ap.conj().transpose(1, 0, 2) if adj else Ap
    assert close(nn.batched_mul(fun(dA.permuted(perm)), dB).to_numpy(), per_slice(Apf, B, out=out))


@pytest.mark.parametrize("TB", ["f64", "f32"])
def test_permuted_output_alpha_beta_and_trivial_batch(nn, TB):
    """test/batchedmul.jl:90-106: PermutedDimsArray output, five-argument mul!, batch extent 1 for B."""
    rng = np.random.default_rng(5)
    A = randn(rng, 4, 3, 2)
    Bp = randn(rng, 5, 3, 2).astype(NP[TB])
    dA, dB = D(nn, A, "f64"), nn.batched_adjoint(D(nn, Bp, TB))
    C1 = per_slice(A, Bp.transpose(1, 0, 2))
    assert close(nn.batched_mul(dA, dB).to_numpy(), C1)
    base = nn.DeviceArray.zeros((5, 2, 4), "f64")
    C2 = base.permuted(3, 1, 2)                            # size (4, 5, 2)
    assert close(nn.batched_mul_(C2, dA, dB).to_numpy(), C1)
    assert close(C2.to_numpy(), C1)
    assert close(nn.batched_mul_(C2, dA, dB, 10).to_numpy(), 10 * C1, 1e-7)
    base.storage.fill_(10)
    assert close(nn.batched_mul_(C2, dA, dB, 1, 10).to_numpy(), C1 + 100)
    Dm = randn(rng, 3, 5, 1).astype(NP[TB])
    r = nn.batched_mul(dA, D(nn, Dm, TB))
    assert r.dims == (4, 5, 2)
    assert close(r.to_numpy(), per_slice(A, Dm))
    # beta = 0 overwrites NaN
    Cn = D(nn, np.full((4, 5, 2), np.nan), "f64")
    assert np.isfinite(nn.batched_mul_(Cn, dA, dB).to_numpy()).all()


def test_large_float64(nn):
    """test/batchedmul.jl:108-119 (N = 50), and sizes that straddle the 64 x 64 tiles and the k step of 16 of the
    fp64 matrix-core kernel, every transpose combination, alpha / beta."""
    rng = np.random.default_rng(6)
    N = 50
    A, B, Dm = rng.random((N, N, N)), rng.random((N, N, N)), rng.random((N, N, 1))
    assert close(nn.batched_mul(D(nn, A, "f64"), D(nn, B, "f64")).to_numpy(), per_slice(A, B))
    assert close(nn.batched_mul(D(nn, A, "f64"), D(nn, Dm, "f64")).to_numpy(), per_slice(A, Dm))
    T = nn.batched_transpose
    for (m, k, n, nb) in ((130, 67, 97, 3), (64, 16, 64, 2), (1, 5, 1, 2), (200, 300, 65, 1), (63, 1, 65, 4)):
        A, B = randn(rng, m, k, nb), randn(rng, k, n, nb)
        dA, dB = D(nn, A, "f64"), D(nn, B, "f64")
        dAt, dBt = D(nn, A.transpose(1, 0, 2), "f64"), D(nn, B.transpose(1, 0, 2), "f64")
        ref = per_slice(A, B)
        for x, y in ((dA, dB), (T(dAt), dB), (dA, T(dBt)), (T(dAt), T(dBt))):
            assert close(nn.batched_mul(x, y).to_numpy(), ref)
        C0 = randn(rng, m, n, nb)
        dC = D(nn, C0, "f64")
        nn.batched_mul_(dC, dA, dB, 2.5, -0.5)
        assert close(dC.to_numpy(), 2.5 * ref - 0.5 * C0)


def test_large_float64_128_wide_tiles(nn):
    """Products with at least 256 tiles of 128 x 128 run the wider tile of the fp64 matrix-core kernel: sizes that end
    inside a tile in both dimensions and inside a k step, a size of whole tiles (no bounds tests on the way), every
    transpose combination, alpha / beta."""
    rng = np.random.default_rng(8)
    T = nn.batched_transpose
    for (m, k, n, nb) in ((300, 70, 260, 50), (256, 64, 128, 128), (129, 33, 128, 70)):
        A, B = randn(rng, m, k, nb), randn(rng, k, n, nb)
        dA, dB = D(nn, A, "f64"), D(nn, B, "f64")
        dAt, dBt = D(nn, A.transpose(1, 0, 2), "f64"), D(nn, B.transpose(1, 0, 2), "f64")
        ref = per_slice(A, B)
        for x, y in ((dA, dB), (T(dAt), dB), (dA, T(dBt)), (T(dAt), T(dBt))):
            assert close(nn.batched_mul(x, y).to_numpy(), ref)
        C0 = randn(rng, m, n, nb)
        dC = D(nn, C0, "f64")
        nn.batched_mul_(dC, dA, dB, 2.5, -0.5)
        assert close(dC.to_numpy(), 2.5 * ref - 0.5 * C0)


def test_float64_matches_float32_path_semantics(nn):
    """The same call in Float32 and Float64 differs only by rounding: the Float64 kernel is not a widened Float32
    product (entries chosen so that Float32 accumulation is visibly worse)."""
    rng = np.random.default_rng(7)
    A, B = randn(rng, 40, 2000, 2), randn(rng, 2000, 30, 2)
    ref = per_slice(A, B)
    r64 = nn.batched_mul(D(nn, A, "f64"), D(nn, B, "f64")).to_numpy()
    r32 = nn.batched_mul(D(nn, A, "f32"), D(nn, B, "f32")).to_numpy()
    e64, e32 = np.abs(r64 - ref).max(), np.abs(r32 - ref).max()
    assert e64 < 1e-11 and e32 > 1e-7 and e64 < 1e-4 * e32


@pytest.mark.parametrize("T16", ["f16", "bf16"])
@pytest.mark.parametrize("TI", ["i32", "i64"])
def test_sixteen_bit_times_integer(nn, T16, TI):
    """promote_type(Float16 | BFloat16, Int) is the 16-bit type, and the reference's batched_mul_generic!
    (src/batched/batchedmul.jl:306-325) returns such an array.  No reference fixture pins the values (parity
    unpinned); here the product is formed in Float32 and rounded once, checked against the Float64 product of the
    same (rounded) operands to one unit of the 16-bit type."""
    from conftest import round_to
    rng = np.random.default_rng(7)
    A = round_to(rng.standard_normal((6, 5, 3)), T16)
    iB = rng.integers(-4, 5, (5, 7, 3))
    dA = nn.DeviceArray.from_numpy(A.astype(np.float32), T16)
    r = nn.batched_mul(dA, D(nn, iB, TI))
    assert r.dtype == T16 and r.dims == (6, 7, 3)
    ref = per_slice(A, iB)
    unit = 2.0 ** (-10 if T16 == "f16" else -7)
    assert np.abs(r.to_numpy() - ref).max() <= unit * np.abs(ref).max()
    r2 = nn.batched_mul(D(nn, iB.transpose(1, 0, 2), TI), nn.batched_transpose(dA))      # integer on the left
    assert r2.dtype == T16 and np.abs(r2.to_numpy() - per_slice(iB.transpose(1, 0, 2), A.transpose(1, 0, 2))).max() <= unit * np.abs(ref).max()
