"""GPU parity of batched_mul / batched_mul! against per-slice products
(test/batchedmul.jl, test/ext_amdgpu/batched_mul.jl)."""
import numpy as np
import pytest

from conftest import round_to

pytestmark = pytest.mark.gpu
TOL = {"f32": 2e-5, "f16": 3e-3, "bf16": 2e-2}     # relative to the largest entry of the result


def bmm(a, b, ta=False, tb=False):
    """test/batchedmul.jl:6-16."""
    out = []
    for i in range(max(a.shape[2], b.shape[2])):
        ai = a[:, :, i if a.shape[2] > 1 else 0].astype(np.float64)
        bi = b[:, :, i if b.shape[2] > 1 else 0].astype(np.float64)
        out.append((ai.T if ta else ai) @ (bi.T if tb else bi))
    return np.stack(out, axis=2)


def close(x, ref, dtype):
    return np.abs(x - ref).max() <= TOL[dtype] * max(np.abs(ref).max(), 1e-30)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_transposes_and_products(nn, dtype):
    """test/batchedmul.jl:46-49 and test/ext_amdgpu/batched_mul.jl:1-13."""
    rng = np.random.default_rng(0)
    A, B, C = (round_to(rng.standard_normal(s), dtype) for s in ((7, 5, 3), (5, 7, 3), (7, 6, 3)))
    dA, dB, dC = (nn.DeviceArray.from_numpy(x, dtype) for x in (A, B, C))
    T = nn.batched_transpose
    assert close(nn.batched_mul(dA, dB).to_numpy(), bmm(A, B), dtype)
    assert close(nn.batched_mul(T(dA), T(dB)).to_numpy(), bmm(A, B, True, True), dtype)
    assert close(nn.batched_mul(T(dA), dC).to_numpy(), bmm(A, C, True), dtype)
    assert close(nn.batched_mul(dA, T(dA)).to_numpy(), bmm(A, A, False, True), dtype)
    assert close(nn.batched_mul(dA, nn.batched_adjoint(dA)).to_numpy(), bmm(A, A, False, True), dtype)
    assert nn.batched_transpose(T(dA)) is dA
    assert nn.batched_mul(dA, dB).dims == (7, 7, 3)


def test_alpha_beta(nn):
    """test/batchedmul.jl:99-101 and test/ext_amdgpu/batched_mul.jl:15-19."""
    rng = np.random.default_rng(1)
    A, B = rng.random((4, 3, 2)).astype(np.float32), rng.random((3, 5, 2)).astype(np.float32)
    dA, dB = nn.DeviceArray.from_numpy(A), nn.DeviceArray.from_numpy(B)
    C1 = bmm(A, B)
    C2 = nn.DeviceArray.zeros((4, 5, 2))
    assert close(nn.batched_mul_(C2, dA, dB, 10).to_numpy(), 10 * C1, "f32")
    C2 = nn.DeviceArray.from_numpy(np.full((4, 5, 2), 10, np.float32))
    assert close(nn.batched_mul_(C2, dA, dB, 1, 10).to_numpy(), C1 + 100, "f32")
    Cpi = nn.DeviceArray.from_numpy(np.full((4, 5, 2), np.pi, np.float32))
    assert close(nn.batched_mul_(Cpi, dA, dB, 2.0, 3.0).to_numpy(), 2 * C1 + 3 * np.pi, "f32")
    # beta = 0 overwrites whatever C held, NaN included
    Cn = nn.DeviceArray.from_numpy(np.full((4, 5, 2), np.nan, np.float32))
    assert np.isfinite(nn.batched_mul_(Cn, dA, dB).to_numpy()).all()


def test_broadcast_batch_and_nd(nn):
    """test/batchedmul.jl:104-106 (batch extent 1 is shared), :367-390 (N-D batches), size doctests
    of src/batched/batchedmul.jl:16-33."""
    rng = np.random.default_rng(2)
    A, D1 = rng.standard_normal((4, 3, 2)).astype(np.float32), rng.standard_normal((3, 5, 1)).astype(np.float32)
    dA, dD = nn.DeviceArray.from_numpy(A), nn.DeviceArray.from_numpy(D1)
    r = nn.batched_mul(dA, dD)
    assert r.dims == (4, 5, 2) and close(r.to_numpy(), bmm(A, D1), "f32")
    r = nn.batched_mul(nn.batched_transpose(dD), nn.batched_transpose(dA))
    assert r.dims == (5, 4, 2) and close(r.to_numpy(), bmm(D1, A, True, True), "f32")
    X, Y = rng.standard_normal((2, 5, 3, 4)).astype(np.float32), rng.standard_normal((5, 9, 3, 4)).astype(np.float32)
    Z = nn.batched_mul(nn.DeviceArray.from_numpy(X), nn.DeviceArray.from_numpy(Y)).to_numpy()
    assert Z.shape == (2, 9, 3, 4)
    assert close(Z.reshape(2, 9, 12, order="F"), bmm(X.reshape(2, 5, 12, order="F"), Y.reshape(5, 9, 12, order="F")), "f32")
    assert nn.batched_mul(nn.DeviceArray.zeros((2, 5, 17)), nn.DeviceArray.zeros((5, 9, 17))).dims == (2, 9, 17)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("m,n,k,b", [(1, 1, 1, 1), (50, 50, 50, 50), (131, 77, 263, 2), (64, 64, 64, 3), (128, 1, 64, 5),
                                     (1024, 256, 64, 4), (33, 65, 17, 7)])
def test_sizes(nn, dtype, m, n, k, b):
    """test/batchedmul.jl:109-119 (N = 50) plus sizes on and off every tile edge; the attention-shaped
    products of src/attention.jl:97,119."""
    rng = np.random.default_rng(m * n + k)
    A, B = round_to(rng.standard_normal((m, k, b)), dtype), round_to(rng.standard_normal((k, n, b)), dtype)
    r = nn.batched_mul(nn.DeviceArray.from_numpy(A, dtype), nn.DeviceArray.from_numpy(B, dtype)).to_numpy()
    assert close(r, bmm(A, B), dtype)


def test_errors(nn):
    """test/batchedmul.jl:76-78 and src/gemm.jl:106-108."""
    z = lambda *d: nn.DeviceArray.zeros(d)
    with pytest.raises(nn.DimensionMismatch, match="batch size mismatch"):
        nn.batched_mul(z(2, 2, 2), z(2, 2, 10))
    with pytest.raises(nn.DimensionMismatch, match="A1 has size"):
        nn.batched_mul(z(2, 3, 2), z(4, 2, 2))
    with pytest.raises(nn.DimensionMismatch):
        nn.batched_mul_(z(2, 2, 3), z(2, 2, 2), z(2, 2, 2))


# ---- the wider batched_mul surface (src/batched/batchedmul.jl:140-218) --------------------------------

def _slices(A, B):
    nb = max(A.shape[2], B.shape[2])
    return np.stack([A[:, :, k if A.shape[2] > 1 else 0] @ B[:, :, k if B.shape[2] > 1 else 0] for k in range(nb)], axis=2)


@pytest.mark.parametrize("perm", [(1, 3, 2), (2, 1, 3), (3, 2, 1)])
@pytest.mark.parametrize("adj", [False, True])
def test_permuted_dims_inputs(nn, perm, adj):
    """test/batchedmul.jl:80-88: lazy PermutedDimsArray operands equal their materialised permutedims;
    perm (3,2,1) has stride 1 along the batch and is copied first (_copy_if_faster)."""
    rng = np.random.default_rng(sum(perm))
    A = rng.standard_normal((4, 4, 4)).astype(np.float32)
    B = rng.standard_normal((4, 4, 4)).astype(np.float32)
    ax = tuple(p - 1 for p in perm)
    dA, dB = nn.DeviceArray.from_numpy(A), nn.DeviceArray.from_numpy(B)
    fun = nn.batched_adjoint if adj else (lambda x: x)
    Ah = A.transpose(1, 0, 2) if adj else A
    got = nn.batched_mul(fun(dA), dB.permuted(perm)).to_numpy()
    assert np.abs(got - _slices(Ah, B.transpose(ax))).max() < 1e-5
    got = nn.batched_mul(fun(dA.permuted(perm)), dB).to_numpy()
    Ap = A.transpose(ax)
    assert np.abs(got - _slices(Ap.transpose(1, 0, 2) if adj else Ap, B)).max() < 1e-5
    assert np.array_equal(dA.permuted(perm).copy().to_numpy(), Ap)          # permutedims


def test_permuted_dims_output_and_five_argument_form(nn):
    """test/batchedmul.jl:90-101: C = PermutedDimsArray(zeros(5,2,4), (3,1,2)) is written through its
    transpose; 10*C1 and C1 + 100 with the alpha / beta arguments."""
    rng = np.random.default_rng(2)
    A = rng.standard_normal((4, 3, 2)).astype(np.float32)
    Bp = rng.standard_normal((5, 3, 2)).astype(np.float32)
    dA, dB = nn.DeviceArray.from_numpy(A), nn.batched_adjoint(nn.DeviceArray.from_numpy(Bp))
    C1 = nn.batched_mul(dA, dB).to_numpy()
    assert np.abs(C1 - _slices(A, Bp.transpose(1, 0, 2))).max() < 1e-5
    parent = nn.DeviceArray.zeros((5, 2, 4))
    C2 = parent.permuted(3, 1, 2)
    assert C2.dims == (4, 5, 2)
    nn.batched_mul_(C2, dA, dB)
    assert np.abs(C2.to_numpy() - C1).max() < 1e-5
    nn.batched_mul_(C2, dA, dB, 10)
    assert np.abs(C2.to_numpy() - 10 * C1).max() < 1e-4
    parent.storage.fill_(10.0)
    nn.batched_mul_(C2, dA, dB, 1, 10)
    assert np.abs(C2.to_numpy() - (C1 + 100)).max() < 1e-4


def test_matrix_operands_and_batched_vec(nn):
    """test/batchedmul.jl:225-236: a matrix (plain or lazily transposed) on either side is shared by every
    batch; batched_vec treats the matrix as a batch of vectors."""
    rng = np.random.default_rng(3)
    A = rng.standard_normal((3, 3, 3)).astype(np.float32)
    M = rng.standard_normal((3, 3)).astype(np.float32)
    V = rng.standard_normal(3).astype(np.float32)
    dA, dM, dV = (nn.DeviceArray.from_numpy(x) for x in (A, M, V))
    cat = lambda f: np.stack([f(k) for k in range(3)], axis=2)
    assert np.abs(nn.batched_mul(dA, dM).to_numpy() - cat(lambda k: A[:, :, k] @ M)).max() < 1e-5
    assert np.abs(nn.batched_mul(dA, nn.transpose(dM)).to_numpy() - cat(lambda k: A[:, :, k] @ M.T)).max() < 1e-5
    assert np.abs(nn.batched_mul(dM, dA).to_numpy() - cat(lambda k: M @ A[:, :, k])).max() < 1e-5
    assert np.abs(nn.batched_mul(nn.adjoint(dM), dA).to_numpy() - cat(lambda k: M.T @ A[:, :, k])).max() < 1e-5
    hcat = lambda f: np.stack([f(k) for k in range(3)], axis=1)
    assert np.abs(nn.batched_vec(dA, dM).to_numpy() - hcat(lambda k: A[:, :, k] @ M[:, k])).max() < 1e-5
    assert np.abs(nn.batched_vec(dA, nn.transpose(dM)).to_numpy() - hcat(lambda k: A[:, :, k] @ M.T[:, k])).max() < 1e-5
    assert np.abs(nn.batched_vec(dA, dV).to_numpy() - hcat(lambda k: A[:, :, k] @ V)).max() < 1e-5


def test_batched_vec_nd(nn):
    """test/batchedmul.jl:337-365 and the size doctests of src/batched/batchedmul.jl:182-196."""
    rng = np.random.default_rng(4)
    A4, B3 = rng.standard_normal((4, 5, 3, 2)).astype(np.float32), rng.standard_normal((5, 3, 2)).astype(np.float32)
    C = nn.batched_vec(nn.DeviceArray.from_numpy(A4), nn.DeviceArray.from_numpy(B3))
    assert C.dims == (4, 3, 2)
    assert np.abs(C.to_numpy() - np.einsum("mkij,kij->mij", A4, B3)).max() < 1e-5
    A5, B4 = rng.standard_normal((3, 4, 2, 3, 2)).astype(np.float32), rng.standard_normal((4, 2, 3, 2)).astype(np.float32)
    C5 = nn.batched_vec(nn.DeviceArray.from_numpy(A5), nn.DeviceArray.from_numpy(B4))
    assert C5.dims == (3, 2, 3, 2)
    assert np.abs(C5.to_numpy() - np.einsum("mkabc,kabc->mabc", A5, B4)).max() < 1e-5
    Z = nn.DeviceArray.zeros
    assert nn.batched_vec(Z((16, 8, 32)), Z((8, 32))).dims == (16, 32)
    assert nn.batched_vec(Z((16, 8, 32)), Z((8,))).dims == (16, 32)
    assert nn.batched_mul(Z((16, 8, 32)), Z((8, 4))).dims == (16, 4, 32)
    assert nn.batched_mul(Z((16, 8)), Z((8, 4, 32))).dims == (16, 4, 32)
    with pytest.raises(nn.DimensionMismatch):
        nn.batched_vec(Z((3, 4, 2)), Z((4, 3)))
    with pytest.raises(nn.DimensionMismatch):
        nn.batched_vec(Z((3, 4, 2, 3)), Z((4, 2, 2)))


# ---- the tiled 16-bit kernel ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("m,n,k,nb", [(128, 128, 64, 2), (136, 200, 72, 3), (64, 264, 8, 1), (320, 72, 200, 2), (68, 132, 36, 2)])
def test_tiled_kernel_all_layouts(nn, dtype, ta, tb, m, n, k, nb):
    """Every N/T combination (lazy batched_transpose views), sizes that are multiples of 8 (of 4 in the last
    case: Float32 takes the tiled kernel, 16-bit types the small-tile one) but not of the 128 x 128 tile,
    against the per-slice product in Float64 (test/batchedmul.jl:6-28)."""
    rng = np.random.default_rng(m + n + k)
    A = round_to(rng.standard_normal((k, m, nb) if ta else (m, k, nb)), dtype)
    B = round_to(rng.standard_normal((n, k, nb) if tb else (k, n, nb)), dtype)
    dA, dB = nn.DeviceArray.from_numpy(A, dtype), nn.DeviceArray.from_numpy(B, dtype)
    T = nn.batched_transpose
    got = nn.batched_mul(T(dA) if ta else dA, T(dB) if tb else dB).to_numpy()
    assert got.shape == (m, n, nb)
    assert close(got, bmm(A, B, ta, tb), dtype)


@pytest.mark.parametrize("dtype", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_large_tile_kernel(nn, dtype, ta, tb):
    """Enough 256 x 256 tiles to fill the chip: the eight-wavefront shape of the 16-bit kernel and of the Float32
    kernel on bf16 planes, ragged in m, n and k, with alpha and beta."""
    rng = np.random.default_rng(17)
    m, n, k, nb = 264, 520, 136, 48
    A = round_to(rng.standard_normal((k, m, nb) if ta else (m, k, nb)), dtype)
    B = round_to(rng.standard_normal((n, k, nb) if tb else (k, n, nb)), dtype)
    C0 = round_to(rng.standard_normal((m, n, nb)), dtype)
    dA, dB, dC = (nn.DeviceArray.from_numpy(x, dtype) for x in (A, B, C0))
    T = nn.batched_transpose
    nn.batched_mul_(dC, T(dA) if ta else dA, T(dB) if tb else dB, 0.5, 2.0)
    assert close(dC.to_numpy(), 0.5 * bmm(A, B, ta, tb) + 2.0 * C0, dtype)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("m,n,k,nb", [(2310, 600, 136, 5), (1160, 200, 72, 3), (300, 2100, 40, 7)])
def test_tile_order_covers_every_tile(nn, dtype, m, n, k, nb):
    """The tiled kernels hand their tiles to the workgroups in a permuted order (runs per die, bands of eight tile
    rows): tile counts that are not multiples of eight in m, in total, or both, so that a tile the permutation
    skipped or visited twice shows as a wrong block of the product."""
    rng = np.random.default_rng(m + n + nb)
    A = round_to(rng.standard_normal((m, k, nb)), dtype)
    B = round_to(rng.standard_normal((k, n, nb)), dtype)
    dC = nn.DeviceArray.from_numpy(np.full((m, n, nb), np.nan), dtype)
    nn.batched_mul_(dC, nn.DeviceArray.from_numpy(A, dtype), nn.DeviceArray.from_numpy(B, dtype))
    assert close(dC.to_numpy(), bmm(A, B, False, False), dtype)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_tiled_kernel_alpha_beta_and_shared_operand(nn, dtype):
    """test/ext_amdgpu/batched_mul.jl:15-19 (C .= pi; batched_mul!(C, A, B, 2, 3)) and the batch-1 operand of
    test/batchedmul.jl:104-106 at a size the tiled kernel takes."""
    rng = np.random.default_rng(5)
    A = round_to(rng.standard_normal((192, 96, 4)), dtype)
    B = round_to(rng.standard_normal((96, 160, 1)), dtype)
    dA, dB = nn.DeviceArray.from_numpy(A, dtype), nn.DeviceArray.from_numpy(B, dtype)
    C0 = round_to(np.full((192, 160, 4), np.pi), dtype)
    dC = nn.DeviceArray.from_numpy(C0, dtype)
    nn.batched_mul_(dC, dA, dB, 2.0, 3.0)
    assert close(dC.to_numpy(), 2 * bmm(A, B) + 3 * C0, dtype)
    # beta = 0 overwrites NaN (BLAS semantics)
    dC.storage.fill_(float("nan"))
    nn.batched_mul_(dC, dA, dB)
    assert close(dC.to_numpy(), bmm(A, B), dtype)


# ---- ComplexF32 (test/batchedmul.jl:51-59, 81-88, 99-119) -------------------------------------------

def _crandn(rng, *shape):
    return (rng.standard_normal(shape) + 1j * rng.standard_normal(shape)).astype(np.complex64)


def _close(got, ref, tol=2e-5):
    assert got.shape == ref.shape
    assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max())


def test_complex_adjoints(nn, oracle):
    """test/batchedmul.jl:51-59: batched_mul of complex arrays against the per-slice product, with
    batched_adjoint on either side (the 'C' flag of src/batched/batchedmul.jl:268, 281)."""
    rng = np.random.default_rng(0)
    cA, cB, cC = _crandn(rng, 7, 5, 3), _crandn(rng, 5, 7, 3), _crandn(rng, 7, 6, 3)
    D = nn.DeviceArray.from_numpy
    dA, dB, dC = D(cA), D(cB), D(cC)
    assert dA.dtype == "c64"
    P = oracle.per_slice_product
    _close(nn.batched_mul(dA, dB).to_numpy(), P(cA, cB))
    _close(nn.batched_mul(nn.batched_adjoint(dA), nn.batched_adjoint(dB)).to_numpy(), P(cA, cB, adjA=True, adjB=True))
    _close(nn.batched_mul(nn.batched_adjoint(dA), dC).to_numpy(), P(cA, cC, adjA=True))
    _close(nn.batched_mul(dA, nn.batched_adjoint(dA)).to_numpy(), P(cA, cA, adjB=True))
    # transposes without conjugation, and the double adjoint unwrapping
    _close(nn.batched_mul(nn.batched_transpose(dA), dC).to_numpy(), P(cA, cC, transA=True))
    assert nn.batched_adjoint(nn.batched_adjoint(dA)) is dA
    _close(nn.batched_adjoint(dA).to_numpy(), np.conj(np.transpose(cA, (1, 0, 2))))
    # element types that differ promote as in the reference (test/batchedmul.jl:73): ComplexF32 x Float32 -> ComplexF32
    ones = np.ones((5, 7, 3), dtype=np.float32)
    mixed = nn.batched_mul(dA, D(ones))
    assert mixed.dtype == "c64"
    _close(mixed.to_numpy(), P(cA, ones.astype(np.complex64)))


@pytest.mark.parametrize("perm", [(1, 3, 2), (2, 1, 3), (3, 2, 1)])
@pytest.mark.parametrize("adj", [False, True])
def test_complex_permuted_dims_inputs(nn, oracle, perm, adj):
    """test/batchedmul.jl:81-88 with ty = complex: lazily permuted operands, plain or under batched_adjoint."""
    rng = np.random.default_rng(sum(perm) * 7 + adj)
    A, B = _crandn(rng, 4, 4, 4), _crandn(rng, 4, 4, 4)
    D = nn.DeviceArray.from_numpy
    fun = nn.batched_adjoint if adj else (lambda x: x)
    p0 = tuple(p - 1 for p in perm)
    ref = oracle.per_slice_product(A, np.transpose(B, p0), adjA=adj)
    _close(nn.batched_mul(fun(D(A)), D(B).permuted(*perm)).to_numpy(), ref)
    ref = oracle.per_slice_product(np.transpose(A, p0), B, adjA=adj)
    _close(nn.batched_mul(fun(D(A).permuted(*perm)), D(B)).to_numpy(), ref)


def test_complex_alpha_beta_broadcast_and_permuted_output(nn, oracle):
    """Five-argument form with complex alpha and beta (test/batchedmul.jl:99-101), a shared batch-1 operand
    (:104-106), beta = 0 overwriting NaN, an output that is a lazily permuted array (:90-96), ragged tile edges."""
    rng = np.random.default_rng(5)
    A, B, C0 = _crandn(rng, 70, 33, 5), _crandn(rng, 33, 67, 1), _crandn(rng, 70, 67, 5)
    D = nn.DeviceArray.from_numpy
    al, be = 0.5 - 2.0j, 1.5 + 0.25j
    C = D(C0)
    assert nn.batched_mul_(C, D(A), D(B), al, be) is C
    _close(C.to_numpy(), al * oracle.per_slice_product(A, B) + be * C0.astype(np.complex128), 5e-5)
    Cn = D(np.full((70, 67, 5), np.nan + 0j, dtype=np.complex64))
    nn.batched_mul_(Cn, D(A), D(B))
    _close(Cn.to_numpy(), oracle.per_slice_product(A, B), 5e-5)
    # output (70, 67, 5) as a permuted view of a (67, 5, 70) array
    base = nn.DeviceArray.zeros((67, 5, 70), "c64")
    out = base.permuted(3, 1, 2)
    assert out.dims == (70, 67, 5)
    nn.batched_mul_(out, D(A), D(B))
    _close(np.transpose(base.to_numpy(), (2, 0, 1)), oracle.per_slice_product(A, B), 5e-5)
    with pytest.raises(nn.DimensionMismatch):
        nn.batched_mul_(nn.DeviceArray.zeros((70, 67, 4), "c64"), D(A), D(_crandn(rng, 33, 67, 5)))
    # matrices on either side and the lazy adjoint of a matrix
    M = _crandn(rng, 33, 9)
    _close(nn.batched_mul(D(A), D(M)).to_numpy(), oracle.per_slice_product(A, M[:, :, None]), 5e-5)
    M2 = _crandn(rng, 9, 70)
    _close(nn.batched_mul(nn.adjoint(D(M2.conj().T.copy())), D(A)).to_numpy(), oracle.per_slice_product(M2[:, :, None], A), 5e-5)


# ---- trivial dimensions & unit strides (test/batchedmul.jl:125-160) ---------------------------------

_WRAPS = ["identity", "batched_adjoint", "batched_transpose", "perm_12", "perm_23"]


def _wrap(nn, kind, host, dev):
    """(host array, device view) of tA(rand(sA..., 3)) for the reference's five wrappers."""
    if kind == "identity":
        return host, dev
    if kind == "batched_adjoint":
        return np.conj(np.transpose(host, (1, 0, 2))), nn.batched_adjoint(dev)
    if kind == "batched_transpose":
        return np.transpose(host, (1, 0, 2)), nn.batched_transpose(dev)
    if kind == "perm_12":
        return np.transpose(host, (1, 0, 2)), dev.permuted(2, 1, 3)
    return np.transpose(host, (0, 2, 1)), dev.permuted(1, 3, 2)


@pytest.mark.parametrize("complex_", [False, True], ids=["Float32", "ComplexF32"])
def test_trivial_dimensions_and_unit_strides(nn, oracle, complex_):
    """test/batchedmul.jl:125-160: every wrapper x every (1|3, 1|3) slice size on both sides, out of place and
    in place with random alpha and beta, and into outputs that are themselves lazy transposes."""
    rng = np.random.default_rng(2024 + complex_)
    D = nn.DeviceArray.from_numpy
    rnd = (lambda *s: _crandn(rng, *s)) if complex_ else (lambda *s: rng.standard_normal(s).astype(np.float32))
    scal = (lambda: complex(rng.random(), rng.random())) if complex_ else (lambda: float(rng.random()))
    ran = 0
    for tA in _WRAPS:
        for sA in [(1, 1), (1, 3), (3, 1), (3, 3)]:
            for tB in _WRAPS:
                for sB in [(1, 1), (1, 3), (3, 1), (3, 3)]:
                    hA0, hB0 = rnd(*sA, 3), rnd(*sB, 3)
                    hA, dA = _wrap(nn, tA, hA0, D(hA0))
                    hB, dB = _wrap(nn, tB, hB0, D(hB0))
                    if not (hA.shape[1] == hB.shape[0] and hA.shape[2] == hB.shape[2] == 3):
                        continue
                    assert dA.dims == hA.shape and dB.dims == hB.shape
                    ref = oracle.per_slice_product(hA, hB)
                    _close(nn.batched_mul(dA, dB).to_numpy(), ref, 1e-5)
                    al, be = scal(), scal()
                    hD = rnd(*ref.shape)
                    want = al * ref + be * hD
                    _close(nn.batched_mul_(D(hD), dA, dB, al, be).to_numpy(), want, 1e-5)
                    # output that is a lazy transpose of a permuted copy: same values, other strides
                    C2 = nn.batched_transpose(D(np.ascontiguousarray(np.transpose(hD, (1, 0, 2)))))
                    assert C2.dims == ref.shape
                    assert nn.batched_mul_(C2, dA, dB, al, be) is C2
                    _close(C2.to_numpy(), want, 1e-5)
                    ran += 1
    assert ran > 100


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_float32_products_through_bf16_planes_keep_float32_accuracy(nn, ta, tb):
    """Float32 batched_mul runs its products as six bf16 matrix instructions on three bf16 planes per operand.  Against
    float64 the error must stay at Float32 rounding level relative to sum |a||b| (2^-24 per product and sum), with
    operand magnitudes spread over 2^+-12 so that every plane carries weight; an Inf in A gives the Inf the Float32
    instruction would."""
    rng = np.random.default_rng(5 + 2 * ta + tb)
    m, k, n, b = 160, 200, 136, 3
    spread = lambda shape: (rng.standard_normal(shape) * np.exp2(rng.integers(-12, 13, shape))).astype(np.float32)
    A, B = spread((k, m, b) if ta else (m, k, b)), spread((n, k, b) if tb else (k, n, b))
    dA, dB = nn.DeviceArray.from_numpy(A, "f32"), nn.DeviceArray.from_numpy(B, "f32")
    opA = nn.batched_transpose(dA) if ta else dA
    opB = nn.batched_transpose(dB) if tb else dB
    C = nn.batched_mul(opA, opB).to_numpy()
    A64 = (A.transpose(1, 0, 2) if ta else A).astype(np.float64)
    B64 = (B.transpose(1, 0, 2) if tb else B).astype(np.float64)
    ref = np.einsum("mkb,knb->mnb", A64, B64)
    scale = np.einsum("mkb,knb->mnb", np.abs(A64), np.abs(B64))
    assert np.abs(C - ref).max() / scale.max() < 1e-6
    assert (np.abs(C - ref) / scale).max() < 4 * 2.0 ** -24 * np.sqrt(k)
    A2 = A.copy()
    if ta:
        A2[3, 7, 1] = np.inf
    else:
        A2[7, 3, 1] = np.inf
    B2 = np.abs(B) + np.float32(1e-3)
    d2 = nn.DeviceArray.from_numpy(A2, "f32")
    C2 = nn.batched_mul(nn.batched_transpose(d2) if ta else d2, nn.batched_transpose(nn.DeviceArray.from_numpy(B2, "f32")) if tb else nn.DeviceArray.from_numpy(B2, "f32")).to_numpy()
    assert np.all(C2[7, :, 1] == np.inf) and np.isfinite(np.delete(C2[:, :, 1], 7, axis=0)).all() and np.isfinite(C2[:, :, 0]).all()
    # a finite value above the largest bf16 (its rounding to bf16 overflows) still multiplies as itself
    A3 = np.zeros_like(A)
    big = np.float32(3.4e38)
    if ta:
        A3[3, 7, 0] = big
    else:
        A3[7, 3, 0] = big
    B3 = np.full_like(B, np.float32(2.0 ** -20))
    d3 = nn.DeviceArray.from_numpy(A3, "f32")
    dB3 = nn.DeviceArray.from_numpy(B3, "f32")
    C3 = nn.batched_mul(nn.batched_transpose(d3) if ta else d3, nn.batched_transpose(dB3) if tb else dB3).to_numpy()
    assert np.allclose(C3[7, :, 0], np.float64(big) * 2.0 ** -20, rtol=1e-6) and np.all(np.delete(C3[:, :, 0], 7, axis=0) == 0)
