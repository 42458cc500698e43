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
