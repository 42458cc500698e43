"""GPU parity of the attention gradient (and the batched_mul pullback) through the C ABI against the
CPU oracle, on the reference's own gradient-test shapes (test/attention.jl:70-76,
test/ext_amdgpu/attention.jl:1-22) and on shapes that reach every kernel."""
import numpy as np
import pytest

from conftest import rel_err, round_to

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def _run(nn, oracle, dtype, E, Ev, Lq, Lkv, batch, H, bias_shape=None, mask_kind=None, with_dalpha=False, flags=0,
         seed=0, scale=1.0, expect=None, pass_y=True):
    rng = np.random.default_rng(seed)
    q = round_to(rng.standard_normal((E, Lq) + batch) * scale, dtype)
    k = round_to(rng.standard_normal((E, Lkv) + batch) * scale, dtype)
    v = round_to(rng.standard_normal((Ev, Lkv) + batch), dtype)
    dy = round_to(rng.standard_normal((Ev, Lq) + batch), dtype)
    bias = None if bias_shape is None else round_to(rng.standard_normal(bias_shape) * 0.5, dtype)
    mask = dmask = None
    if mask_kind == "causal":
        mask = oracle.make_causal_mask(Lq)
        dmask = nn.make_causal_mask(nn.DeviceArray.zeros((1, Lq)))
    elif mask_kind == "random":
        mask = rng.random((Lkv, Lq)) < 0.8
        mask[0] = True
        dmask = nn.DeviceArray.from_numpy(mask)
    da = round_to(rng.standard_normal((Lkv, Lq, H) + batch), dtype) if with_dalpha else None
    D = nn.DeviceArray.from_numpy
    dq_, dk_, dv_ = D(q, dtype), D(k, dtype), D(v, dtype)
    dbias_ = None if bias is None else D(bias, dtype)
    y = None
    if pass_y:
        y, _ = nn.dot_product_attention(dq_, dk_, dv_, dbias_, mask=dmask, nheads=H, return_weights=False)
    got = nn.dot_product_attention_grad(D(dy, dtype), dq_, dk_, dv_, dbias_, y=y, mask=dmask, nheads=H,
                                        dalpha=None if da is None else D(da, dtype), _flags=flags)
    if expect is not None:
        assert nn.last_attention_bwd_kernel() == expect, nn.last_attention_bwd_kernel()
    ref = oracle.attention_bwd_f64(q, k, v, dy, bias, mask, H, da)
    errs = []
    for g, r, name in zip(got, ref, ("dq", "dk", "dv", "dbias")):
        if r is None:
            assert g is None
            continue
        g = g.to_numpy()
        assert g.shape == r.shape, name
        errs.append(rel_err(g, r))
        assert errs[-1] <= TOL[dtype], (name, errs[-1])
    return errs


def test_reference_gradient_case(nn, oracle):
    """test/attention.jl:70-76: q (4,5,1), k = v (4,3,1), bias (3,5), nheads = 2."""
    _run(nn, oracle, "f32", 4, 4, 5, 3, (1,), 2, bias_shape=(3, 5), expect="generic")


@pytest.mark.parametrize("batch", [(), (1,), (2,), (2, 1, 3)])
@pytest.mark.parametrize("nheads", [1, 3, 5])
def test_reference_gpu_comparison_shapes(nn, oracle, batch, nheads):
    """test/ext_amdgpu/attention.jl:1-22: n = 15, lenq = 3, lenkv = 4, gradients compared at 1e-5."""
    _run(nn, oracle, "f32", 15, 15, 3, 4, batch, nheads, seed=nheads)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("mask_kind", [None, "causal", "random"])
def test_generic_kernels(nn, oracle, dtype, mask_kind):
    L = 70
    _run(nn, oracle, dtype, 48, 24, L, L if mask_kind == "causal" else 300, (2,), 3, mask_kind=mask_kind,
         bias_shape=(L if mask_kind == "causal" else 300, L, 1, 2), with_dalpha=True, seed=5, scale=0.5, expect="generic")


def test_generic_on_mfma_shapes(nn, oracle):
    """The shapes the MFMA kernels take, forced through the generic kernels (the on-device cross-check)."""
    _run(nn, oracle, "bf16", 256, 256, 100, 130, (2,), 2, mask_kind="random", flags=nn._lib.MI_ATTN_FORCE_GENERIC,
         scale=0.3, expect="generic")


def test_fully_masked_query_gives_nan_gradients(nn):
    """A query with every key dropped has NaN weights (src/softmax.jl:73-75), hence NaN gradients for it
    and for every key/value of that (head, batch); other batches are untouched."""
    rng = np.random.default_rng(0)
    D = nn.DeviceArray.from_numpy
    q, k = rng.standard_normal((8, 4, 2)), rng.standard_normal((8, 5, 2))
    mask = np.ones((5, 4, 1, 2), dtype=bool)
    mask[:, 2, 0, 1] = False
    dq, dk, dv, _ = nn.dot_product_attention_grad(D(rng.standard_normal((8, 4, 2))), D(q), D(k), D(k), mask=D(mask), nheads=1)
    dq, dk = dq.to_numpy(), dk.to_numpy()
    assert np.isnan(dq[:, 2, 1]).all() and np.isfinite(dq[:, :, 0]).all() and np.isfinite(dq[:, [0, 1, 3], 1]).all()
    assert np.isnan(dk[:, :, 1]).all() and np.isfinite(dk[:, :, 0]).all()


def test_errors(nn):
    Z = nn.DeviceArray.zeros
    with pytest.raises(nn.DimensionMismatch):
        nn.dot_product_attention_grad(Z((4, 3, 1)), Z((4, 5, 1)), Z((4, 3, 1)), Z((4, 3, 1)))
    with pytest.raises(nn.ArgumentError, match="divisible"):
        nn.dot_product_attention_grad(Z((6, 5, 1)), Z((6, 5, 1)), Z((6, 3, 1)), Z((6, 3, 1)), nheads=4)


@pytest.mark.parametrize("shared", [None, "A", "B"])
def test_batched_mul_pullback(nn, oracle, shared):
    """rrule of batched_mul (src/batched/batchedmul.jl:96-110), incl. the sum over slices for an operand
    with batch extent 1."""
    rng = np.random.default_rng(1)
    A = rng.standard_normal((7, 5, 1 if shared == "A" else 4)).astype(np.float32)
    B = rng.standard_normal((5, 6, 1 if shared == "B" else 4)).astype(np.float32)
    dC = rng.standard_normal((7, 6, 4)).astype(np.float32)
    D = nn.DeviceArray.from_numpy
    dA, dB = nn.batched_mul_pullback(D(A), D(B), D(dC))
    rA = np.einsum("mnb,knb->mkb", dC, np.broadcast_to(B, (5, 6, 4)))
    rB = np.einsum("mkb,mnb->knb", np.broadcast_to(A, (7, 5, 4)), dC)
    if shared == "A":
        rA = rA.sum(axis=2, keepdims=True)
    if shared == "B":
        rB = rB.sum(axis=2, keepdims=True)
    assert dA.dims == rA.shape and dB.dims == rB.shape
    assert np.abs(dA.to_numpy() - rA).max() < 1e-4 and np.abs(dB.to_numpy() - rB).max() < 1e-4
