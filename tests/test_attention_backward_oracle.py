"""Pins the attention-gradient oracle (oracle/attention_backward_oracle.c): central finite differences
of the forward oracle, as the reference's own gradtest does (test/attention.jl:70-76), plus an
independent einsum statement."""
import numpy as np
import pytest


def _finite_difference(f, x, h=1e-6):
    g = np.zeros_like(x)
    for idx in np.ndindex(x.shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        g[idx] = (f(xp) - f(xm)) / (2 * h)
    return g


CASES = [
    # (E, Ev, Lq, Lkv, batch, H, bias shape, mask)
    (4, 4, 5, 3, (1,), 2, (3, 5), None),              # test/attention.jl:70-76
    (6, 3, 4, 4, (2,), 3, None, "causal"),
    (4, 8, 3, 5, (2,), 2, (5, 3, 2, 2), "random"),
    (4, 4, 3, 4, (1, 2), 1, (4, 1, 1, 2), None),
]


@pytest.mark.parametrize("E,Ev,Lq,Lkv,batch,H,bias_shape,mask_kind", CASES)
@pytest.mark.parametrize("with_dweights", [False, True])
def test_gradient_against_finite_differences(oracle, E, Ev, Lq, Lkv, batch, H, bias_shape, mask_kind, with_dweights):
    rng = np.random.default_rng(E * 100 + Lq * 10 + Lkv)
    q = rng.random((E, Lq) + batch)
    k = rng.random((E, Lkv) + batch)
    v = rng.random((Ev, Lkv) + batch)
    bias = None if bias_shape is None else rng.standard_normal(bias_shape)
    mask = None
    if mask_kind == "causal":
        mask = oracle.make_causal_mask(Lq)
    elif mask_kind == "random":
        mask = rng.random((Lkv, Lq)) < 0.6
        mask[0] = True
    dout = rng.standard_normal((Ev, Lq) + batch)
    dw = rng.standard_normal((Lkv, Lq, H) + batch) if with_dweights else None

    def loss(q_, k_, v_, b_):
        y, a = oracle.attention_f64(q_, k_, v_, b_, mask, H)
        return (y * dout).sum() + (0.0 if dw is None else (a * dw).sum())

    dq, dk, dv, db = oracle.attention_bwd_f64(q, k, v, dout, bias, mask, H, dw)
    assert np.abs(dq - _finite_difference(lambda z: loss(z, k, v, bias), q)).max() < 1e-7
    assert np.abs(dk - _finite_difference(lambda z: loss(q, z, v, bias), k)).max() < 1e-7
    assert np.abs(dv - _finite_difference(lambda z: loss(q, k, z, bias), v)).max() < 1e-7
    if bias is not None:
        assert db.shape == bias.shape
        assert np.abs(db - _finite_difference(lambda z: loss(q, k, v, z), bias)).max() < 1e-7
    # independent statement
    for got, ref in zip((dq, dk, dv, db), oracle.numpy_attention_bwd(q, k, v, dout, bias, mask, H, dw)):
        if got is not None:
            assert np.abs(got - ref).max() < 1e-12


def test_masked_positions_get_no_gradient(oracle):
    """Dropped logits are constants (-Inf): the bias gradient is exactly zero there."""
    rng = np.random.default_rng(0)
    q, k = rng.random((4, 4, 1)), rng.random((4, 4, 1))
    bias = rng.standard_normal((4, 4))
    mask = oracle.make_causal_mask(4)
    _, _, _, db = oracle.attention_bwd_f64(q, k, k, rng.standard_normal((4, 4, 1)), bias, mask, 2)
    assert np.all(db[~mask] == 0)
    assert np.all(db[:, 1:][mask[:, 1:]] != 0)      # (query 0 keeps one key: weight 1, gradient 0)


@pytest.mark.parametrize("E,Ev,Lq,Lkv,batch,H,bias_shape,mask_kind", CASES[:3])
@pytest.mark.parametrize("with_dweights", [False, True])
def test_gradient_through_dropout_against_finite_differences(oracle, E, Ev, Lq, Lkv, batch, H, bias_shape, mask_kind,
                                                             with_dweights):
    """fdrop = dropout multiplies the weights by a fixed array (0 or 1/(1-p), src/dropout.jl:38-53) before the
    value product and before they are returned (src/attention.jl:126): with the keep decisions held fixed the
    forward is a smooth function, and its finite differences pin the gradient through dropout."""
    rng = np.random.default_rng(E * 100 + Lq * 10 + Lkv + 7)
    q = rng.random((E, Lq) + batch)
    k = rng.random((E, Lkv) + batch)
    v = rng.random((Ev, Lkv) + batch)
    bias = None if bias_shape is None else rng.standard_normal(bias_shape)
    mask = None
    if mask_kind == "causal":
        mask = oracle.make_causal_mask(Lq)
    elif mask_kind == "random":
        mask = rng.random((Lkv, Lq)) < 0.6
        mask[0] = True
    p = 0.3
    g = oracle.dropout_keep_mask((Lkv, Lq, H) + batch, p, seed=99) / (1.0 - p)
    assert 0 < (g == 0).mean() < 1
    dout = rng.standard_normal((Ev, Lq) + batch)
    dw = rng.standard_normal((Lkv, Lq, H) + batch) if with_dweights else None
    B = int(np.prod(batch))
    D, Dv = E // H, Ev // H

    def loss(q_, k_, v_, b_):
        _, a = oracle.attention_f64(q_, k_, v_, b_, mask, H)
        ad = a * g                                              # what fdrop returns
        v4 = v_.reshape(Dv, H, Lkv, B, order="F")
        y = np.einsum("dhjb,jihb->dhib", v4, ad.reshape(Lkv, Lq, H, B, order="F")).reshape((Ev, Lq) + batch, order="F")
        return (y * dout).sum() + (0.0 if dw is None else (ad * dw).sum())

    dq, dk, dv, db = oracle.attention_bwd_f64(q, k, v, dout, bias, mask, H, dw, keep_scale=g)
    assert np.abs(dq - _finite_difference(lambda z: loss(z, k, v, bias), q)).max() < 1e-7
    assert np.abs(dk - _finite_difference(lambda z: loss(q, z, v, bias), k)).max() < 1e-7
    assert np.abs(dv - _finite_difference(lambda z: loss(q, k, z, bias), v)).max() < 1e-7
    if bias is not None:
        assert np.abs(db - _finite_difference(lambda z: loss(q, k, v, z), bias)).max() < 1e-7
    for got, ref in zip((dq, dk, dv, db), oracle.numpy_attention_bwd(q, k, v, dout, bias, mask, H, dw, keep_scale=g)):
        if got is not None:
            assert np.abs(got - ref).max() < 1e-12
