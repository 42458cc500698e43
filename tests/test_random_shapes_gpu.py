"""Randomised shape sweep over the attention kernels (forward and gradient) against the CPU oracle: lengths
that straddle every tile edge, head counts, batches, causal / random masks, all three element types.
Seeds are fixed, so a failure names a reproducible case."""
import numpy as np
import pytest

from conftest import rel_err, round_to

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    dtype = ["f32", "f16", "bf16"][seed % 3]
    D = [64, 128][(seed // 3) % 2]
    H = int(rng.integers(1, 4))
    B = int(rng.integers(1, 3))
    edges = [1, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 513]
    Lq = int(rng.choice(edges))
    mask_kind = [None, "causal", "random"][int(rng.integers(0, 3))]
    Lkv = Lq if mask_kind == "causal" else int(rng.choice(edges + [700, 1100]))
    return rng, dtype, D, H, B, Lq, Lkv, mask_kind


@pytest.mark.parametrize("seed", range(36))
def test_forward_and_gradient(nn, oracle, seed):
    rng, dtype, D, H, B, Lq, Lkv, mask_kind = _case(seed)
    E = D * H
    q = round_to(rng.standard_normal((E, Lq, B)) * 0.5, dtype)
    k = round_to(rng.standard_normal((E, Lkv, B)) * 0.5, dtype)
    v = round_to(rng.standard_normal((E, Lkv, B)), dtype)
    dy = round_to(rng.standard_normal((E, Lq, B)), dtype)
    Dv = nn.DeviceArray.from_numpy
    dq_, dk_, dv_, ddy = Dv(q, dtype), Dv(k, dtype), Dv(v, dtype), Dv(dy, dtype)
    mask = dmask = None
    if mask_kind == "causal":
        mask, dmask = oracle.make_causal_mask(Lq), nn.make_causal_mask(dq_)
    elif mask_kind == "random":
        mask = rng.random((Lkv, Lq)) < 0.7
        mask[0] = True
        dmask = Dv(mask)
    save = bool(seed % 2)
    y, a = nn.dot_product_attention(dq_, dk_, dv_, mask=dmask, nheads=H, weights_dtype="f32", save_for_backward=save)
    y_ref, a_ref = oracle.attention_f64(q, k, v, None, mask, H)
    assert rel_err(y.to_numpy(), y_ref) <= TOL[dtype], (dtype, D, H, B, Lq, Lkv, mask_kind, nn.last_attention_kernel())
    assert np.abs(a.to_numpy() - a_ref).max() <= TOL[dtype]
    got = nn.dot_product_attention_grad(ddy, dq_, dk_, dv_, y=y, mask=dmask, nheads=H)
    ref = oracle.attention_bwd_f64(q, k, v, dy, None, mask, H)
    for g, r_, name in zip(got[:3], ref[:3], ("dq", "dk", "dv")):
        err = np.abs(g.to_numpy() - r_).max() / max(np.abs(r_).max(), 0.05)
        assert err <= TOL[dtype], (name, err, dtype, D, H, B, Lq, Lkv, mask_kind, nn.last_attention_bwd_kernel())


# ---- second sweep: head dims other than 64 / 128, bias shapes, mask kinds, dropout, returned weights -------------

import os
N_SEEDS = int(os.environ.get("MI355ATTN_SWEEP_SEEDS", "45"))   # raise for a longer one-off sweep
DIMS16 = [8, 16, 24, 32, 40, 48, 64, 72, 80, 96, 112, 128, 136, 160, 192, 256]
DIMS32 = [4, 12, 20, 32, 36, 64, 68, 96, 128]


def _case2(seed):
    rng = np.random.default_rng(5000 + seed)
    dtype = ["bf16", "f16", "f32"][seed % 3]
    dims = DIMS32 if dtype == "f32" else DIMS16
    D, Dv = int(rng.choice(dims)), int(rng.choice(dims))
    H, B = int(rng.integers(1, 4)), int(rng.integers(1, 3))
    Lq = int(rng.choice([1, 31, 33, 64, 65, 127, 129, 200, 256, 300]))
    mask_kind = [None, "causal", "random", "keys", "random_hb"][int(rng.integers(0, 5))]
    aligned = bool(rng.integers(0, 2))   # rows of bias / mask start 16-byte aligned: the staged paths
    Lkv = Lq if mask_kind == "causal" else int(rng.choice([48, 64, 112, 208, 320, 400] if aligned else [47, 65, 131, 333]))
    if mask_kind == "keys" and Lkv < 100:   # the key-padding pattern of the gradient helper drops the first 70 keys of one batch element
        Lkv += 256 if aligned else 255
    bias_kind = [None, None, "full", "row", "shared"][int(rng.integers(0, 5))]
    return rng, dtype, D, Dv, H, B, Lq, Lkv, mask_kind, bias_kind


def _shapes(Lq, Lkv, H, B, mask_kind, bias_kind):
    bias_shape = {None: None, "full": (Lkv, Lq, H, B), "row": (Lkv, 1), "shared": (Lkv, Lq)}[bias_kind]
    mask_shape = {None: None, "causal": None, "random": (Lkv, Lq), "keys": (Lkv, 1, 1, B), "random_hb": (Lkv, Lq, H, B)}[mask_kind]
    return bias_shape, mask_shape


@pytest.mark.parametrize("seed", range(N_SEEDS))
def test_forward_head_dims_bias_masks(nn, oracle, seed):
    """Forward call against the oracle: head dims of q, k and of v drawn independently (zero-padded tiles), every
    bias / mask layout the kernels tell apart, with and without the weights."""
    from test_attention_gpu import _check
    rng, dtype, D, Dv, H, B, Lq, Lkv, mask_kind, bias_kind = _case2(seed)
    bias_shape, mask_shape = _shapes(Lq, Lkv, H, B, mask_kind, bias_kind)
    _check(nn, oracle, rng, dtype, D * H, Lq, Lkv, B, H, Ev=Dv * H, causal=mask_kind == "causal", bias_shape=bias_shape,
           mask_shape=mask_shape, scale=0.5, weights=bool(seed % 2))


@pytest.mark.parametrize("seed", range(N_SEEDS))
def test_gradient_head_dims_bias_masks(nn, oracle, seed):
    """Gradient (with the bias gradient where there is a bias) against the float64 oracle over the same space, one
    head dim for q, k and v, dropout in a quarter of the cases, saved statistics in half."""
    from test_attention_backward_gpu import _run
    rng, dtype, D, _, H, B, Lq, Lkv, mask_kind, bias_kind = _case2(seed)
    bias_shape, _ = _shapes(Lq, Lkv, H, B, mask_kind, bias_kind)
    dropout = (0.2, 17 + seed) if rng.integers(0, 4) == 0 else None
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, (B,), H, bias_shape=bias_shape, mask_kind=mask_kind, seed=seed, scale=0.4,
         dropout=dropout, saved=bool(rng.integers(0, 2)))


# ---- third sweep: query-dependent masks on the software-pipelined kernel (16-bit, head dims 64 / 128, no weights) ----

@pytest.mark.parametrize("seed", range(24))
def test_dense_masks_without_weights(nn, oracle, seed):
    """Lengths around every edge of the packed mask (32-key words, groups of 128 keys, 256-query padding), masks shared
    or per head / batch element, sparse enough that whole blocks, whole rows and the
    first blocks of a row are dropped; with and without the causal pattern on top.  Forward result against the
    float64 oracle; rows that keep no key are NaN in both."""
    rng = np.random.default_rng(7000 + seed)
    dtype = ["bf16", "f16"][seed % 2]
    D = [64, 128][(seed // 2) % 2]
    H, B = int(rng.integers(1, 4)), int(rng.integers(1, 3))
    edges = [1, 31, 33, 64, 127, 128, 129, 255, 256, 257, 300, 513, 700]
    Lq = int(rng.choice(edges))
    causal = bool(rng.integers(0, 2))
    Lkv = Lq if causal else int(rng.choice(edges + [1100, 1290]))
    E = D * H
    q = round_to(rng.standard_normal((E, Lq, B)) * 0.7, dtype)
    k = round_to(rng.standard_normal((E, Lkv, B)) * 0.7, dtype)
    v = round_to(rng.standard_normal((E, Lkv, B)), dtype)
    shape = [(Lkv, Lq), (Lkv, Lq, H, 1), (Lkv, Lq, 1, B), (Lkv, Lq, H, B)][int(rng.integers(0, 4))]
    keep = float(rng.choice([0.9, 0.5, 0.05]))
    mask = rng.random(shape) < keep
    full = mask.reshape(shape + (1,) * (4 - len(shape)))
    if Lq > 2:
        full[: Lkv // 2, 1] = False      # the first half of the keys dropped for one query
        full[:, 2] = False               # and everything for another
    Dv = nn.DeviceArray.from_numpy
    dq_, dk_, dv_ = Dv(q, dtype), Dv(k, dtype), Dv(v, dtype)
    dmask = Dv(mask)
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, mask=(nn.make_causal_mask(dq_) & dmask) if causal else dmask, nheads=H,
                                    return_weights=False)
    omask = np.broadcast_to(full, (Lkv, Lq, H, B))
    if causal:
        omask = omask & oracle.make_causal_mask(Lq).reshape(Lkv, Lq, 1, 1)
    y_ref, _ = oracle.attention_f64(q, k, v, None, np.ascontiguousarray(omask), H)
    y = y.to_numpy()
    nan_ref = np.isnan(y_ref)
    assert np.array_equal(np.isnan(y), nan_ref), (dtype, D, H, B, Lq, Lkv, causal, shape, keep)
    err = rel_err(np.where(nan_ref, 0, y), np.where(nan_ref, 0, y_ref))
    assert err <= TOL[dtype], (err, dtype, D, H, B, Lq, Lkv, causal, shape, keep, nn.last_attention_kernel())


# ---- fourth sweep: Float32 calls on few workgroups (a workgroup per 32 queries / 32 keys, forward and gradient) ----

N_SMALL = int(os.environ.get("MI355ATTN_SMALL_SEEDS", "40"))


@pytest.mark.parametrize("seed", range(N_SMALL))
def test_float32_calls_on_few_workgroups(nn, oracle, seed):
    """Lengths around the 32-row blocks and 128-row chunks those kernels cut the sequences into, head dims on both tile
    widths, with and without the weights, the causal mask and bias / mask arrays in the forward call, saved statistics
    or not, Bool mask arrays of every layout and fused dropout in the gradient call."""
    from test_attention_gpu import _check
    from test_attention_backward_gpu import _run
    rng = np.random.default_rng(9000 + seed)
    D = int(rng.choice([16, 32, 48, 64, 64, 64, 96, 128]))
    H, B = int(rng.integers(1, 5)), int(rng.integers(1, 4))
    edges = [1, 5, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 160, 255, 256, 257, 300, 383, 385, 500, 512]
    Lq = int(rng.choice(edges + [640, 1000]))
    causal = bool(rng.integers(0, 2))
    Lkv = Lq if causal else int(rng.choice(edges + [513, 769, 897, 1024]))
    extras = int(rng.integers(0, 3)) == 0
    bias_shape = (Lkv, Lq, H, 1) if extras else None
    mask_shape = (Lkv, Lq) if extras and not causal else None
    _check(nn, oracle, rng, "f32", D * H, Lq, Lkv, B, H, causal=causal, bias_shape=bias_shape, mask_shape=mask_shape,
           scale=0.5, expect="flash32", weights=bool(seed % 2))
    gmask = "causal" if causal else [None, "random", "keys", "random_hb"][int(rng.integers(0, 4))]
    if gmask == "keys" and Lkv < 100:   # the key-padding pattern of the gradient helper drops the first 70 keys of one batch element
        gmask = "random"
    dropout = (0.2, 31 + seed) if rng.integers(0, 4) == 0 else None
    _run(nn, oracle, "f32", D * H, D * H, Lq, Lkv, (B,), H, mask_kind=gmask, seed=seed, scale=0.4,
         saved=bool((seed // 2) % 2), dropout=dropout)
