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
