"""Attention weights returned in the element type of the inputs, for Float16 / BFloat16 calls.

The reference returns alpha in the element type of q (src/attention.jl:83 returns the array
`dot_product_attention_scores` built from q and k, src/attention.jl:112-127), so a 16-bit call hands
back 16-bit weights.  These cases call the device path with the default weights type and check the
values, for every kernel that stores them: the MFMA kernel's three store shapes (rows that start
16-byte aligned go through a transposing LDS stage, rows of a multiple of 4 keys are stored as 8-byte
runs, anything else element by element), the zeros it writes above the diagonal of a causal call, the
single-query kernels and the generic kernel.

Bounds.  alpha against the Float32 CPU result on the same rounded inputs: 1e-2 (the tolerance for
16-bit element types).  Masked entries: exactly 0.  Column sums: every stored weight is a Float32
weight w_j rounded to nearest, w_j (1 + d_j) with |d_j| <= u (u = 2^-8 for BFloat16, 2^-11 for
Float16), or, below the smallest normal Float16 2^-14, off by at most half a subnormal step 2^-25.
Hence |sum_j stored_j - 1| <= u * sum_j w_j + Lkv * 2^-25 [Float16 only] + 1e-5, the last term being
the bound the Float32 weights themselves meet.
"""
import numpy as np
import pytest

from conftest import rel_err, round_to

pytestmark = pytest.mark.gpu
TOL = 1e-2
UNIT_ROUNDOFF = {"bf16": 2.0 ** -8, "f16": 2.0 ** -11}
STORED = {"bf16": "bf16", "f16": "f16"}


def colsum_bound(dtype, Lkv):
    return UNIT_ROUNDOFF[dtype] + (Lkv * 2.0 ** -25 if dtype == "f16" else 0.0) + 1e-5


def _inputs(rng, dtype, E, Lq, Lkv, B, Ev=None, scale=1.0):
    q = round_to(rng.standard_normal((E, Lq, B)) * scale, dtype)
    k = round_to(rng.standard_normal((E, Lkv, B)) * scale, dtype)
    v = round_to(rng.standard_normal((Ev or E, Lkv, B)), dtype)
    return q, k, v


def _check_alpha(a_dev, ar, dtype, keep=None):
    """a_dev: DeviceArray of weights in the input element type; ar: Float32 oracle weights."""
    assert a_dev.dtype == STORED[dtype], a_dev.dtype                   # alpha has the element type of q
    a = a_dev.to_numpy().astype(np.float32)
    assert a.shape == ar.shape
    assert np.isfinite(a).all()
    werr = float(np.abs(a - ar).max())
    assert werr <= TOL, werr
    # every stored weight is the nearest 16-bit value of a Float32 weight within 1e-5 of the oracle's
    ulp_ok = np.abs(a - ar) <= UNIT_ROUNDOFF[dtype] * np.abs(ar) + 2.0 ** -24 + 2e-5
    assert ulp_ok.all(), float(np.abs(a - ar).max())
    Lkv = a.shape[0]
    cs = float(np.abs(a.astype(np.float64).sum(axis=0) - 1).max())
    assert cs <= colsum_bound(dtype, Lkv), (cs, colsum_bound(dtype, Lkv))
    if keep is not None:
        keep = np.broadcast_to(np.asarray(keep).reshape(keep.shape + (1,) * (a.ndim - keep.ndim)), a.shape)
        assert int(np.count_nonzero(a[~keep])) == 0
    return a


def _call(nn, q, k, v, dtype, H, bias=None, mask=None, causal=False, flags=0):
    dq, dk, dv = (nn.DeviceArray.from_numpy(x, dtype) for x in (q, k, v))
    db = nn.DeviceArray.from_numpy(bias, dtype) if bias is not None else None
    dm = nn.make_causal_mask(dq) if causal else (nn.DeviceArray.from_numpy(mask) if mask is not None else None)
    return nn.dot_product_attention(dq, dk, dv, db, mask=dm, nheads=H, _flags=flags)     # default weights type


FLASH16_NATIVE = [
    # dtype, E, Lq, Lkv, B, H, kwargs.      Weight rows are Lkv * 2 bytes long.
    ("bf16", 256, 128, 128, 2, 2, {}),                                  # aligned rows: LDS-transposed store
    ("f16", 128, 96, 160, 2, 2, {}),
    ("bf16", 256, 200, 336, 1, 2, {}),                                  # aligned, ragged tiles in both lengths
    ("f16", 128, 70, 200, 2, 2, {}),                                    # Lkv % 8 == 0, last key tile partial
    ("bf16", 128, 100, 332, 1, 2, {}),                                  # Lkv % 4 == 0 only: 8-byte runs
    ("f16", 128, 65, 132, 2, 1, {}),
    ("bf16", 256, 200, 333, 1, 2, {}),                                  # odd Lkv: element stores
    ("f16", 64, 33, 65, 3, 1, {}),
    ("bf16", 128, 50, 130, 2, 2, {}),                                   # Lkv % 2 == 0 only
    ("bf16", 256, 256, 256, 2, 2, dict(causal=True)),                   # zeros above the diagonal, aligned
    ("f16", 128, 192, 192, 1, 2, dict(causal=True)),
    ("bf16", 256, 130, 130, 1, 2, dict(causal=True)),                   # causal, unaligned
    ("f16", 128, 333, 333, 1, 2, dict(causal=True)),                    # causal, odd
    ("bf16", 128, 520, 520, 1, 2, dict(causal=True)),                   # several key tiles skipped per query tile
    ("f16", 128, 64, 320, 2, 2, dict(bias_shape=(320, 64, 2, 2), mask_shape=(320, 64))),      # staged bias / mask tiles
    ("f16", 128, 70, 131, 2, 2, dict(bias_shape=(131, 70), mask_shape=(131, 70, 1, 2))),      # direct bias / mask, odd
    ("bf16", 256, 150, 400, 2, 2, dict(mask_shape=(400, 150, 1, 2))),   # dense mask staged alone
    ("bf16", 256, 150, 400, 2, 2, dict(mask_shape=(400, 1, 1, 2))),     # key-padding mask
    ("f16", 128, 70, 131, 2, 2, dict(mask_shape=(131,))),
    ("bf16", 128, 192, 192, 2, 2, dict(causal=True, bias_shape=(192, 192, 2, 1))),
    ("bf16", 64, 200, 264, 2, 2, {}),                                   # head dim 32 in a 64-wide tile
    ("f16", 192, 130, 130, 1, 2, dict(causal=True)),                    # head dim 96
    ("bf16", 512, 100, 208, 1, 2, {}),                                  # head dim 256
    ("bf16", 96, 90, 200, 2, 2, dict(Ev=224)),                          # head dims 48 (q, k) and 112 (v)
    ("bf16", 256, 128, 1024, 1, 2, {}),                                 # long rows
]


@pytest.mark.parametrize("case", FLASH16_NATIVE, ids=lambda c: f"{c[0]}-E{c[1]}-Lq{c[2]}-Lkv{c[3]}-B{c[4]}-H{c[5]}-" + "-".join(c[6]))
def test_flash16_native_weights(nn, oracle, case):
    dtype, E, Lq, Lkv, B, H, kw = case
    kw = dict(kw)
    rng = np.random.default_rng(hash((E, Lq, Lkv, B, H, 16)) % 2**32)
    q, k, v = _inputs(rng, dtype, E, Lq, Lkv, B, kw.pop("Ev", None))
    causal = kw.pop("causal", False)
    bias = round_to(0.5 * rng.standard_normal(kw["bias_shape"]), dtype) if "bias_shape" in kw else None
    mask = None
    if "mask_shape" in kw:
        mask = rng.random(kw["mask_shape"]) < 0.9
        mask[0, ...] = True
    y, a = _call(nn, q, k, v, dtype, H, bias, mask, causal)
    assert nn.last_attention_kernel() == "flash16"
    omask = oracle.make_causal_mask(Lq) if causal else mask
    yr, ar = oracle.nnlib_attention_f32(q, k, v, bias, omask, H, nthreads=8)
    assert rel_err(y.to_numpy(), yr) <= TOL
    _check_alpha(a, ar, dtype, omask)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_native_weights_equal_rounded_f32_weights(nn, dtype):
    """The 16-bit weights are the Float32 weights of the same call rounded to nearest even, bit for bit:
    both come from the same accumulators, only the store differs."""
    rng = np.random.default_rng(40)
    for Lq, Lkv, causal in ((200, 336, False), (130, 130, True), (97, 333, False)):
        q, k, v = _inputs(rng, dtype, 256, Lq, Lkv, 2)
        dq, dk, dv = (nn.DeviceArray.from_numpy(x, dtype) for x in (q, k, v))
        dm = nn.make_causal_mask(dq) if causal else None
        _, a16 = nn.dot_product_attention(dq, dk, dv, mask=dm, nheads=2)
        _, a32 = nn.dot_product_attention(dq, dk, dv, mask=dm, nheads=2, weights_dtype="f32")
        assert a16.dtype == dtype and a32.dtype == "f32"
        assert np.array_equal(a16.to_numpy().astype(np.float32), round_to(a32.to_numpy(), dtype))


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_native_weights_context_lengths(nn, oracle, dtype):
    """Key-padding masks that keep a prefix of the keys: the pairs with a length run the variant without mask code
    (exact zeros past the length), the others the key-mask variant; both store 16-bit weights."""
    rng = np.random.default_rng(41)
    E, H, Lq, Lkv, B = 256, 2, 140, 336, 4
    q, k, v = _inputs(rng, dtype, E, Lq, Lkv, B)
    mask = np.ones((Lkv, 1, 1, B), dtype=bool)
    mask[250:, 0, 0, 0] = False
    mask[1:, 0, 0, 1] = False
    mask[:, 0, 0, 2] = rng.random(Lkv) < 0.5
    mask[0, 0, 0, 2] = True
    y, a = _call(nn, q, k, v, dtype, H, mask=mask)
    assert nn.last_attention_kernel() == "flash16"
    yr, ar = oracle.nnlib_attention_f32(q, k, v, None, mask, H, nthreads=4)
    assert rel_err(y.to_numpy(), yr) <= TOL
    _check_alpha(a, ar, dtype, mask)


@pytest.mark.parametrize("dtype,E,H,Lkv,B", [("bf16", 512, 4, 1500, 2), ("bf16", 256, 2, 4096, 3), ("f16", 512, 8, 777, 1),
                                             ("f16", 1024, 8, 2048, 2), ("bf16", 128, 1, 513, 1)])
def test_decode_native_weights(nn, oracle, dtype, E, H, Lkv, B):
    """One query per (head, batch): the split kernel keeps raw scores, a third kernel writes the 16-bit weights."""
    rng = np.random.default_rng(E + Lkv + 1)
    q, k, v = _inputs(rng, dtype, E, 1, Lkv, B)
    y, a = _call(nn, q, k, v, dtype, H)
    assert nn.last_attention_kernel() == "decode"
    yr, ar = oracle.nnlib_attention_f32(q, k, v, None, None, H, nthreads=4)
    assert rel_err(y.to_numpy(), yr) <= TOL
    _check_alpha(a, ar, dtype)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_decode_native_weights_with_mask(nn, oracle, dtype):
    rng = np.random.default_rng(43)
    E, H, Lkv, B = 256, 4, 1500, 3
    q, k, v = _inputs(rng, dtype, E, 1, Lkv, B)
    mask = rng.random((Lkv, 1, H, B)) < 0.6
    mask[0] = True
    mask[900:, 0, :, 0] = False
    y, a = _call(nn, q, k, v, dtype, H, mask=mask)
    assert nn.last_attention_kernel() == "decode"
    yr, ar = oracle.nnlib_attention_f32(q, k, v, None, mask, H, nthreads=4)
    assert rel_err(y.to_numpy(), yr) <= TOL
    _check_alpha(a, ar, dtype, mask)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("shape", ["mfma-shape", "odd-head-dim"])
def test_generic_native_weights(nn, oracle, dtype, shape):
    """The generic kernel, forced on a shape the MFMA kernel takes and picked for head dims it does not."""
    rng = np.random.default_rng(44)
    if shape == "mfma-shape":
        E, Ev, Lq, Lkv, B, H, flags = 128, 128, 70, 131, 2, 2, nn._lib.MI_ATTN_FORCE_GENERIC
    else:
        E, Ev, Lq, Lkv, B, H, flags = 44, 84, 37, 75, 2, 2, 0
    q, k, v = _inputs(rng, dtype, E, Lq, Lkv, B, Ev)
    bias = round_to(0.5 * rng.standard_normal((Lkv, Lq, H, 1)), dtype)
    mask = rng.random((Lkv, Lq)) < 0.9
    mask[0] = True
    y, a = _call(nn, q, k, v, dtype, H, bias, mask, flags=flags)
    assert nn.last_attention_kernel() == "generic"
    yr, ar = oracle.nnlib_attention_f32(q, k, v, bias, mask, H, nthreads=4)
    assert rel_err(y.to_numpy(), yr) <= TOL
    _check_alpha(a, ar, dtype, mask)
    # causal through the generic kernel
    q, k, v = _inputs(rng, dtype, E, Lq, Lq, B, Ev)
    y, a = _call(nn, q, k, v, dtype, H, causal=True, flags=flags)
    assert nn.last_attention_kernel() == "generic"
    cm = oracle.make_causal_mask(Lq)
    yr, ar = oracle.nnlib_attention_f32(q, k, v, None, cm, H, nthreads=4)
    assert rel_err(y.to_numpy(), yr) <= TOL
    _check_alpha(a, ar, dtype, cm)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_scores_native_weights(nn, oracle, dtype):
    """dot_product_attention_scores on 16-bit 4-D inputs returns 16-bit weights equal to those of the 3-D call."""
    rng = np.random.default_rng(45)
    D, H, Lq, Lkv, B = 64, 2, 90, 200, 2
    q = round_to(rng.standard_normal((D, H, Lq, B)), dtype)
    k = round_to(rng.standard_normal((D, H, Lkv, B)), dtype)
    mask = rng.random((Lkv, Lq)) < 0.8
    mask[0] = True
    a = nn.dot_product_attention_scores(nn.DeviceArray.from_numpy(q, dtype), nn.DeviceArray.from_numpy(k, dtype),
                                        mask=nn.DeviceArray.from_numpy(mask))
    q3, k3 = q.reshape(D * H, Lq, B, order="F"), k.reshape(D * H, Lkv, B, order="F")
    _, ar = oracle.nnlib_attention_f32(q3, k3, k3, None, mask, H, nthreads=4)
    _check_alpha(a, ar, dtype, mask)


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_native_weights_with_dropout(nn, dtype):
    """Fused dropout on 16-bit weights: the returned weights are the dropped ones (src/attention.jl:126), i.e. the
    Float32 weights times 0 or 1/(1-p), rounded once to the 16-bit type."""
    rng = np.random.default_rng(46)
    q, k, v = _inputs(rng, dtype, 128, 100, 264, 2)
    dq, dk, dv = (nn.DeviceArray.from_numpy(x, dtype) for x in (q, k, v))
    p = 0.25
    _, a_drop = nn.dot_product_attention(dq, dk, dv, nheads=2, fdrop=nn.Dropout(p, seed=7))
    _, a32 = nn.dot_product_attention(dq, dk, dv, nheads=2, weights_dtype="f32")
    keep = nn.dropout(nn.DeviceArray.from_numpy(np.ones(a32.dims, np.float32)), p, seed=7).to_numpy() > 0
    expect = round_to(np.where(keep, a32.to_numpy() / np.float32(1 - p), 0), dtype)
    got = a_drop.to_numpy().astype(np.float32)
    assert a_drop.dtype == dtype
    assert np.count_nonzero(got[~keep]) == 0
    assert np.abs(got - expect).max() <= UNIT_ROUNDOFF[dtype] * np.abs(expect).max() + 1e-6
