"""GPU parity of dot_product_attention / dot_product_attention_scores against the CPU oracle.

Patterned on the reference's own tests (test/attention.jl, test/ext_amdgpu/attention.jl).
Tolerances: Float32 max error <= 1e-4 of output scale; Float16/BFloat16 <= 1e-2 against the
Float32 CPU result on the same (already rounded) inputs; weight columns sum to 1 within 1e-5
(checked on Float32 weights).
"""
import itertools
import json
import os

import numpy as np
import pytest

from conftest import rel_err, round_to

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _run(nn, q, k, v, dtype, bias=None, mask=None, nheads=1, causal=False, **kw):
    dq, dk, dv = (nn.DeviceArray.from_numpy(a, dtype) for a in (q, k, v))
    db = nn.DeviceArray.from_numpy(bias, dtype) if bias is not None else None
    if causal:
        dm = nn.make_causal_mask(dq, dims=2)
    else:
        dm = nn.DeviceArray.from_numpy(mask) if mask is not None else None
    y, a = nn.dot_product_attention(dq, dk, dv, db, mask=dm, nheads=nheads, **kw)
    return y.to_numpy(), (a.to_numpy() if a is not None else None)


def _check(nn, oracle, rng, dtype, E, Lq, Lkv, B, H, *, Ev=None, causal=False, bias_shape=None, mask_shape=None,
           scale=1.0, expect=None, weights=True, batch_shape=None, flags=0):
    Ev = Ev or E
    bs = batch_shape if batch_shape is not None else (B,)
    q = round_to(rng.standard_normal((E, Lq) + bs) * scale, dtype)
    k = round_to(rng.standard_normal((E, Lkv) + bs) * scale, dtype)
    v = round_to(rng.standard_normal((Ev, Lkv) + bs), dtype)
    bias = round_to(0.5 * rng.standard_normal(bias_shape), dtype) if bias_shape else None
    mask = None
    if mask_shape:
        mask = rng.random(mask_shape) < 0.9
        mask[0, ...] = True          # no fully masked column
    omask = mask
    if causal:
        omask = oracle.make_causal_mask(Lq)
    y, a = _run(nn, q, k, v, dtype, bias, mask, H, causal, return_weights=weights,
                weights_dtype="f32" if weights else None, _flags=flags)
    if expect:
        assert nn.last_attention_kernel() == expect, nn.last_attention_kernel()
    yr, ar = oracle.nnlib_attention_f32(q, k, v, bias, omask, H, nthreads=8)
    assert y.shape == yr.shape
    yerr = rel_err(y, yr)
    assert yerr <= TOL[dtype], (yerr, nn.last_attention_kernel())
    if weights:
        assert a.shape == ar.shape
        werr = float(np.abs(a - ar).max())
        assert werr <= TOL[dtype], werr
        colsum_err = float(np.abs(a.sum(axis=0) - 1).max())
        assert colsum_err <= 1e-5, colsum_err
        if omask is not None:
            keep = np.broadcast_to(np.asarray(omask).reshape(omask.shape + (1,) * (a.ndim - omask.ndim)), a.shape)
            n_leaked = int(np.count_nonzero(a[~keep]))
            assert n_leaked == 0, n_leaked
    return y, a


def test_specific_results(nn):
    """Golden vectors of test/attention.jl:25-34."""
    g = json.load(open(os.path.join(GOLD, "attention_specific_results.json")))
    q = (np.arange(1, 13, dtype=np.float32) / 12).reshape(4, 3, 1, order="F")
    y, a = _run(nn, q, q, q, "f32", nheads=2)
    assert np.abs(y - np.array(g["ytrue"]).reshape(4, 3, 1, order="F")).max() < 1e-5
    assert np.abs(a - np.array(g["alphatrue"]).reshape(3, 3, 2, 1, order="F")).max() < 1e-5


@pytest.mark.parametrize("batch_shape", [(), (1,), (2,), (2, 1, 3)])
@pytest.mark.parametrize("nheads", [1, 3, 5])
def test_different_batchsizes(nn, oracle, batch_shape, nheads):
    """Shape grid of test/attention.jl:1-15 and test/ext_amdgpu/attention.jl:1-23."""
    rng = np.random.default_rng(0)
    n, lenq, lenkv = 15, 3, 4
    q = rng.random((n, lenq) + batch_shape, dtype=np.float32)
    k = rng.random((n, lenkv) + batch_shape, dtype=np.float32)
    v = rng.random((n, lenkv) + batch_shape, dtype=np.float32)
    y, a = _run(nn, q, k, v, "f32", nheads=nheads)
    assert y.shape == (n, lenq) + batch_shape
    assert a.shape == (lenkv, lenq, nheads) + batch_shape
    assert np.allclose(a.sum(axis=0), 1, atol=1e-6)
    yr, ar = oracle.nnlib_attention_f32(q, k, v, nheads=nheads)
    assert np.abs(y - yr).max() < 1e-5 and np.abs(a - ar).max() < 1e-5


def test_scores_equal_attention_weights(nn):
    """test/attention.jl:17-23."""
    q = (np.arange(1, 25, dtype=np.float32) / 24).reshape(4, 2, 3, 1, order="F")
    dq = nn.DeviceArray.from_numpy(q)
    a = nn.dot_product_attention_scores(dq, dq).to_numpy()
    q2 = nn.DeviceArray.from_numpy(q.reshape(8, 3, 1, order="F"))
    _, a2 = nn.dot_product_attention(q2, q2, q2, nheads=2)
    assert np.allclose(a, a2.to_numpy(), atol=1e-6)


def test_mask_zero_pattern(nn):
    """test/attention.jl:36-52: weights are positive exactly where the mask keeps."""
    rng = np.random.default_rng(1)
    q = rng.random((4, 2, 3, 1), dtype=np.float32)
    k = rng.random((4, 2, 5, 1), dtype=np.float32)
    mask = rng.random((5, 3)) < 0.5
    mask[0, :] = True
    a = nn.dot_product_attention_scores(nn.DeviceArray.from_numpy(q), nn.DeviceArray.from_numpy(k),
                                        mask=nn.DeviceArray.from_numpy(mask)).to_numpy()
    assert np.all((a[:, :, 0, 0] > 0) == mask) and np.all((a[:, :, 1, 0] > 0) == mask)
    x = nn.DeviceArray.from_numpy(rng.random((4, 2, 3, 1), dtype=np.float32))
    cm = nn.make_causal_mask(x, dims=3)
    a = nn.dot_product_attention_scores(x, x, mask=cm).to_numpy()
    dense = cm.to_numpy()
    assert dense.dtype == bool and np.array_equal(dense, np.triu(np.ones((3, 3), bool)))
    assert np.all((a[:, :, 0, 0] > 0) == dense) and np.all((a[:, :, 1, 0] > 0) == dense)


def test_bias_shapes(nn, oracle):
    """test/attention.jl:61-68."""
    rng = np.random.default_rng(2)
    q = rng.random((4, 5, 1), dtype=np.float32)
    k = rng.random((4, 3, 1), dtype=np.float32)
    bias = rng.standard_normal((3, 5)).astype(np.float32)
    y, a = _run(nn, q, k, k, "f32", bias=bias, nheads=2)
    assert a.shape == (3, 5, 2, 1) and y.shape == (4, 5, 1)
    yr, ar = oracle.nnlib_attention_f32(q, k, k, bias, None, 2)
    assert np.abs(y - yr).max() < 1e-5 and np.abs(a - ar).max() < 1e-5


def test_dropout_path(nn):
    """test/attention.jl:54-59: a non-identity fdrop runs scores -> fdrop -> batched_mul, and the
    returned weights are the dropped ones."""
    rng = np.random.default_rng(3)
    x = nn.DeviceArray.from_numpy(rng.random((10, 10, 10), dtype=np.float32))

    def fdrop(alpha, p=0.5):
        h = alpha.to_numpy()
        keep = np.random.default_rng(4).random(h.shape) > p
        return nn.DeviceArray.from_numpy((keep * h / (1 - p)).astype(np.float32))

    y, a = nn.dot_product_attention(x, x, x, nheads=2, fdrop=fdrop)
    a = a.to_numpy()
    assert 0.4 < np.mean(a > 0) < 0.6
    v4 = x.to_numpy().reshape(5, 2, 10, 10, order="F")
    ref = np.einsum("jihb,dhjb->dhib", a, v4).reshape(10, 10, 10, order="F")
    assert np.abs(y.to_numpy() - ref).max() < 1e-5


def test_errors(nn):
    """ArgumentError conditions of src/attention.jl:42,55-78."""
    z = lambda *d: nn.DeviceArray.zeros(d)
    with pytest.raises(nn.ArgumentError, match="divisible"):
        nn.dot_product_attention(z(6, 3, 1), z(6, 4, 1), z(6, 4, 1), nheads=4)
    with pytest.raises(nn.ArgumentError, match="Batch dimensions"):
        nn.dot_product_attention(z(6, 3, 2), z(6, 4, 1), z(6, 4, 1))
    with pytest.raises(nn.ArgumentError, match="query and key"):
        nn.dot_product_attention(z(6, 3, 1), z(4, 4, 1), z(6, 4, 1))
    with pytest.raises(nn.ArgumentError, match="key and value"):
        nn.dot_product_attention(z(6, 3, 1), z(6, 4, 1), z(6, 5, 1))
    with pytest.raises(nn.DimensionMismatch):
        nn.dot_product_attention(z(6, 3, 1), z(6, 4, 1), z(6, 4, 1), z(5, 3))


# ---- MFMA flash kernels against the oracle ---------------------------------------------------------

FLASH16_CASES = [
    # dtype, E, Lq, Lkv, B, H, kwargs
    ("bf16", 256, 128, 128, 2, 2, {}),
    ("bf16", 256, 200, 333, 1, 2, {}),                       # ragged tails in both lengths
    ("bf16", 256, 256, 256, 2, 2, dict(causal=True)),
    ("bf16", 256, 130, 130, 1, 2, dict(causal=True)),
    ("f16", 128, 96, 160, 2, 2, {}),
    ("f16", 128, 192, 192, 1, 2, dict(causal=True)),
    ("f16", 128, 64, 320, 2, 2, dict(bias_shape=(320, 64, 2, 2), mask_shape=(320, 64))),
    ("f16", 128, 70, 131, 2, 2, dict(bias_shape=(131, 70), mask_shape=(131, 70, 1, 2))),   # unaligned strides
    ("bf16", 128, 64, 256, 1, 1, dict(bias_shape=(256, 1, 1, 1))),
    ("bf16", 256, 128, 128, 1, 2, dict(causal=True, mask_shape=(128, 128))),
    ("f16", 64, 33, 65, 3, 1, {}),
    # 16-byte aligned bias / mask rows: tiles staged through LDS; ragged tails in both lengths
    ("f16", 128, 70, 336, 2, 2, dict(bias_shape=(336, 70, 2, 2), mask_shape=(336, 70, 1, 2))),
    ("bf16", 256, 150, 400, 1, 2, dict(bias_shape=(400, 150, 1, 1), mask_shape=(400, 1, 2, 1))),
    ("bf16", 128, 192, 192, 2, 2, dict(causal=True, bias_shape=(192, 192, 2, 1))),
    # masks that do not depend on the query (key-padding masks): one mask byte per key, raw-score path
    ("bf16", 256, 150, 400, 2, 2, dict(mask_shape=(400, 1, 1, 2))),
    ("f16", 128, 70, 131, 2, 2, dict(mask_shape=(131,))),                 # unaligned length: byte loads
    ("bf16", 128, 200, 520, 1, 2, dict(mask_shape=(520, 1, 2))),
    # dense masks without bias whose rows start 16-byte aligned: mask tiles staged alone, raw-score path
    ("bf16", 256, 150, 400, 2, 2, dict(mask_shape=(400, 150, 1, 2))),
    ("f16", 128, 70, 336, 2, 2, dict(mask_shape=(336, 70))),
    ("bf16", 192, 200, 208, 1, 2, dict(mask_shape=(208, 200, 2, 1))),     # head dim 96
    # long enough for the steady-state loop of the software-pipelined kernel, head dims 64 and 128
    ("bf16", 128, 300, 700, 1, 2, {}),
    ("bf16", 128, 520, 520, 1, 2, dict(causal=True)),
    ("f16", 64, 257, 1100, 2, 1, {}),
    ("f16", 128, 600, 600, 1, 2, dict(causal=True)),
    ("bf16", 256, 300, 700, 1, 2, {}),
    ("f16", 256, 520, 520, 1, 2, dict(causal=True)),
    # head dims below the 64- / 128-wide tiles (multiples of 8): zero-padded in flight
    ("bf16", 192, 200, 333, 1, 2, {}),                                   # 96
    ("f16", 64, 130, 130, 2, 2, dict(causal=True)),                      # 32
    ("bf16", 160, 150, 400, 1, 2, dict(bias_shape=(400, 150, 2, 1), mask_shape=(400, 150))),   # 80, staged tiles
    ("f16", 80, 70, 131, 2, 2, dict(bias_shape=(131, 70), mask_shape=(131, 70, 1, 2))),        # 40, unaligned strides
    ("bf16", 96, 90, 200, 2, 2, dict(Ev=224)),                           # q, k: 48; v: 112
    ("f16", 240, 64, 256, 1, 2, dict(Ev=48, causal=False, mask_shape=(256, 1, 1, 1))),   # q, k: 120; v: 24; key mask
    ("bf16", 16, 40, 70, 3, 2, {}),                                      # 8
    ("bf16", 224, 520, 520, 1, 2, dict(causal=True)),                    # 112, long
    # head dims above 128 up to 256: 256-wide tiles, one workgroup per CU, bias / mask on the direct path
    ("bf16", 512, 200, 333, 1, 2, {}),                                   # 256
    ("f16", 384, 260, 260, 2, 2, dict(causal=True)),                     # 192
    ("bf16", 320, 150, 400, 1, 2, dict(bias_shape=(400, 150, 2, 1), mask_shape=(400, 150))),   # 160
    ("f16", 512, 70, 131, 2, 2, dict(Ev=144, mask_shape=(131, 1, 1, 2))),                      # q, k: 256; v: 72
    ("bf16", 136, 100, 520, 1, 1, dict(Ev=256, mask_shape=(520,))),                            # q, k: 136; v: 256; key mask
]


@pytest.mark.parametrize("case", FLASH16_CASES, ids=lambda c: f"{c[0]}-E{c[1]}-Lq{c[2]}-Lkv{c[3]}-B{c[4]}-H{c[5]}-" + "-".join(c[6]))
@pytest.mark.parametrize("weights", [False, True], ids=["noweights", "weights"])
def test_flash16_parity(nn, oracle, case, weights):
    dtype, E, Lq, Lkv, B, H, kw = case
    rng = np.random.default_rng(hash((E, Lq, Lkv, B, H)) % 2**32)
    _check(nn, oracle, rng, dtype, E, Lq, Lkv, B, H, expect="flash16", weights=weights, **kw)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_generic_kernel_parity(nn, oracle, dtype):
    """The generic kernel on a shape the MFMA kernels do not take (head dims 22 / 42: rows are not whole
    16-byte chunks)."""
    rng = np.random.default_rng(7)
    _check(nn, oracle, rng, dtype, 44, 37, 75, 2, 2, Ev=84, bias_shape=(75, 37, 2, 1), mask_shape=(75, 37),
           expect="generic")


def test_flash16_matches_generic_on_device(nn):
    """Both kernels on identical device buffers (bf16, causal)."""
    rng = np.random.default_rng(8)
    q, k, v = (nn.DeviceArray.from_numpy(rng.standard_normal((256, 192, 2)).astype(np.float32), "bf16") for _ in range(3))
    cm = nn.make_causal_mask(q)
    y1, a1 = nn.dot_product_attention(q, k, v, mask=cm, nheads=2, weights_dtype="f32")
    assert nn.last_attention_kernel() == "flash16"
    y2, a2 = nn.dot_product_attention(q, k, v, mask=cm, nheads=2, weights_dtype="f32", _flags=1)
    assert nn.last_attention_kernel() == "generic"
    assert rel_err(y1.to_numpy(), y2.to_numpy()) < 1e-2
    assert np.abs(a1.to_numpy() - a2.to_numpy()).max() < 1e-2


def test_fully_masked_column_is_nan(nn):
    """src/softmax.jl:73-75 gives exp(-Inf - -Inf) = NaN for an all-dropped column (by code reading;
    no reference test pins it).  Both kernel families must agree with that."""
    rng = np.random.default_rng(9)
    for dtype, E, H, flags in (("f32", 12, 2, 0), ("f32", 16, 2, 0), ("bf16", 128, 1, 0)):   # generic, flash32, flash16
        q = rng.standard_normal((E, 40, 1)).astype(np.float32)
        k = rng.standard_normal((E, 70, 1)).astype(np.float32)
        mask = np.ones((70, 40), bool)
        mask[:, 5] = False
        y, a = _run(nn, q, k, k, dtype, mask=mask, nheads=H, weights_dtype="f32")
        assert np.isnan(y[:, 5, 0]).all() and np.isnan(a[:, 5]).all()
        assert np.isfinite(np.delete(y, 5, axis=1)).all()


FLASH32_CASES = [
    ("f32", 128, 128, 128, 2, 2, {}),
    ("f32", 128, 200, 333, 1, 2, {}),
    ("f32", 256, 130, 130, 1, 2, dict(causal=True)),
    ("f32", 128, 256, 256, 2, 2, dict(causal=True, scale=0.125)),
    ("f32", 128, 64, 320, 2, 2, dict(bias_shape=(320, 64, 2, 2), mask_shape=(320, 64))),
    ("f32", 128, 70, 131, 2, 2, dict(bias_shape=(131, 70), mask_shape=(131, 70, 1, 2))),
    ("f32", 256, 96, 96, 1, 2, dict(causal=True, mask_shape=(96, 96))),
    ("f32", 64, 33, 65, 3, 1, {}),
    # head dims below the tile width (multiples of 4)
    ("f32", 192, 200, 333, 1, 2, {}),                                    # 96
    ("f32", 72, 130, 130, 2, 2, dict(causal=True)),                      # 36
    ("f32", 48, 70, 131, 2, 2, dict(Ev=160, bias_shape=(131, 70), mask_shape=(131, 70, 1, 2))),   # q, k: 24; v: 80
    ("f32", 8, 40, 70, 3, 2, {}),                                        # 4
]


@pytest.mark.parametrize("case", FLASH32_CASES, ids=lambda c: f"{c[0]}-E{c[1]}-Lq{c[2]}-Lkv{c[3]}-B{c[4]}-H{c[5]}-" + "-".join(c[6]))
@pytest.mark.parametrize("weights", [False, True], ids=["noweights", "weights"])
def test_flash32_parity(nn, oracle, case, weights):
    dtype, E, Lq, Lkv, B, H, kw = case
    rng = np.random.default_rng(hash((E, Lq, Lkv, B, H, 32)) % 2**32)
    _check(nn, oracle, rng, dtype, E, Lq, Lkv, B, H, expect="flash32", weights=weights, **kw)


SMALL_F32_CASES = [
    # Float32, at most 128 keys, weights returned: every load up front, scores kept in registers between the statistics
    # and the weights (one pass).  Ragged key counts around the 64-key tile, ragged and multi-tile query counts,
    # head dims below the 64-wide tile, every combination of causal / bias / mask the two-pass kernel takes.
    (64, 1, 1, 1, 1, {}),
    (64, 37, 63, 2, 1, {}),
    (128, 129, 64, 1, 2, {}),
    (128, 300, 65, 2, 2, {}),
    (512, 128, 128, 4, 8, {}),                                           # the smallest benchmark configuration
    (128, 128, 128, 2, 2, dict(causal=True)),
    (96, 127, 127, 1, 2, dict(causal=True, scale=0.125)),
    (40, 65, 65, 3, 2, dict(causal=True)),                               # second key tile: one key, one query
    (128, 70, 128, 2, 2, dict(bias_shape=(128, 70, 2, 2), mask_shape=(128, 70))),
    (56, 131, 66, 2, 2, dict(bias_shape=(66, 131), mask_shape=(66, 131, 1, 2))),
    (128, 96, 96, 1, 2, dict(causal=True, mask_shape=(96, 96))),
    (48, 33, 90, 2, 2, dict(Ev=96, mask_shape=(90, 1, 2, 2))),           # v wider than q, k; key-padding style mask
    # more than 256 blocks of 32 queries: the workgroup of eight wavefronts (one per key tile and query block)
    # instead of one workgroup of four per query block
    (512, 160, 128, 8, 8, {}),
    (256, 97, 97, 17, 4, dict(causal=True)),
    (128, 1100, 100, 4, 2, dict(bias_shape=(100, 1100, 2, 1), mask_shape=(100, 1100))),
    (256, 128, 128, 17, 4, dict(causal=True, mask_shape=(128, 128, 1, 17))),
    (512, 160, 64, 8, 8, {}),                                            # at most 64 keys and many blocks: two workgroups per compute unit
    (256, 60, 60, 33, 4, dict(causal=True)),
    (128, 1100, 50, 4, 2, dict(bias_shape=(50, 1100, 2, 1), mask_shape=(50, 1100))),
]


@pytest.mark.parametrize("case", SMALL_F32_CASES, ids=lambda c: f"E{c[0]}-Lq{c[1]}-Lkv{c[2]}-B{c[3]}-H{c[4]}-" + "-".join(c[5]))
def test_small_float32_problem_with_weights(nn, oracle, case):
    E, Lq, Lkv, B, H, kw = case
    rng = np.random.default_rng(1000 * E + 10 * Lq + Lkv)
    _check(nn, oracle, rng, "f32", E, Lq, Lkv, B, H, expect="flash32", weights=True, **kw)


@pytest.mark.parametrize("case", [c for c in SMALL_F32_CASES if (c[1] + 31) // 32 * c[3] * c[4] <= 256],
                         ids=lambda c: f"E{c[0]}-Lq{c[1]}-Lkv{c[2]}-B{c[3]}-H{c[4]}-" + "-".join(c[5]))
def test_small_float32_problem_without_weights(nn, oracle, case):
    """Calls of at most 256 blocks of 32 queries take the one-pass kernel without the weights output too."""
    E, Lq, Lkv, B, H, kw = case
    rng = np.random.default_rng(1000 * E + 10 * Lq + Lkv + 1)
    _check(nn, oracle, rng, "f32", E, Lq, Lkv, B, H, expect="flash32", weights=False, **kw)


MID_F32_CASES = [
    # Float32, 129 to 512 keys (1024 at head dims up to 64), few blocks of 32 queries: a workgroup per query block that keeps the scores of
    # every 128-key chunk in registers (one to four chunks, ragged last chunk and last block, causal diagonal inside a
    # chunk, bias / mask, v wider than q and k)
    (128, 129, 129, 1, 2, {}),
    (512, 256, 256, 4, 8, {}),
    (256, 100, 512, 2, 4, {}),
    (128, 77, 385, 3, 2, {}),
    (64, 300, 300, 1, 1, dict(causal=True)),
    (512, 256, 256, 4, 8, dict(causal=True)),
    (128, 511, 511, 1, 2, dict(causal=True, scale=0.125)),
    (128, 70, 200, 2, 2, dict(bias_shape=(200, 70, 2, 2), mask_shape=(200, 70))),
    (56, 131, 450, 2, 2, dict(bias_shape=(450, 131), mask_shape=(450, 131, 1, 2))),
    (128, 260, 260, 1, 2, dict(causal=True, mask_shape=(260, 260))),
    (48, 33, 290, 2, 2, dict(Ev=96, bias_shape=(290, 33, 2, 1))),
    # head dims above 64 (128-wide tiles: one chunk buffer)
    (1024, 128, 128, 4, 8, {}),
    (256, 100, 100, 2, 2, dict(causal=True)),
    (192, 77, 385, 3, 2, {}),
    (144, 260, 260, 1, 2, dict(causal=True, mask_shape=(260, 260))),
    (256, 70, 200, 2, 2, dict(bias_shape=(200, 70, 2, 2), mask_shape=(200, 70))),
    (128, 40, 512, 2, 1, dict(Ev=96, bias_shape=(512, 40))),
    (80, 1, 130, 2, 1, {}),
    # 513 to 1024 keys at head dims up to 64: eight chunks
    (128, 100, 1024, 1, 2, {}),
    (64, 700, 700, 1, 1, dict(causal=True)),
    (128, 40, 770, 2, 2, dict(bias_shape=(770, 40, 2, 1), mask_shape=(770, 40))),
    (96, 513, 513, 1, 3, dict(causal=True, mask_shape=(513, 513))),
    # 257 to 512 blocks: with the weights or the causal mask this kernel, otherwise the two-pass kernel
    (256, 256, 256, 12, 4, {}),
    (256, 200, 200, 16, 4, dict(causal=True)),
]


@pytest.mark.parametrize("weights", [True, False], ids=["weights", "no-weights"])
@pytest.mark.parametrize("case", MID_F32_CASES, ids=lambda c: f"E{c[0]}-Lq{c[1]}-Lkv{c[2]}-B{c[3]}-H{c[4]}-" + "-".join(c[5]))
def test_mid_float32_problem_on_few_workgroups(nn, oracle, case, weights):
    E, Lq, Lkv, B, H, kw = case
    rng = np.random.default_rng(1000 * E + 10 * Lq + Lkv + 7)
    _check(nn, oracle, rng, "f32", E, Lq, Lkv, B, H, expect="flash32", weights=weights, **kw)


def test_small_float32_problem_special_values(nn, oracle):
    """+Inf logits (src/softmax.jl:73-75: the weights become the indicator of the +Inf entries, normalised), a query
    with nothing kept (NaN) and scores without a value product, at a size the one-pass kernel takes."""
    rng = np.random.default_rng(77)
    E, Lq, Lkv, H = 64, 40, 100, 2
    q, k, v = (rng.standard_normal((E, L, 1)).astype(np.float32) for L in (Lq, Lkv, Lkv))
    bias = (0.3 * rng.standard_normal((Lkv, Lq))).astype(np.float32)
    bias[3, 7] = bias[90, 7] = np.inf                 # two +Inf logits in one column, in different key tiles
    bias[70, 9] = np.inf
    mask = rng.random((Lkv, Lq)) < 0.8
    mask[:, 11] = False                               # nothing kept
    mask[3, 7] = mask[90, 7] = mask[70, 9] = True
    with np.errstate(invalid="ignore", over="ignore"):
        yr, ar = oracle.nnlib_attention_f32(q, k, v, bias, mask, H, nthreads=4)
    y, a = _run(nn, q, k, v, "f32", bias, mask, H, weights_dtype="f32")
    assert nn.last_attention_kernel() == "flash32"
    assert np.array_equal(np.isnan(a), np.isnan(ar)) and np.array_equal(np.isnan(y), np.isnan(yr))
    assert np.isnan(a[:, 11]).all() and np.isnan(y[:, 11]).all()
    ok = ~np.isnan(ar)
    assert np.abs(a[ok] - ar[ok]).max() <= 1e-5
    assert a[3, 7, 0, 0] == 0.5 and a[90, 7, 0, 0] == 0.5 and a[70, 9, 1, 0] == 1.0
    oky = ~np.isnan(yr)
    assert np.abs(y[oky] - yr[oky]).max() <= 1e-4 * np.abs(yr[oky]).max()
    # scores only (no values, no output)
    D = nn.DeviceArray.from_numpy
    q4, k4 = (x.reshape(E // H, H, -1, 1, order="F") for x in (q, k))
    s = nn.dot_product_attention_scores(D(q4), D(k4), D(bias)).to_numpy()
    assert nn.last_attention_kernel() == "flash32"
    with np.errstate(invalid="ignore", over="ignore"):
        sr = oracle.nnlib_attention_f32(q, k, v, bias, None, H, nthreads=4)[1]
    assert np.abs(s - sr).max() <= 1e-5


@pytest.mark.parametrize("dtype,E,H,Lkv,B", [("bf16", 512, 4, 1500, 2), ("bf16", 256, 2, 4096, 3), ("f16", 512, 8, 777, 1),
                                             ("f16", 1024, 8, 2048, 2), ("bf16", 128, 1, 513, 1),
                                             ("f32", 512, 4, 1500, 2), ("f32", 256, 4, 2048, 3), ("f32", 64, 1, 777, 1)])
@pytest.mark.parametrize("weights", [False, True], ids=["noweights", "weights"])
def test_decode_parity(nn, oracle, dtype, E, H, Lkv, B, weights):
    """Split-kv path for a single query per (head, batch); with the weights returned (as the reference always does)
    the raw scores are kept and normalised by a third kernel."""
    rng = np.random.default_rng(E + Lkv)
    _check(nn, oracle, rng, dtype, E, 1, Lkv, B, H, expect="decode", weights=weights)


@pytest.mark.parametrize("dtype,E,H,mask_shape", [("bf16", 512, 4, (1500, 1, 1, 3)), ("f16", 256, 4, (1500, 1, 4, 3)),
                                                  ("bf16", 128, 2, (1500,)), ("f32", 256, 2, (1500, 1, 2, 3))])
def test_decode_with_context_length_masks(nn, oracle, dtype, E, H, mask_shape):
    """A single query per (head, batch) with a mask: padded contexts of different lengths per batch element, a
    pattern per head, one (head, batch) pair with nothing kept (NaN, src/softmax.jl:73-75)."""
    rng = np.random.default_rng(5)
    Lkv, B = 1500, 3
    q, k, v = (round_to(rng.standard_normal((E, L, B)), dtype) for L in (1, Lkv, Lkv))
    mask = rng.random(mask_shape) < 0.6
    if len(mask_shape) == 4:
        mask[900:, 0, :, 0] = False                  # context of 900 keys
        mask[:700, 0, :, 1] = False                  # whole leading splits dropped
        mask[:, 0, 0, 2] = False                     # nothing kept for (head 0 or all heads, batch 2)
    with np.errstate(invalid="ignore"):
        yr, ar = oracle.nnlib_attention_f32(q, k, v, None, mask, H, nthreads=4)
    for weights in (False, True):
        y, a = _run(nn, q, k, v, dtype, None, mask, H, return_weights=weights, weights_dtype="f32" if weights else None)
        assert nn.last_attention_kernel() == "decode"
        assert np.array_equal(np.isnan(y), np.isnan(yr))
        if len(mask_shape) == 4:
            assert np.isnan(y).any()
        ok = ~np.isnan(yr)
        assert np.abs(y[ok] - yr[ok]).max() / np.abs(yr[ok]).max() <= TOL[dtype]
        if weights:
            assert np.array_equal(np.isnan(a), np.isnan(ar))
            okw = ~np.isnan(ar)
            assert np.abs(a[okw] - ar[okw]).max() <= TOL[dtype]
            assert np.count_nonzero(a[okw & ~np.broadcast_to(mask.reshape(mask.shape + (1,) * (4 - mask.ndim)), a.shape)]) == 0


def test_decode_matches_generic_on_device(nn):
    rng = np.random.default_rng(11)
    q = nn.DeviceArray.from_numpy(rng.standard_normal((512, 1, 2)).astype(np.float32), "bf16")
    k = nn.DeviceArray.from_numpy(rng.standard_normal((512, 3000, 2)).astype(np.float32), "bf16")
    v = nn.DeviceArray.from_numpy(rng.standard_normal((512, 3000, 2)).astype(np.float32), "bf16")
    y1, _ = nn.dot_product_attention(q, k, v, nheads=4, return_weights=False)
    assert nn.last_attention_kernel() == "decode"
    y2, _ = nn.dot_product_attention(q, k, v, nheads=4, return_weights=False, _flags=nn._lib.MI_ATTN_FORCE_GENERIC)
    assert nn.last_attention_kernel() == "generic"
    assert rel_err(y1.to_numpy(), y2.to_numpy()) < 1e-2


SPLIT_CASES = [
    ("f16", 128, 100, 3000, 1, 2, dict(bias_shape=(3000, 100, 2, 1), mask_shape=(3000, 100))),
    ("f16", 128, 256, 4096, 2, 2, dict(bias_shape=(4096, 256, 2, 2))),
    ("bf16", 128, 2048, 2048, 1, 2, dict(causal=True)),            # head dim 64: general kernel, causal pieces
    ("bf16", 64, 70, 2500, 3, 1, {}),
    ("f16", 256, 130, 2100, 1, 2, dict(mask_shape=(2100, 130))),    # head dim 128 with a mask
    ("bf16", 192, 130, 2100, 1, 2, dict(Ev=160, mask_shape=(2100, 130))),   # head dims 96 / 80 in 128-wide tiles
    ("f16", 96, 70, 2500, 2, 2, {}),                                  # head dim 48 in 64-wide tiles
    ("bf16", 256, 100, 2300, 2, 1, {}),                               # head dim 256
    ("f16", 256, 130, 2112, 1, 2, dict(mask_shape=(2112, 130))),      # mask tiles staged alone
    # Float32: the same split + merge
    ("f32", 128, 100, 3000, 1, 2, dict(bias_shape=(3000, 100, 2, 1), mask_shape=(3000, 100))),
    ("f32", 64, 70, 2500, 3, 1, {}),
    ("f32", 256, 130, 2100, 1, 2, dict(mask_shape=(2100, 130))),
    ("f32", 72, 300, 4096, 1, 2, dict(Ev=160)),                       # head dims 36 / 80
    ("f32", 128, 2048, 2048, 1, 2, dict(causal=True)),
]


@pytest.mark.parametrize("case", SPLIT_CASES, ids=lambda c: f"{c[0]}-E{c[1]}-Lq{c[2]}-Lkv{c[3]}-B{c[4]}-H{c[5]}-" + "-".join(c[6]))
def test_split_kv_parity(nn, oracle, case):
    """Few (query tile, head, batch) workgroups and a long key range: the key range is cut into pieces,
    one workgroup each, and a second kernel merges the partial (m, l, o)."""
    dtype, E, Lq, Lkv, B, H, kw = case
    rng = np.random.default_rng(hash((E, Lq, Lkv, B, H, 7)) % 2**32)
    import ctypes
    _check(nn, oracle, rng, dtype, E, Lq, Lkv, B, H, expect="flash32" if dtype == "f32" else "flash16", weights=False, **kw)
    from nnlib_amd import ops
    assert ops._workspace is not None and ops._workspace.numel() > 0      # the split path was taken


def test_split_kv_fully_masked_query(nn):
    rng = np.random.default_rng(12)
    q = rng.standard_normal((128, 40, 1)).astype(np.float32)
    k = rng.standard_normal((128, 2600, 1)).astype(np.float32)
    mask = np.ones((2600, 40), bool)
    mask[:, 7] = False
    mask[:2000, 9] = False             # whole pieces masked, but not the query
    y, _ = _run(nn, q, k, k, "f16", mask=mask, nheads=2, return_weights=False)
    assert np.isnan(y[:, 7, 0]).all()
    assert np.isfinite(np.delete(y, 7, axis=1)).all()


@pytest.mark.parametrize("dtype,E,Lkv,expect", [("f32", 128, 136, "flash32"), ("f16", 128, 144, "flash16"),
                                                ("bf16", 128, 131, "flash16"), ("f16", 44, 75, "generic")],
                         ids=["flash32", "flash16-staged", "flash16-direct", "generic"])
@pytest.mark.parametrize("weights", [False, True], ids=["noweights", "weights"])
def test_plus_inf_logits(nn, oracle, dtype, E, Lkv, expect, weights):
    """src/softmax.jl:69-75: a column whose maximum is +Inf becomes the normalised indicator of its +Inf
    entries.  +Inf enters through the bias; one query has it in two tiles, one in a later tile only."""
    rng = np.random.default_rng(31)
    Lq, B, H = 40, 2, 2
    q = round_to(rng.standard_normal((E, Lq, B)), dtype)
    k = round_to(rng.standard_normal((E, Lkv, B)), dtype)
    v = round_to(rng.standard_normal((E, Lkv, B)), dtype)
    bias = round_to(0.5 * rng.standard_normal((Lkv, Lq, H, B)), dtype)
    bias[3, 5] = np.inf
    bias[Lkv - 2, 5] = np.inf
    bias[70, 9] = np.inf
    bias[0, 11, 1, 0] = np.inf
    y, a = _run(nn, q, k, v, dtype, bias, None, H, return_weights=weights, weights_dtype="f32")
    assert nn.last_attention_kernel() == expect
    yr, ar = oracle.nnlib_attention_f32(q, k, v, bias, None, H)
    assert np.isfinite(yr).all()
    tol = 1e-4 if dtype == "f32" else 1e-2
    assert rel_err(y, yr) < tol
    if weights:
        assert np.allclose(a, ar, atol=tol)
        assert a[3, 5, 0, 0] == 0.5 and a[Lkv - 2, 5, 1, 1] == 0.5 and a[70, 9, 0, 1] == 1.0 and a[1, 5, 0, 0] == 0.0


@pytest.mark.parametrize("dtype,E,H", [("bf16", 256, 2), ("f16", 128, 2)])
@pytest.mark.parametrize("weights", [False, True], ids=["noweights", "weights"])
def test_key_padding_masks(nn, oracle, dtype, E, H, weights):
    """Masks broadcast along the queries (batched sequences of different lengths): a padded tail, a dropped head
    that spans the whole first tile, scattered keys, and one batch element with every key dropped (NaN, as
    src/softmax.jl:73-75 gives for a fully masked column)."""
    rng = np.random.default_rng(21)
    Lq, Lkv, B = 140, 330, 4
    q, k, v = (round_to(rng.standard_normal((E, L, B)), dtype) for L in (Lq, Lkv, Lkv))
    mask = np.ones((Lkv, 1, 1, B), dtype=bool)
    mask[250:, 0, 0, 0] = False            # padded tail
    mask[:100, 0, 0, 1] = False            # the first tile and a half dropped
    mask[:, 0, 0, 2] = rng.random(Lkv) < 0.5
    mask[:, 0, 0, 3] = False               # nothing kept
    y, a = _run(nn, q, k, v, dtype, None, mask, H, return_weights=weights, weights_dtype="f32" if weights else None)
    assert nn.last_attention_kernel() == "flash16"
    with np.errstate(invalid="ignore"):
        yr, ar = oracle.nnlib_attention_f32(q, k, v, None, mask, H, nthreads=4)
    assert np.isnan(y[:, :, 3]).all() and np.isnan(yr[:, :, 3]).all()
    assert rel_err(y[:, :, :3], yr[:, :, :3]) <= TOL[dtype]
    if weights:
        assert np.isnan(a[..., 3]).all()
        assert np.abs(a[..., :3] - ar[..., :3]).max() <= TOL[dtype]
        keep = np.broadcast_to(mask, a.shape)[..., :3]
        assert np.count_nonzero(a[..., :3][~keep]) == 0


@pytest.mark.parametrize("dtype,E,H,Lq,Lkv", [("bf16", 256, 2, 140, 332), ("f16", 128, 2, 300, 1100), ("bf16", 128, 1, 513, 2048),
                                              ("f32", 128, 2, 140, 332), ("f32", 72, 2, 300, 1100),
                                              ("bf16", 256, 2, 140, 333), ("f16", 64, 1, 513, 2049), ("f32", 128, 2, 140, 333)])
@pytest.mark.parametrize("per_head", [False, True], ids=["per-batch", "per-head"])
def test_context_length_masks(nn, oracle, dtype, E, H, Lq, Lkv, per_head):
    """Key-padding masks that keep a prefix of the keys (padded batches): a device-side pass measures every (head,
    batch) pair, the software-pipelined kernel computes the pairs whose mask is a context length as a shorter L_kv and
    the general kernel the rest (scattered masks, an empty one: NaN).  Every pair must come from exactly one of them."""
    rng = np.random.default_rng(Lq + Lkv)
    B = 6
    q, k, v = (round_to(rng.standard_normal((E, L, B)), dtype) for L in (Lq, Lkv, Lkv))
    mask = np.ones((Lkv, 1, H if per_head else 1, B), dtype=bool)
    mask[Lkv - 82:, 0, :, 0] = False            # context length Lkv - 82
    mask[1:, 0, :, 1] = False                   # a single key
    mask[:, 0, :, 3] = rng.random((Lkv, mask.shape[2])) < 0.5   # scattered: not a prefix
    mask[:, 0, :, 4] = False                    # nothing kept
    mask[:37, 0, :, 5] = False                  # a suffix is kept: not a prefix
    if per_head:
        mask[200:, 0, 0, 2] = False             # batch element 2: one head padded, the others full
    with np.errstate(invalid="ignore"):
        yr, ar = oracle.nnlib_attention_f32(q, k, v, None, mask, H, nthreads=4)
    ok = [0, 1, 2, 3, 5]
    for weights in (False, True):   # with the weights: the general kernels' variant without mask code takes the pairs with a length
        y, a = _run(nn, q, k, v, dtype, None, mask, H, return_weights=weights, weights_dtype="f32" if weights else None)
        assert nn.last_attention_kernel() == ("flash32" if dtype == "f32" else "flash16")
        assert np.isnan(y[:, :, 4]).all() and np.isnan(yr[:, :, 4]).all()
        assert not np.isnan(y[:, :, ok]).any()
        assert rel_err(y[:, :, ok], yr[:, :, ok]) <= TOL[dtype]
        if weights:
            assert np.abs(a[..., ok] - ar[..., ok]).max() <= TOL[dtype]
            keep = np.broadcast_to(mask, a.shape)[..., ok]
            assert np.count_nonzero(a[..., ok][~keep]) == 0          # exact zeros past the context length
            assert np.abs(a[..., ok].sum(axis=0) - 1).max() <= 1e-5


@pytest.mark.parametrize("dtype,D,H,L,B,causal", [("bf16", 128, 4, 512, 40, True), ("bf16", 128, 4, 512, 40, False),
                                                  ("f16", 64, 8, 768, 16, True), ("bf16", 128, 2, 1024, 36, True),
                                                  ("f16", 128, 3, 256, 90, False)])
def test_prefill_parity_on_grids_larger_than_the_chip(nn, oracle, dtype, D, H, L, B, causal):
    """More (query tile, head, batch) workgroups than CUs on the software-pipelined kernel (whole 256-row query tiles,
    L_kv a multiple of 256): several rounds of workgroups per CU.  Every column of every workgroup is checked."""
    rng = np.random.default_rng(L + B)
    E = D * H
    q, k, v = (round_to(rng.standard_normal((E, L, B)), dtype) for _ in range(3))
    y, _ = _run(nn, q, k, v, dtype, None, None, H, causal, return_weights=False)
    assert nn.last_attention_kernel() == "flash16"
    yr, _ = oracle.nnlib_attention_f32(q, k, v, None, oracle.make_causal_mask(L) if causal else None, H, nthreads=8)
    err = np.abs(y - yr).reshape(E, -1).max(axis=0) / np.abs(yr).max()          # per (query, batch) column
    assert err.max() <= TOL[dtype], (float(err.max()), int(err.argmax()))


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,B,causal,split", [
    ("bf16", 128, 4, 256, 4096, 2, False, True),     # 8 workgroups of 256 queries: the keys are cut into pieces
    ("f16", 64, 8, 200, 8192, 1, False, True),
    ("bf16", 128, 2, 130, 2500, 3, False, True),     # ragged lengths on the split path
    ("bf16", 128, 8, 4096, 4096, 1, True, True),     # 128 unequal causal jobs: split as well
    ("bf16", 128, 4, 256, 1024, 2, False, False),    # too few keys to cut: stays one piece
    ("bf16", 128, 32, 1024, 2048, 2, False, False),  # 256 workgroups: the pipelined kernel keeps the call
])
def test_few_queries_many_keys_take_the_split_kernel(nn, oracle, dtype, D, H, Lq, Lkv, B, causal, split):
    """Calls without bias / mask / weights whose (256-query tile, head, batch) count cannot fill the chip leave the
    software-pipelined kernel, which never splits the keys, for the general kernel with a split key range (seen from
    outside as a workspace request); parity holds on both sides of the rule."""
    rng = np.random.default_rng(Lq + Lkv)
    E = D * H
    q = round_to(rng.standard_normal((E, Lq, B)), dtype)
    k, v = (round_to(rng.standard_normal((E, Lkv, B)), dtype) for _ in range(2))
    y, _ = _run(nn, q, k, v, dtype, None, None, H, causal, return_weights=False)
    assert nn.last_attention_kernel() == "flash16"
    assert (nn.last_attention_workspace() > 0) == split
    yr, _ = oracle.nnlib_attention_f32(q, k, v, None, oracle.make_causal_mask(Lq) if causal else None, H, nthreads=8)
    err = np.abs(y - yr).reshape(E, -1).max(axis=0) / np.abs(yr).max()
    assert err.max() <= TOL[dtype], (float(err.max()), int(err.argmax()))


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("pattern", ["rise5", "rise20", "fall", "zigzag"])
@pytest.mark.parametrize("weights", [False, True], ids=["noweights", "weights"])
def test_logits_that_drift_along_the_keys(nn, oracle, dtype, pattern, weights):
    """The kernels raise their running maximum only when a tile outgrows it by 2^8, so weights relative to a stale
    maximum reach 2^8 before the next rescale.  Logits that climb by about 5 or 20 powers of two per 64-key tile, fall,
    or alternate exercise every branch of that rule; results must still match the reference arithmetic."""
    rng = np.random.default_rng(11)
    D, H, L, B = 64, 2, 640, 2
    E = D * H
    per_tile = {"rise5": 5.0, "rise20": 20.0, "fall": -5.0, "zigzag": 5.0}[pattern] * np.log(2.0)
    j = np.arange(L, dtype=np.float64)
    ramp = per_tile * (j / 64.0)
    if pattern == "zigzag":
        ramp = per_tile * 2.0 * ((np.floor(j / 64.0) % 2) * 2 - 1)
    # logits = (k . q) / sqrt(D): q = 1 on every feature, k_j = ramp_j / sqrt(D) on every feature, plus noise
    q = round_to(np.ones((E, L, B)) + 0.05 * rng.standard_normal((E, L, B)), dtype)
    k = round_to((ramp / np.sqrt(D))[None, :, None] + 0.05 * rng.standard_normal((E, L, B)), dtype)
    v = round_to(rng.standard_normal((E, L, B)), dtype)
    y, a = _run(nn, q, k, v, dtype, None, None, H, False, return_weights=weights, weights_dtype="f32" if weights else None)
    yr, ar = oracle.nnlib_attention_f32(q, k, v, None, None, H, nthreads=8)
    assert rel_err(y, yr) <= TOL[dtype], (rel_err(y, yr), nn.last_attention_kernel())
    if weights:
        assert float(np.abs(a - ar).max()) <= TOL[dtype]
        assert float(np.abs(a.sum(axis=0) - 1).max()) <= 1e-5


def _mask_words_bytes(Lq, Lkv, slices):
    """Workspace of a call that takes the software-pipelined kernel with a packed dense mask: 16 bytes per query
    (rounded up to 256) and group of 128 keys, per mask slice."""
    return slices * ((Lkv + 127) // 128) * ((Lq + 255) // 256 * 256) * 16


DENSE_MASK_CASES = [
    # dtype, E, Lq, Lkv, B, H, causal, mask shape
    ("bf16", 256, 300, 700, 2, 2, False, (700, 300)),                # head dim 128, one mask for all, ragged sizes
    ("bf16", 256, 520, 520, 1, 2, True, (520, 520)),                  # causal .& array
    ("f16", 128, 257, 1100, 2, 2, False, (1100, 257, 2, 1)),          # head dim 64, a mask per head
    ("f16", 256, 600, 600, 2, 2, True, (600, 600, 1, 2)),             # a mask per batch element, causal
    ("bf16", 128, 700, 300, 3, 1, False, (300, 700, 1, 3)),
    ("bf16", 512, 1030, 1290, 1, 4, False, (1290, 1030)),             # more than four tiles: the unrolled steady loop
    ("f16", 256, 1500, 1500, 1, 4, True, (1500, 1500, 4, 1)),
]


@pytest.mark.parametrize("case", DENSE_MASK_CASES, ids=lambda c: f"{c[0]}-E{c[1]}-Lq{c[2]}-Lkv{c[3]}-B{c[4]}-H{c[5]}-{'causal' if c[6] else 'plain'}-mask{'x'.join(map(str, c[7]))}")
def test_dense_masks_on_the_pipelined_kernel(nn, oracle, case):
    """Query-dependent Bool masks without bias, weights and dropout: packed into bits by a pre-pass and applied by the
    software-pipelined kernel (the plan's workspace is the packed mask).  Besides a random mask the rows hold the
    special cases of a running maximum that starts without a kept key: a query that keeps nothing (NaN, as the
    reference's softmax over a column of -Inf gives, src/softmax.jl:73-75), queries whose first kept key comes blocks
    later, a query that keeps only the last key, and a query whose only kept keys score far below the masked ones
    of its first block (their weights must not underflow against a maximum taken from nothing)."""
    dtype, E, Lq, Lkv, B, H, causal, mshape = case
    rng = np.random.default_rng(hash(case[1:6]) % 2**32)
    D = E // H
    q = rng.standard_normal((E, Lq, B))
    k = rng.standard_normal((E, Lkv, B))
    v = rng.standard_normal((E, Lkv, B))
    mask = rng.random(mshape) < 0.85
    full = mask.reshape(mshape + (1,) * (4 - len(mshape)))
    full[:, 3] = False                                   # keeps nothing
    full[:200, 5] = False                                # first kept key in the seventh 32-key block at the earliest
    full[:, 7] = False
    full[(7 if causal else Lkv - 1), 7] = True           # one key (the last one the causal pattern allows)
    full[:, 9] = False
    full[64:96, 9] = True                                # one block
    # query 130: scores of +-8 sqrt(D) against keys 0..127; keeps only the strongly negative ones
    q[:, 130] = 8.0
    k[:, :64] = 1.0
    k[:, 64:128] = -1.0
    full[:, 130] = False
    full[64:128, 130] = True
    q, k, v = (round_to(a, dtype) for a in (q, k, v))
    dq, dk, dv = (nn.DeviceArray.from_numpy(a, dtype) for a in (q, k, v))
    dm = nn.DeviceArray.from_numpy(mask)
    y, _ = nn.dot_product_attention(dq, dk, dv, mask=(nn.make_causal_mask(dq, dims=2) & dm) if causal else dm, nheads=H,
                                    return_weights=False)
    assert nn.last_attention_kernel() == "flash16"
    slices = (mshape[2] if len(mshape) > 2 else 1) * (mshape[3] if len(mshape) > 3 else 1)
    assert nn.ops._last_workspace == _mask_words_bytes(Lq, Lkv, slices)
    omask = np.broadcast_to(full, (Lkv, Lq, H, B))
    if causal:
        omask = omask & oracle.make_causal_mask(Lq).reshape(Lkv, Lq, 1, 1)
    yr, _ = oracle.nnlib_attention_f32(q, k, v, None, np.ascontiguousarray(omask), H, nthreads=8)
    y = y.to_numpy()
    nan_ref = np.isnan(yr)
    assert nan_ref[:, 3].all() and (nan_ref.sum() == nan_ref[:, 3].size if not causal else True)
    assert np.array_equal(np.isnan(y), nan_ref)
    err = rel_err(np.where(nan_ref, 0, y), np.where(nan_ref, 0, yr))
    assert err <= TOL[dtype], err
    # the query with the far-away scores averages the values of the keys it keeps
    assert np.abs(y[:, 130] - v[:, 64:128].mean(axis=1)).max() <= 2e-2


def test_dense_mask_with_strides_and_without_room_for_the_packed_copy(nn, oracle):
    """The pre-pass reads the mask through its strides (here a mask stored query-major, passed as its transpose), and a
    caller whose workspace cannot hold the packed mask is served by the general kernel with the same result."""
    import ctypes
    import torch
    L = nn._lib
    lib = L.load()
    E, Lq, Lkv, B, H = 256, 384, 640, 2, 2
    rng = np.random.default_rng(11)
    q, k, v = (round_to(rng.standard_normal((E, n, B)), "bf16") for n in (Lq, Lkv, Lkv))
    mask_t = rng.random((Lq, Lkv)) < 0.8                      # [query][key] in column-major order: key stride Lq
    mask_t[:, 0] = True
    tq, tk, tv = (torch.from_numpy(np.ascontiguousarray(a.transpose(2, 1, 0))).cuda().to(torch.bfloat16) for a in (q, k, v))
    tm = torch.from_numpy(np.ascontiguousarray(mask_t.T)).cuda().to(torch.uint8)   # memory order: key slowest
    outs = []
    for with_ws in (True, False):
        out = torch.full((B, Lq, E), float("nan"), device="cuda", dtype=torch.bfloat16)
        d = L.mi_attn_desc()
        d.struct_size = ctypes.sizeof(L.mi_attn_desc)
        d.dtype = d.weights_dtype = L.MI_BF16
        d.E = d.Ev = E
        d.Lq, d.Lkv, d.H, d.B = Lq, Lkv, H, B
        d.q, d.k, d.v, d.out = tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), out.data_ptr()
        d.mask = tm.data_ptr()
        d.mask_strides = (ctypes.c_int64 * 4)(Lq, 1, 0, 0)
        ws = ctypes.c_size_t(0)
        L.check(lib.mi_attention_workspace_size(ctypes.byref(d), ctypes.byref(ws)))
        assert ws.value == _mask_words_bytes(Lq, Lkv, 1)
        if with_ws:
            buf = torch.empty(ws.value, dtype=torch.uint8, device="cuda")
            d.workspace, d.workspace_bytes = buf.data_ptr(), buf.numel()
        L.check(lib.mi_attention_fwd(ctypes.byref(d), None))
        torch.cuda.synchronize()
        outs.append(out.float().cpu().numpy().transpose(2, 1, 0))
    yr, _ = oracle.nnlib_attention_f32(q, k, v, None, np.asfortranarray(mask_t.T), H, nthreads=8)
    for y in outs:
        assert rel_err(y, yr) <= TOL["bf16"]


def test_few_queries_without_a_workspace_fall_back_to_the_pipelined_kernel(nn):
    """mi_attention_fwd with no workspace on a call whose plan is the key-split kernel: served by the software-pipelined
    kernel (which needs none) instead of MI_EWORKSPACE; same result to the 16-bit bound."""
    import ctypes
    import torch
    L = nn._lib
    lib = L.load()
    E, Lq, Lkv, B, H = 512, 256, 4096, 2, 4
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = (torch.randn(E * n * B, device="cuda", generator=g).to(torch.bfloat16) for n in (Lq, Lkv, Lkv))
    outs = []
    for with_ws in (True, False):
        out = torch.full((E * Lq * B,), float("nan"), device="cuda", dtype=torch.bfloat16)
        d = L.mi_attn_desc()
        d.struct_size = ctypes.sizeof(L.mi_attn_desc)
        d.dtype = d.weights_dtype = L.MI_BF16
        d.E = d.Ev = E
        d.Lq, d.Lkv, d.H, d.B = Lq, Lkv, H, B
        d.q, d.k, d.v, d.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
        ws = ctypes.c_size_t(0)
        L.check(lib.mi_attention_workspace_size(ctypes.byref(d), ctypes.byref(ws)))
        assert ws.value > 0
        if with_ws:
            buf = torch.empty(ws.value, dtype=torch.uint8, device="cuda")
            d.workspace, d.workspace_bytes = buf.data_ptr(), buf.numel()
        L.check(lib.mi_attention_fwd(ctypes.byref(d), None))
        torch.cuda.synchronize()
        outs.append(out.float())
    assert not torch.isnan(outs[0]).any() and not torch.isnan(outs[1]).any()
    assert float((outs[0] - outs[1]).abs().max() / outs[0].abs().max()) <= 1e-2


@pytest.mark.parametrize("dtype,E,H,Lkv,B", [("bf16", 512, 4, 1500, 2), ("bf16", 256, 2, 4096, 3), ("f16", 512, 8, 777, 1),
                                             ("f16", 1024, 8, 2048, 2), ("f32", 512, 4, 1500, 2), ("f32", 64, 1, 777, 1)])
@pytest.mark.parametrize("Lq", [2, 3, 4])
@pytest.mark.parametrize("mask", [None, "keys"])
def test_a_few_queries_stream_like_one(nn, oracle, dtype, E, H, Lkv, B, Lq, mask):
    """Two to four queries per batch element against a long context (no weights, no bias, a mask only if it does not
    depend on the query) take the single-query kernels: a wavefront carries 2 or 4 softmax states through one pass over
    K and V (three queries run as four).  Parity per query against the oracle."""
    rng = np.random.default_rng(E + Lkv + Lq)
    q, k, v = (round_to(rng.standard_normal(s), dtype) for s in ((E, Lq, B), (E, Lkv, B), (E, Lkv, B)))
    m = None
    if mask == "keys":      # (Lkv, 1, 1, B): the context lengths / scattered keys of a padded batch
        m = rng.random((Lkv, 1, 1, B)) < 0.8
        m[0] = True
    y, _ = _run(nn, q, k, v, dtype, None, m, H, False, return_weights=False)
    assert nn.last_attention_kernel() == "decode"
    om = None if m is None else np.broadcast_to(m, (Lkv, Lq, 1, B))
    yr, _ = oracle.nnlib_attention_f32(q, k, v, None, om, H, nthreads=8)
    err = np.abs(y - yr).reshape(E, -1).max(axis=0) / np.abs(yr).max()
    assert err.max() <= TOL[dtype], (float(err.max()), int(err.argmax()))


def test_a_few_queries_with_weights_or_a_query_dependent_mask_take_the_tiled_kernel(nn, oracle):
    rng = np.random.default_rng(9)
    _check(nn, oracle, rng, "bf16", 256, 3, 1500, 2, 2, expect="flash16", weights=True)
    _check(nn, oracle, rng, "bf16", 256, 3, 1504, 2, 2, expect="flash16", weights=False, mask_shape=(1504, 3))


def _f64_attention(q, k, v, H, causal=False):
    """Brute force in float64 on the float32 inputs, with q divided by sqrt(D) in float32 as src/attention.jl:118 does."""
    E, Lq, B = q.shape
    Lkv, D = k.shape[1], E // H
    y = np.zeros((v.shape[0], Lq, B))
    a = np.zeros((Lkv, Lq, H, B))
    Dv = v.shape[0] // H
    for b in range(B):
        for h in range(H):
            qs = (q[h * D:(h + 1) * D, :, b] / np.float32(np.sqrt(np.float32(D)))).astype(np.float64)
            s = k[h * D:(h + 1) * D, :, b].astype(np.float64).T @ qs
            if causal:
                s = np.where(np.arange(Lkv)[:, None] <= np.arange(Lq)[None, :], s, -np.inf)
            w = np.exp(s - s.max(axis=0, keepdims=True))
            w /= w.sum(axis=0, keepdims=True)
            a[:, :, h, b] = w
            y[h * Dv:(h + 1) * Dv, :, b] = v[h * Dv:(h + 1) * Dv, :, b].astype(np.float64) @ w
    return y, a


_F32_SCRIPT = """
import sys, numpy as np
sys.path.insert(0, %r)
import nnlib_amd as nn
d = np.load(sys.argv[1])
q, k, v = (nn.DeviceArray.from_numpy(d[n], "f32") for n in "qkv")
y, a = nn.dot_product_attention(q, k, v, nheads=int(d["H"]), mask=(nn.make_causal_mask(q, dims=2) if int(d["causal"]) else None))
np.savez(sys.argv[2], y=y.to_numpy(), a=a.to_numpy())
"""


@pytest.mark.parametrize("E,H,L,causal", [(256, 4, 300, False), (256, 4, 257, True), (256, 2, 200, False), (96, 1, 130, True)],
                         ids=["D64", "D64-causal", "D128", "D96-causal"])
def test_float32_products_through_bf16_planes_keep_float32_accuracy(nn, oracle, tmp_path, E, H, L, causal):
    """Float32 calls run their products as six bf16 matrix instructions per Float32 one (three planes per operand).
    Against float64 on the same inputs the result must be as close as the Float32 matrix instruction's, which a child
    process computes with MI355ATTN_F32_MFMA=1: values spread over 2^+-12 so that every plane carries weight."""
    import os, subprocess, sys
    rng = np.random.default_rng(E + L)
    spread = lambda shape: (rng.standard_normal(shape) * np.exp2(rng.integers(-12, 1, shape))).astype(np.float32)
    q, k, v = spread((E, L, 2)), spread((E, L, 2)), spread((E, L, 2))
    y64, a64 = _f64_attention(q, k, v, H, causal)
    y, a = _run(nn, q, k, v, "f32", nheads=H, causal=causal, weights_dtype="f32")
    assert nn.last_attention_kernel() == "flash32"
    err_y, err_a = np.abs(y - y64).max() / np.abs(y64).max(), np.abs(a - a64).max()
    assert err_y < 5e-6 and err_a < 5e-6, (err_y, err_a)
    # the same call on the Float32 matrix instruction, in a process of its own (the choice is made once per process)
    np.savez(tmp_path / "in.npz", q=q, k=k, v=v, H=H, causal=int(causal))
    env = dict(os.environ, MI355ATTN_F32_MFMA="1")
    pkg = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nnlib.jl_amd")
    subprocess.run([sys.executable, "-c", _F32_SCRIPT % pkg, str(tmp_path / "in.npz"), str(tmp_path / "out.npz")], env=env, check=True, timeout=300)
    ref = np.load(tmp_path / "out.npz")
    err_y2, err_a2 = np.abs(ref["y"] - y64).max() / np.abs(y64).max(), np.abs(ref["a"] - a64).max()
    assert err_y2 < 5e-6 and err_a2 < 5e-6, (err_y2, err_a2)
    assert err_y < 4 * err_y2 + 2e-7 and err_a < 4 * err_a2 + 2e-7, (err_y, err_y2, err_a, err_a2)


def test_float32_products_with_infinite_inputs(nn, oracle):
    """An Inf in k whose q entries are all negative makes that key's logits -Inf, as the Float32 instruction would
    (an Inf goes through the planes with its sign): the key gets no weight and the rest is the call without it.  A NaN
    in v poisons only the outputs that weight it."""
    rng = np.random.default_rng(77)
    E, L = 64, 140
    q = rng.standard_normal((E, L, 1)).astype(np.float32)
    k = rng.standard_normal((E, L, 1)).astype(np.float32)
    v = rng.standard_normal((E, L, 1)).astype(np.float32)
    q[7] = -np.abs(q[7]) - 0.5
    k[7, 33, 0] = np.inf
    y, a = _run(nn, q, k, v, "f32", nheads=1, weights_dtype="f32")
    assert nn.last_attention_kernel() == "flash32"
    assert np.all(a[33, :, 0, 0] == 0) and np.isfinite(y).all() and np.isfinite(a).all()
    keep = np.arange(L) != 33
    yr, ar = oracle.nnlib_attention_f32(q, k[:, keep], v[:, keep], None, None, 1)
    assert rel_err(y, yr) < 1e-5 and np.allclose(a[keep], ar, atol=1e-6)
    v2 = v.copy()
    v2[5, 90, 0] = np.nan
    y2, _ = _run(nn, q, k, v2, "f32", nheads=1, weights_dtype="f32")
    assert np.isnan(y2[5]).all() and np.isfinite(np.delete(y2, 5, axis=0)).all()
