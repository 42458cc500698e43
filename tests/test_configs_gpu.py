"""The five benchmark configurations at full size through the C ABI.

Inputs come from the library's counter-based generator, exactly as bench.py makes them, and are
copied back to the host for the CPU oracle.  Where the whole job is too large for the oracle to
finish in seconds, a subset of (head, batch) slices is checked and size-independent properties cover
the rest (weight columns sum to 1; a value tensor of ones gives an output of ones; a zero key tensor
gives the mean of the values)."""
import ctypes

import numpy as np
import pytest

import bench
from conftest import rel_err

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def _slices(a, heads, D, b):
    """Rows of the given heads of batch element b from a Julia-shaped (E, L, B) host array."""
    return np.concatenate([a[h * D:(h + 1) * D, :, b:b + 1] for h in heads], axis=0)


def _run(r):
    r.step()
    r._lib.check(r.lib.mi_device_sync())


@pytest.mark.parametrize("key,heads,batches", [("c1", range(8), [0, 3]), ("c2", [0, 7, 15], [0, 7]),
                                               ("c3", [0, 31], [1]), ("c4", [0, 9], [0, 3]), ("c5", [0, 13, 31], [0, 15])])
def test_config_against_oracle(nn, oracle, key, heads, batches):
    w = bench.WORKLOADS[key]
    r = bench.Runner(key)
    _run(r)
    D = w["E"] // w["H"]
    heads = list(heads)
    y = r.out.to_numpy()
    alpha = r.alpha.to_numpy() if r.alpha is not None else None
    q, k, v = r.q.to_numpy(), None, None
    mask = r.mask.to_numpy() if r.mask is not None else None
    if w["causal"]:
        mask = oracle.make_causal_mask(w["Lq"])
    for b in batches:
        kb = r.k.storage[b * w["E"] * w["Lkv"]:(b + 1) * w["E"] * w["Lkv"]].float().cpu().numpy().reshape(w["E"], w["Lkv"], 1, order="F")
        vb = r.v.storage[b * w["E"] * w["Lkv"]:(b + 1) * w["E"] * w["Lkv"]].float().cpu().numpy().reshape(w["E"], w["Lkv"], 1, order="F")
        qs, ks, vs = _slices(q, heads, D, b), _slices(kb, heads, D, 0), _slices(vb, heads, D, 0)
        bias = None
        if r.bias is not None:
            n = w["Lkv"] * w["Lq"]
            bias = np.stack([r.bias.storage[(b * w["H"] + h) * n:(b * w["H"] + h + 1) * n].float().cpu().numpy()
                             .reshape(w["Lkv"], w["Lq"], order="F") for h in heads], axis=2)[..., None]
        yr, ar = oracle.nnlib_attention_f32(qs, ks, vs, bias, mask, len(heads), nthreads=16)
        err = rel_err(_slices(y, heads, D, b), yr)
        assert err <= TOL[w["dtype"]], (key, b, err)
        if alpha is not None:
            a = alpha[:, :, heads, b]
            werr = float(np.abs(a - ar[..., 0]).max())
            assert werr <= TOL[w["dtype"]], (key, b, werr)
    if alpha is not None:
        colsum_err = float(np.abs(alpha.sum(axis=0, dtype=np.float64) - 1).max())
        assert colsum_err <= 1e-5, colsum_err            # every weight column of the whole job
        if w["causal"]:
            upper = np.triu(np.ones((w["Lkv"], w["Lq"]), bool))
            assert np.count_nonzero(alpha[~upper]) == 0
    assert r.kernel == {"c1": "flash32", "c2": "flash32", "c3": "flash16", "c4": "flash16", "c5": "decode"}[key]


@pytest.mark.parametrize("key", ["c3", "c4", "c5"])
def test_config_size_independent_properties(nn, key):
    """Whole job, no oracle: V = 1 must give exactly-normalised output 1 (tests the softmax sums on every
    row); K = 0 with no bias gives uniform weights over the kept keys, i.e. the mean of V."""
    w = bench.WORKLOADS[key]
    r = bench.Runner(key)
    r.v.storage.fill_(1.0)
    _run(r)
    y = r.out.to_numpy()
    assert np.abs(y - 1).max() <= 1e-2
    if key != "c4":
        lib, _lib = r.lib, r._lib
        _lib.check(lib.mi_randn_fill(r.v.ptr, r.v.code, r.v.length, 7, 2, 1.0, None))
        r.k.storage.zero_()
        _run(r)
        y = r.out.to_numpy()
        v = r.v.to_numpy().astype(np.float64)
        if w["causal"]:
            ref = np.cumsum(v, axis=1) / np.arange(1, w["Lkv"] + 1)[None, :, None]
        else:
            ref = np.repeat(v.mean(axis=1, keepdims=True), w["Lq"], axis=1)
        assert rel_err(y, ref) <= 1e-2
