"""Dropout of the attention weights (fdrop = dropout(., p), src/attention.jl:126 with src/dropout.jl:38-53):
the standalone kernel and the copy fused into the attention kernels, against the CPU oracle combined
with a numpy restatement of the library's published keep-decision stream."""
import numpy as np
import pytest

from conftest import rel_err, round_to

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("p", [0.0, 0.3, 0.5, 1.0])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_standalone_dropout_matches_the_published_stream(nn, oracle, p, dtype):
    rng = np.random.default_rng(0)
    x = round_to(rng.standard_normal((37, 11, 3)) + 3.0, dtype)          # no zeros in x
    y = nn.dropout(nn.DeviceArray.from_numpy(x, dtype), p, seed=42).to_numpy()
    keep = oracle.dropout_keep_mask(x.shape, p, 42)
    assert np.array_equal(y != 0, keep)
    scale = 0.0 if p == 1.0 else 1.0 / (1.0 - np.float32(p))
    assert np.allclose(y, np.where(keep, x * scale, 0), rtol=1e-2 if dtype == "bf16" else 1e-6)
    # another seed gives another mask; the kept fraction is 1 - p (docstring example of src/dropout.jl:16-18)
    big = nn.dropout(nn.DeviceArray.from_numpy(np.ones((10000, 5), dtype=np.float32)), p, seed=7).to_numpy()
    assert abs(big.mean() - (0.0 if p == 1.0 else 1.0)) < 0.03


def test_reference_statistical_test(nn):
    """test/attention.jl:54-59 and test/ext_amdgpu/attention.jl:36-42: about half the weights survive p = 0.5."""
    rng = np.random.default_rng(1)
    q = nn.DeviceArray.from_numpy(rng.random((10, 10, 10)).astype(np.float32))
    for fdrop in (nn.Dropout(0.5, seed=3), lambda a: nn.dropout(a, 0.5, seed=3)):
        y, alpha = nn.dot_product_attention(q, q, q, nheads=2, fdrop=fdrop)
        assert 0.6 > (alpha.to_numpy() > 0).mean() > 0.4


CASES = [
    # dtype, E, Lq, Lkv, B, H, causal, weights, expected kernel
    ("f32", 30, 7, 9, 2, 3, False, True, "generic"),
    ("f32", 128, 96, 160, 2, 2, False, True, "flash32"),
    ("f32", 128, 100, 100, 1, 2, True, False, "flash32"),
    ("f32", 128, 150, 100, 2, 2, False, True, "flash32"),       # at most 128 keys with the weights returned: the resident kernel
    ("f32", 96, 128, 128, 1, 2, True, True, "flash32"),
    ("bf16", 128, 70, 200, 2, 2, False, False, "flash16"),
    ("bf16", 256, 130, 130, 2, 2, True, True, "flash16"),
    ("f16", 128, 64, 4096, 1, 2, False, False, "flash16"),      # few query tiles, long keys: split-kv + merge
    ("bf16", 256, 300, 300, 1, 2, True, False, "flash16"),      # head dim 128, no weights, runs of four keys: the pipelined kernel
    ("f16", 256, 520, 1300, 1, 2, False, False, "flash16"),     # its unrolled steady loop (more than four key tiles)
    ("bf16", 128, 700, 700, 2, 2, True, False, "flash16"),      # head dim 64, causal, steady loop and diagonal steps
    ("bf16", 256, 100, 301, 1, 2, False, False, "flash16"),     # key count not a multiple of 4: the general kernel
    ("bf16", 512, 1, 1500, 2, 4, False, False, "decode"),       # one query: the streaming kernels, hashes under the K / V stream
    ("f16", 256, 3, 2048, 2, 2, False, False, "decode"),        # a few queries carried through one stream
    ("bf16", 512, 1, 1501, 2, 4, False, False, "flash16"),      # one query, key count not a multiple of 4
]


@pytest.mark.parametrize("dtype,E,Lq,Lkv,B,H,causal,weights,expect", CASES)
def test_fused_dropout_against_oracle(nn, oracle, dtype, E, Lq, Lkv, B, H, causal, weights, expect):
    rng = np.random.default_rng(E + Lq + Lkv)
    p, seed = 0.25, 2024
    q = round_to(rng.standard_normal((E, Lq, B)) * 0.5, dtype)
    k = round_to(rng.standard_normal((E, Lkv, B)) * 0.5, dtype)
    v = round_to(rng.standard_normal((E, Lkv, B)), dtype)
    D = nn.DeviceArray.from_numpy
    dq_, dk_, dv_ = D(q, dtype), D(k, dtype), D(v, dtype)
    mask = nn.make_causal_mask(dq_) if causal else None
    y, a = nn.dot_product_attention(dq_, dk_, dv_, mask=mask, nheads=H, fdrop=nn.Dropout(p, seed), return_weights=weights,
                                    weights_dtype="f32")
    assert nn.last_attention_kernel() == expect
    _, a_ref = oracle.attention_f64(q, k, v, None, oracle.make_causal_mask(Lq) if causal else None, H)
    keep = oracle.dropout_keep_mask(a_ref.shape, p, seed)
    a_ref = np.where(keep, a_ref / (1.0 - np.float32(p)), 0.0)            # alpha = fdrop(softmax(...))
    Dh = E // H
    y_ref = np.einsum("jihb,dhjb->dhib", a_ref, v.reshape(Dh, H, Lkv, B, order="F")).reshape(E, Lq, B, order="F")
    assert rel_err(y.to_numpy(), y_ref) <= (1e-4 if dtype == "f32" else 1e-2)
    if weights:
        an = a.to_numpy()
        assert np.array_equal(an != 0, a_ref != 0)                        # returned weights are post-dropout
        assert np.abs(an - a_ref).max() <= (1e-5 if dtype == "f32" else 1e-2)
    # the unfused route (scores -> standalone dropout -> batched product) takes the same decisions
    y2, a2 = nn.dot_product_attention(dq_, dk_, dv_, mask=mask, nheads=H, fdrop=lambda w: nn.dropout(w, p, seed=seed))
    assert rel_err(y2.to_numpy(), y_ref) <= (1e-4 if dtype == "f32" else 2e-2)
    assert np.array_equal(a2.to_numpy() != 0, a_ref != 0)


def test_scores_with_fused_dropout_and_edge_probabilities(nn):
    rng = np.random.default_rng(5)
    q = nn.DeviceArray.from_numpy(rng.random((4, 2, 3, 1)).astype(np.float32))
    a0 = nn.dot_product_attention_scores(q, q).to_numpy()
    assert np.array_equal(nn.dot_product_attention_scores(q, q, fdrop=nn.Dropout(0.0)).to_numpy(), a0)
    assert np.all(nn.dot_product_attention_scores(q, q, fdrop=nn.Dropout(1.0)).to_numpy() == 0)
    a = nn.dot_product_attention_scores(q, q, fdrop=nn.Dropout(0.5, seed=1)).to_numpy()
    assert np.all((a == 0) | np.isclose(a, 2 * a0))
    with pytest.raises(nn.ArgumentError, match="probability"):
        nn.Dropout(1.5)
    with pytest.raises(nn.ArgumentError, match="probability"):
        nn.dropout(q, -0.1)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape,dims", [((6, 5), 1), ((6, 5), 2), ((4, 3, 5), (1, 3)), ((4, 3, 5), 2), ((3, 4, 2, 5), (2, 4)),
                                        ((300, 70), 1), ((7,), 1), ((4, 3), (1, 2))])
def test_dropout_along_dims(nn, oracle, dtype, shape, dims):
    """dropout(x, p; dims) (src/dropout.jl:38-53): the random array has the extent of x along dims and 1 elsewhere,
    so slices along the other dimensions share their decisions (the doctest: dims = 1 zeroes whole rows)."""
    rng = np.random.default_rng(3)
    x = round_to(rng.standard_normal(shape) + 3.0, dtype)
    p, seed = 0.4, 11
    got = nn.dropout(nn.DeviceArray.from_numpy(x, dtype), p, seed=seed, dims=dims).to_numpy()
    ds = (dims,) if isinstance(dims, int) else dims
    mshape = tuple(n if d + 1 in ds else 1 for d, n in enumerate(shape))
    keep = oracle.dropout_keep_mask(mshape, p, seed)
    ref = np.where(np.broadcast_to(keep, shape), x / (1 - p), 0.0)
    assert np.array_equal(got == 0, ~np.broadcast_to(keep, shape))
    assert np.abs(got - ref).max() <= (1e-6 if dtype == "f32" else 2e-2) * np.abs(ref).max()
    if len(ds) == len(shape):     # every dimension owns its decisions: the same as dims = :
        assert np.array_equal(got, nn.dropout(nn.DeviceArray.from_numpy(x, dtype), p, seed=seed).to_numpy())


@pytest.mark.parametrize("dtype,E,H,Lq,Lkv", [("bf16", 256, 2, 300, 520), ("f16", 128, 2, 140, 332)])
def test_fused_dropout_with_context_lengths(nn, oracle, dtype, E, H, Lq, Lkv):
    """A key-padding mask that keeps a prefix of the keys (a context length per batch element) together with dropout:
    the pairs with a length run the kernels without mask code on that many keys, and the keep decisions are still
    those of the weight's position in the full (Lkv, Lq, H, B) array."""
    rng = np.random.default_rng(E + Lq)
    B, p, seed = 3, 0.2, 77
    q = round_to(rng.standard_normal((E, Lq, B)) * 0.5, dtype)
    k = round_to(rng.standard_normal((E, Lkv, B)) * 0.5, dtype)
    v = round_to(rng.standard_normal((E, Lkv, B)), dtype)
    lens = [Lkv, Lkv - 37, 64]
    mask = np.zeros((Lkv, 1, 1, B), dtype=bool)
    for b, n in enumerate(lens):
        mask[:n, 0, 0, b] = True
    D = nn.DeviceArray.from_numpy
    y, _ = nn.dot_product_attention(D(q, dtype), D(k, dtype), D(v, dtype), mask=D(mask), nheads=H, fdrop=nn.Dropout(p, seed),
                                    return_weights=False)
    assert nn.last_attention_kernel() == "flash16"
    _, a_ref = oracle.attention_f64(q, k, v, None, np.broadcast_to(mask, (Lkv, Lq, H, B)).copy(), H)
    keep = oracle.dropout_keep_mask(a_ref.shape, p, seed)
    a_ref = np.where(keep, a_ref / (1.0 - np.float32(p)), 0.0)
    Dh = E // H
    y_ref = np.einsum("jihb,dhjb->dhib", a_ref, v.reshape(Dh, H, Lkv, B, order="F")).reshape(E, Lq, B, order="F")
    assert rel_err(y.to_numpy(), y_ref) <= 1e-2
