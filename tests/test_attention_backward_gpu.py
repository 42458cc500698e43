"""GPU parity of the attention gradient (and the batched_mul pullback) through the C ABI against the
CPU oracle, on the reference's own gradient-test shapes (test/attention.jl:70-76,
test/ext_amdgpu/attention.jl:1-22) and on shapes that reach every kernel."""
import numpy as np
import pytest

from conftest import rel_err, round_to

pytestmark = pytest.mark.gpu
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def _run(nn, oracle, dtype, E, Ev, Lq, Lkv, batch, H, bias_shape=None, mask_kind=None, with_dalpha=False, flags=0,
         seed=0, scale=1.0, expect=None, pass_y=True, dropout=None, saved=False):
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
    elif mask_kind in ("random_hb", "random_b"):   # a mask plane per (head, batch element) / per batch element
        mask = rng.random((Lkv, Lq, H if mask_kind == "random_hb" else 1) + batch) < 0.8
        mask[0] = True
        dmask = nn.DeviceArray.from_numpy(mask)
    elif mask_kind == "lengths":    # padded batch: context lengths per batch element, plus one scattered pattern
        mask = np.ones((Lkv, 1, 1) + batch, dtype=bool)
        nb = mask.shape[-1]
        for i in range(nb):
            if i % 3 == 1:
                mask[Lkv - min(90, Lkv // 2):, ..., i] = False        # a padded tail
            elif i % 3 == 2:
                mask[..., i] = (rng.random(Lkv) < 0.6).reshape((Lkv, 1, 1) + (1,) * (len(batch) - 1))
                mask[0, ..., i] = True
        dmask = nn.DeviceArray.from_numpy(mask)
    elif mask_kind == "keys":       # key-padding mask: no query dependence, one pattern per batch element
        mask = rng.random((Lkv, 1, 1) + batch) < 0.7
        mask[Lkv // 2, ...] = True
        mask[:70, 0, 0, ..., -1] = False          # the first tile and a bit dropped for the last batch element
        dmask = nn.DeviceArray.from_numpy(mask)
    da = round_to(rng.standard_normal((Lkv, Lq, H) + batch), dtype) if with_dalpha else None
    D = nn.DeviceArray.from_numpy
    dq_, dk_, dv_ = D(q, dtype), D(k, dtype), D(v, dtype)
    dbias_ = None if bias is None else D(bias, dtype)
    y = None
    fdrop, keep_scale = nn.identity, None
    if dropout is not None:
        p, dseed = dropout
        fdrop = nn.Dropout(p, dseed)
        keep_scale = oracle.dropout_keep_mask((Lkv, Lq, H) + batch, p, dseed) / (1.0 - p)
    if pass_y:
        y, _ = nn.dot_product_attention(dq_, dk_, dv_, dbias_, mask=dmask, nheads=H, return_weights=False, fdrop=fdrop,
                                        save_for_backward=saved)
    got = nn.dot_product_attention_grad(D(dy, dtype), dq_, dk_, dv_, dbias_, y=y, mask=dmask, nheads=H,
                                        dalpha=None if da is None else D(da, dtype), fdrop=fdrop, _flags=flags)
    if expect is not None:
        assert nn.last_attention_bwd_kernel() == expect, nn.last_attention_bwd_kernel()
    ref = oracle.attention_bwd_f64(q, k, v, dy, bias, mask, H, da, keep_scale=keep_scale)
    errs = []
    for g, r, name in zip(got, ref, ("dq", "dk", "dv", "dbias")):
        if r is None:
            assert g is None
            continue
        g = g.to_numpy()
        assert g.shape == r.shape, name
        # error against the gradient's scale; a gradient that is identically zero (one key: the weights
        # are constant) is held to an absolute bound instead
        errs.append(float(np.abs(g - r).max() / max(np.abs(r).max(), 0.05)))
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


MFMA_CASES = [
    # dtype, D, H, Lq, Lkv, batch, mask_kind, bias_shape
    ("bf16", 128, 2, 256, 256, (2,), None, None),
    ("bf16", 128, 2, 200, 200, (1,), "causal", None),
    ("f16", 128, 1, 130, 333, (2,), "random", None),
    ("bf16", 64, 3, 257, 257, (2,), "causal", None),
    ("f16", 64, 2, 100, 450, (1, 2), None, None),
    ("bf16", 64, 2, 96, 160, (2,), "random", "full"),
    ("f16", 128, 2, 64, 64, (1,), None, "row"),
    ("bf16", 128, 1, 1, 700, (3,), None, None),
    ("bf16", 64, 1, 500, 1, (1,), None, None),
    # head dims below the 64- / 128-wide tiles (multiples of 8): zero-padded in flight
    ("bf16", 96, 2, 200, 260, (2,), None, None),
    ("f16", 32, 3, 257, 257, (1,), "causal", None),
    ("bf16", 80, 2, 130, 333, (2,), "random", None),
    ("f16", 40, 2, 96, 160, (2,), "random", "full"),
    ("bf16", 112, 1, 300, 300, (1,), "causal", None),
    ("f16", 8, 2, 70, 90, (2,), None, "row"),
    # head dims above 128 up to 256: 256-wide tiles, one workgroup per CU, dV and dK always in separate passes
    ("bf16", 256, 1, 200, 260, (2,), None, None),
    ("f16", 192, 2, 257, 257, (1,), "causal", None),
    ("bf16", 160, 1, 130, 333, (2,), "random", None),
    ("f16", 256, 1, 96, 160, (2,), "random", "full"),
]


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,batch,mask_kind,bias_kind", MFMA_CASES)
def test_mfma_kernels(nn, oracle, dtype, D, H, Lq, Lkv, batch, mask_kind, bias_kind):
    """bf16 / f16 inputs with head dims up to 128 (multiples of 8) take the MFMA kernels when the forward result is passed;
    tile-ragged lengths, causal and random masks, bias."""
    bias_shape = None
    if bias_kind == "full":
        bias_shape = (Lkv, Lq, H) + batch if len(batch) == 1 else None
    elif bias_kind == "row":
        bias_shape = (Lkv, 1)
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, batch, H, bias_shape=bias_shape, mask_kind=mask_kind, seed=Lq + Lkv,
         scale=0.4, expect="flash16")


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,batch,mask_kind,bias_shape,expect", [
    ("f32", 64, 2, 130, 200, (2,), None, (200, 130, 2, 2), "flash32"),
    ("f32", 128, 1, 96, 160, (2,), "random", (160, 96), "flash32"),          # broadcast over heads and batch: summed
    ("bf16", 128, 2, 200, 200, (2,), "causal", (200, 200, 2, 1), "flash16"),
    ("f16", 64, 2, 70, 300, (3,), None, (300, 1, 1, 3), "flash16"),          # one bias value per key and batch element
    # plain (non-atomic) sums: own entries per query, head and batch element ...
    ("bf16", 64, 2, 130, 200, (2,), "random", (200, 130, 2, 2), "flash16"),
    # ... and entries shared by the batch elements, one launch per batch element (enough workgroups per launch)
    ("bf16", 8, 16, 2048, 64, (3,), None, (64, 2048, 16, 1), "flash16"),
    ("f16", 16, 16, 2048, 96, (2,), "random", (96, 2048, 16), "flash16"),
    ("f32", 64, 2, 130, 200, (2,), "random", (200, 130, 2, 2), "flash32"),
    ("f32", 8, 16, 2048, 64, (3,), None, (64, 2048, 16, 1), "flash32"),
])
def test_bias_gradient_from_the_mfma_kernels(nn, oracle, dtype, D, H, Lq, Lkv, batch, mask_kind, bias_shape, expect):
    """The bias gradient is dS summed over the dims the bias broadcasts along; the dQ kernels add it with Float32
    atomics (the reference gets it from the broadcast rule of `.+`, src/attention.jl:129-131)."""
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, batch, H, bias_shape=bias_shape, mask_kind=mask_kind, seed=Lq * 3 + Lkv,
         scale=0.4, expect=expect)


F32_CASES = [
    # D, H, Lq, Lkv, batch, mask_kind, saved statistics
    (64, 2, 200, 200, (2,), "causal", False),
    (64, 2, 130, 333, (1,), None, True),
    (64, 1, 96, 160, (2,), "random", False),
    (128, 2, 257, 257, (1,), "causal", True),
    (128, 1, 100, 450, (2,), None, False),
    (128, 1, 70, 130, (1,), "random", False),
    (64, 3, 1, 300, (2,), None, False),
    # head dims below the tile width (multiples of 4)
    (96, 2, 230, 230, (1,), "causal", True),
    (36, 2, 130, 333, (2,), None, False),
    (4, 3, 70, 90, (2,), "random", False),
    # statistics saved by the forward kernels that run a workgroup per 32 queries: the rows between the last query
    # block and the padded length of the statistics are zeros
    (64, 2, 40, 100, (2,), None, True),
    (64, 1, 70, 70, (1,), "causal", True),
    (32, 2, 33, 300, (1,), None, True),
    # ... and the gradient kernels that run a workgroup per 32 queries / 32 keys (at most 512 such blocks, saved
    # statistics, head dim <= 64): several 128-row chunks, ragged ends, the causal diagonal inside a chunk
    (64, 2, 300, 300, (1,), "causal", True),
    (48, 2, 129, 257, (2,), None, True),
    (64, 8, 128, 128, (4,), None, True),
    (64, 1, 1, 200, (3,), None, True),
    (64, 1, 500, 31, (1,), None, True),
    # the same kernels reading a Bool mask array (no bias), with and without saved statistics
    (64, 2, 100, 200, (2,), "random", True),
    (32, 4, 257, 129, (1,), "random", True),
    (64, 2, 130, 600, (1,), "random", False),
    (64, 8, 32, 32, (80,), None, True),                  # 640 sequences of one block: those kernels at any number of pairs
    (64, 8, 30, 90, (70,), None, True),                  # ... the dQ kernel only
    # more blocks than that: the workgroups of 128 queries / keys with saved statistics
    (64, 4, 128, 128, (40,), None, True),
    (64, 4, 100, 100, (40,), "causal", True),
]


@pytest.mark.parametrize("D,H,Lq,Lkv,batch,mask_kind,saved", F32_CASES)
def test_f32_mfma_kernels(nn, oracle, D, H, Lq, Lkv, batch, mask_kind, saved):
    """Float32 inputs with head dims up to 128 (multiples of 4) take the fp32-MFMA gradient kernels (tolerance 1e-4 of the
    gradient's scale), with and without the statistics saved by the forward call."""
    rng = np.random.default_rng(D + Lq + Lkv)
    E = D * H
    q, k, v, dy = (rng.standard_normal(s).astype(np.float32) * sc for s, sc in
                   (((E, Lq) + batch, 0.4), ((E, Lkv) + batch, 0.4), ((E, Lkv) + batch, 1.0), ((E, Lq) + batch, 1.0)))
    Dv = nn.DeviceArray.from_numpy
    dq_, dk_, dv_, ddy = Dv(q), Dv(k), Dv(v), Dv(dy)
    mask = dmask = None
    if mask_kind == "causal":
        mask, dmask = oracle.make_causal_mask(Lq), nn.make_causal_mask(dq_)
    elif mask_kind == "random":
        mask = rng.random((Lkv, Lq)) < 0.8
        mask[0] = True
        dmask = Dv(mask)
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, mask=dmask, nheads=H, return_weights=False, save_for_backward=saved)
    assert (getattr(y, "saved_stats", None) is not None) == saved
    got = nn.dot_product_attention_grad(ddy, dq_, dk_, dv_, y=y, mask=dmask, nheads=H)
    assert nn.last_attention_bwd_kernel() == "flash32"
    ref = oracle.attention_bwd_f64(q, k, v, dy, None, mask, H)
    for g, r_, name in zip(got[:3], ref[:3], ("dq", "dk", "dv")):
        err = np.abs(g.to_numpy() - r_).max() / max(np.abs(r_).max(), 0.05)
        assert err <= 1e-4, (name, err)


def test_mfma_kernels_with_bias_input_but_no_bias_gradient(nn, oracle):
    """A bias changes the weights the MFMA kernels recompute; its own gradient needs the generic path, so
    here the bias gradient is not requested (C ABI level: dbias = NULL)."""
    import ctypes
    rng = np.random.default_rng(3)
    dtype, E, Lq, Lkv, H, B = "bf16", 128, 70, 200, 2, 2
    q, k, v, dy = (round_to(rng.standard_normal(s) * 0.5, dtype) for s in ((E, Lq, B), (E, Lkv, B), (E, Lkv, B), (E, Lq, B)))
    bias = round_to(rng.standard_normal((Lkv, Lq, H, B)) * 0.5, dtype)
    mask = rng.random((Lkv, Lq)) < 0.8
    mask[0] = True
    D = nn.DeviceArray.from_numpy
    dq_, dk_, dv_, db_, dm_, ddy = D(q, dtype), D(k, dtype), D(v, dtype), D(bias, dtype), D(mask), D(dy, dtype)
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, db_, mask=dm_, nheads=H, return_weights=False)
    L = nn._lib
    d = L.mi_attn_bwd_desc()
    d.struct_size = ctypes.sizeof(L.mi_attn_bwd_desc)
    nn.ops._fill_desc(d.fwd, dq_, dk_, dv_, db_, dm_, H, B, E, E, Lq, Lkv, 0)
    d.fwd.out, d.dout = y.ptr, ddy.ptr
    gq, gk, gv = (nn.DeviceArray.empty(a.dims, dtype) for a in (dq_, dk_, dv_))
    d.dq, d.dk, d.dv = gq.ptr, gk.ptr, gv.ptr
    kern, ws = ctypes.c_int32(-1), ctypes.c_size_t(0)
    L.check(L.load().mi_attention_bwd_plan(ctypes.byref(d), ctypes.byref(kern), ctypes.byref(ws)))
    assert L.KERNEL_NAMES[kern.value] == "flash16"
    wsbuf = nn.DeviceArray.empty((ws.value // 4 + 4,), "f32")
    d.workspace, d.workspace_bytes = wsbuf.ptr, ws.value
    L.check(L.load().mi_attention_bwd(ctypes.byref(d), None))
    ref = oracle.attention_bwd_f64(q, k, v, dy, bias, mask, H)
    for g, r_ in zip((gq, gk, gv), ref):
        assert rel_err(g.to_numpy(), r_) <= 1e-2


@pytest.mark.parametrize("dtype,D,H,L,Lkv,causal", [("bf16", 128, 2, 300, 300, True), ("bf16", 128, 1, 513, 200, False),
                                                    ("f16", 64, 2, 130, 130, True), ("f16", 64, 2, 64, 2500, False)])
def test_statistics_saved_by_the_forward_call(nn, oracle, dtype, D, H, L, Lkv, causal):
    """save_for_backward keeps the softmax row statistics of the forward call (both 16-bit forward
    kernels write them); the gradient then skips its own statistics pass and must not change."""
    rng = np.random.default_rng(L + Lkv)
    E, B = D * H, 2
    q, k, v, dy = (round_to(rng.standard_normal(s) * 0.5, dtype) for s in ((E, L, B), (E, Lkv, B), (E, Lkv, B), (E, L, B)))
    Dv = nn.DeviceArray.from_numpy
    dq_, dk_, dv_, ddy = Dv(q, dtype), Dv(k, dtype), Dv(v, dtype), Dv(dy, dtype)
    mask = nn.make_causal_mask(dq_) if causal else None
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, mask=mask, nheads=H, return_weights=False, save_for_backward=True)
    assert y.saved_stats is not None
    y_plain, _ = nn.dot_product_attention(dq_, dk_, dv_, mask=mask, nheads=H, return_weights=False)
    assert rel_err(y.to_numpy(), y_plain.to_numpy()) < 1e-2          # (the saving call never splits the key range)
    with_stats = nn.dot_product_attention_grad(ddy, dq_, dk_, dv_, y=y, mask=mask, nheads=H)
    assert nn.last_attention_bwd_kernel() == "flash16"
    ref = oracle.attention_bwd_f64(q, k, v, dy, None, oracle.make_causal_mask(L) if causal else None, H)
    for g, r_ in zip(with_stats[:3], ref[:3]):
        assert np.abs(g.to_numpy() - r_).max() / max(np.abs(r_).max(), 0.05) <= 1e-2


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,batch,mask_kind,saved,dropout", [
    ("bf16", 128, 2, 200, 320, (2,), "random", False, None),
    ("f16", 64, 2, 130, 208, (3,), "random_b", True, None),
    ("bf16", 96, 2, 257, 272, (2,), "random_hb", True, None),
    ("f16", 128, 1, 70, 400, (2,), "random", False, (0.25, 77)),
    ("bf16", 32, 3, 300, 64, (1,), "random_hb", False, None),
])
def test_dense_mask_on_the_lean_paths(nn, oracle, dtype, D, H, Lq, Lkv, batch, mask_kind, saved, dropout):
    """A dense Bool mask without bias whose rows start 16-byte aligned: the dQ kernel reads staged mask tiles, the
    dK / dV kernels 64-bit words packed by a small kernel first (one per key and query tile)."""
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, batch, H, mask_kind=mask_kind, expect="flash16", saved=saved, dropout=dropout,
         seed=Lq + Lkv, scale=0.4)


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,B,causal_too,saved,dropout", [
    ("bf16", 128, 2, 200, 332, 4, False, True, None),
    ("f16", 64, 2, 300, 1100, 3, False, True, None),
    ("bf16", 96, 1, 513, 520, 5, False, True, (0.2, 5)),
    ("bf16", 128, 2, 200, 332, 4, False, False, None),      # without saved statistics: the statistics pass walks the context length too
    ("f32", 64, 2, 200, 332, 4, False, True, None),
    ("f32", 96, 1, 300, 520, 3, False, False, None),        # Float32: also without saved statistics
    ("f32", 36, 2, 130, 1100, 5, False, True, None),
    # lengths that are not multiples of 4 (mask rows unaligned): the pairs without a length run the per-element paths
    ("bf16", 128, 2, 200, 333, 4, False, True, None),
    ("f16", 64, 1, 130, 1101, 3, False, False, None),
    ("f32", 64, 2, 130, 333, 3, False, True, None),
    ("bf16", 64, 2, 100, 333, 3, False, True, (0.2, 9)),    # with dropout the unaligned case stays on the per-element paths
])
def test_context_lengths_in_the_gradient(nn, oracle, dtype, D, H, Lq, Lkv, B, causal_too, saved, dropout):
    """Key-padding masks with saved statistics: pairs whose mask keeps a prefix of the keys run the unmasked gradient
    kernels on that many keys (the padding gets zero gradients), the others the key-mask kernels."""
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, (B,), H, mask_kind="lengths", expect="flash32" if dtype == "f32" else "flash16",
         saved=saved, dropout=dropout, seed=Lq + Lkv, scale=0.4)


@pytest.mark.parametrize("dtype,D,expect", [("bf16", 96, "flash16"), ("f32", 64, "flash32"), ("f32", 6, "generic")])
def test_forward_result_is_recomputed_when_missing(nn, oracle, dtype, D, expect):
    """The MFMA gradient kernels need the forward result; a call without `y` runs one forward call first rather
    than falling back to the generic kernels (which still take the shapes nothing else does)."""
    _run(nn, oracle, dtype, 2 * D, 2 * D, 130, 200, (2,), 2, mask_kind="random", pass_y=False, expect=expect, seed=11, scale=0.5)
    _run(nn, oracle, dtype, 2 * D, 2 * D, 150, 150, (1,), 2, mask_kind="causal", pass_y=False, expect=expect, seed=12, scale=0.5,
         dropout=(0.2, 99))
    # a single query: the forward call that recomputes the result is the split-kv kernel, which saves no row statistics
    _run(nn, oracle, dtype, 2 * D, 2 * D, 1, 700, (3,), 2, mask_kind=None, pass_y=False, expect=expect, seed=13, scale=0.5)
    # key-padding mask (the forward call measures context lengths in its workspace) and a bias with its gradient
    _run(nn, oracle, dtype, 2 * D, 2 * D, 140, 330, (3,), 2, mask_kind="lengths", pass_y=False, expect=expect, seed=14, scale=0.5)
    _run(nn, oracle, dtype, 2 * D, 2 * D, 70, 200, (2,), 2, mask_kind=None, bias_shape=(200, 70, 2, 1), pass_y=False, expect=expect,
         seed=15, scale=0.5)


def test_mfma_and_generic_kernels_agree(nn):
    """Same call through both kernel families (the generic one forced by flag)."""
    rng = np.random.default_rng(9)
    D = nn.DeviceArray.from_numpy
    q, k, v, dy = (D(rng.standard_normal(s) * 0.5, "f16") for s in ((256, 150, 2), (256, 310, 2), (256, 310, 2), (256, 150, 2)))
    y, _ = nn.dot_product_attention(q, k, v, nheads=4, return_weights=False)
    a = nn.dot_product_attention_grad(dy, q, k, v, y=y, nheads=4)
    assert nn.last_attention_bwd_kernel() == "flash16"
    b = nn.dot_product_attention_grad(dy, q, k, v, y=y, nheads=4, _flags=nn._lib.MI_ATTN_FORCE_GENERIC)
    assert nn.last_attention_bwd_kernel() == "generic"
    for x, z in zip(a[:3], b[:3]):
        assert rel_err(x.to_numpy(), z.to_numpy()) < 5e-3


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


@pytest.mark.parametrize("dtype,E,H,Lq,Lkv,batch,mask_kind,bias_shape,with_dalpha,saved,expect", [
    ("f32", 12, 2, 9, 7, (2,), None, (7, 9), True, False, "generic"),            # odd head dim, bias gradient, weight cotangent
    ("f32", 18, 3, 6, 6, (1,), "causal", None, False, False, "generic"),
    ("f32", 72, 3, 70, 70, (2,), "causal", None, False, False, "flash32"),       # D = 24 in 64-wide tiles
    ("bf16", 192, 2, 150, 200, (2,), None, None, False, True, "flash16"),        # D = 96 in 128-wide tiles, lean dropout path
    ("f16", 512, 2, 140, 140, (1,), "causal", None, False, False, "flash16"),    # D = 256
    ("bf16", 128, 2, 150, 200, (2,), None, None, False, False, "flash16"),       # D = 64
    ("bf16", 256, 2, 192, 192, (1,), "causal", None, False, True, "flash16"),    # D = 128, statistics from the forward call
    ("f16", 256, 2, 70, 300, (2,), "random", None, False, False, "flash16"),
    ("f16", 128, 2, 130, 130, (1,), "causal", (130, 130, 2, 1), False, False, "flash16"),
    ("f32", 128, 2, 150, 200, (2,), None, None, False, True, "flash32"),         # D = 64
    ("f32", 256, 2, 192, 192, (1,), "causal", None, False, False, "flash32"),    # D = 128
    ("f32", 128, 2, 70, 300, (1,), "random", None, False, False, "flash32"),
    ("f32", 128, 2, 150, 200, (60,), None, None, False, True, "flash32"),        # more than 512 blocks of 32 queries: the per-element kernels
])
def test_gradient_through_fused_dropout(nn, oracle, dtype, E, H, Lq, Lkv, batch, mask_kind, bias_shape, with_dalpha, saved,
                                        expect):
    """fdrop = Dropout(p, seed) in the forward call: the pullback redraws the same keep decisions
    (src/attention.jl:126, src/dropout.jl:38-53; oracle pinned by finite differences with the mask held fixed)."""
    if bias_shape is not None and expect != "generic":
        # a bias input without a bias gradient: the MFMA kernels' bias path
        _bias_input_case(nn, oracle, dtype, E, H, Lq, Lkv, batch, mask_kind, bias_shape, expect)
        return
    _run(nn, oracle, dtype, E, E, Lq, Lkv, batch, H, bias_shape=bias_shape, mask_kind=mask_kind, with_dalpha=with_dalpha,
         expect=expect, dropout=(0.25, 4242), saved=saved, seed=5)


def _bias_input_case(nn, oracle, dtype, E, H, Lq, Lkv, batch, mask_kind, bias_shape, expect):
    rng = np.random.default_rng(17)
    q, k, v, dy = (round_to(rng.standard_normal((E, L) + batch), dtype) for L in (Lq, Lkv, Lkv, Lq))
    bias = round_to(rng.standard_normal(bias_shape) * 0.5, dtype)
    mask = oracle.make_causal_mask(Lq) if mask_kind == "causal" else None
    dmask = nn.make_causal_mask(nn.DeviceArray.zeros((1, Lq))) if mask_kind == "causal" else None
    D = nn.DeviceArray.from_numpy
    fdrop = nn.Dropout(0.25, 777)
    g = oracle.dropout_keep_mask((Lkv, Lq, H) + batch, 0.25, 777) / 0.75
    dq_, dk_, dv_, db_ = D(q, dtype), D(k, dtype), D(v, dtype), D(bias, dtype)
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, db_, mask=dmask, nheads=H, return_weights=False, fdrop=fdrop)
    lib = nn._lib.load()
    import ctypes
    d = nn._lib.mi_attn_bwd_desc()
    d.struct_size = ctypes.sizeof(nn._lib.mi_attn_bwd_desc)
    B = int(np.prod(batch))
    nn.ops._fill_desc(d.fwd, dq_, dk_, dv_, db_, dmask, H, B, E, E, Lq, Lkv, 0, fdrop)
    ddy = D(dy, dtype)
    d.fwd.out, d.dout = y.ptr, ddy.ptr
    outs = [nn.DeviceArray.empty(a.shape, dtype) for a in (q, k, v)]
    d.dq, d.dk, d.dv = (o.ptr for o in outs)
    kern, ws = ctypes.c_int32(0), ctypes.c_size_t(0)
    nn._lib.check(lib.mi_attention_bwd_plan(ctypes.byref(d), ctypes.byref(kern), ctypes.byref(ws)))
    assert nn._lib.KERNEL_NAMES[kern.value] == expect
    wsbuf = nn.DeviceArray.empty((ws.value // 4 + 4,), "f32")
    d.workspace, d.workspace_bytes = wsbuf.ptr, ws.value
    nn._lib.check(lib.mi_attention_bwd(ctypes.byref(d), None))
    ref = oracle.attention_bwd_f64(q, k, v, dy, bias, mask, H, keep_scale=g)
    for o, r in zip(outs, ref[:3]):
        assert np.abs(o.to_numpy() - r).max() / max(np.abs(r).max(), 0.05) <= TOL[dtype]


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,batch,saved,dropout", [
    ("bf16", 128, 2, 192, 256, (2,), False, None),
    ("bf16", 64, 2, 150, 200, (3,), True, None),
    ("f16", 128, 1, 70, 328, (2,), False, (0.25, 99)),
    ("f16", 64, 2, 257, 132, (2,), True, (0.25, 99)),
])
def test_key_padding_mask_on_the_lean_paths(nn, oracle, dtype, D, H, Lq, Lkv, batch, saved, dropout):
    """A mask that does not depend on the query keeps the two-wavefront gradient kernels: one mask byte per key
    (dQ: read per 32-key block; dK / dV: a lane's key is kept or dropped for the whole kernel)."""
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, batch, H, mask_kind="keys", expect="flash16", saved=saved, dropout=dropout,
         seed=9)


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


@pytest.mark.parametrize("dtype,D,H,L,B,saved", [("bf16", 128, 2, 300, 4, True), ("f16", 64, 2, 513, 3, False), ("f32", 64, 2, 200, 3, True),
                                                 ("bf16", 96, 1, 333, 3, True)])
def test_causal_and_padding_mask(nn, oracle, dtype, D, H, L, B, saved):
    """`make_causal_mask(x) .& padding` (a causal language model on a padded batch): the causal half stays symbolic, the
    key-padding array is measured on the device; forward output and gradients against the oracle with the dense product."""
    rng = np.random.default_rng(L + D)
    E = D * H
    q, k, v, dy = (round_to(rng.standard_normal((E, L, B)) * sc, dtype) for sc in (0.4, 0.4, 1.0, 1.0))
    pad = np.ones((L, 1, 1, B), dtype=bool)
    pad[L - 77:, 0, 0, 1] = False                 # a padded tail
    pad[:, 0, 0, 2] = rng.random(L) < 0.7         # scattered (not a context length)
    pad[0, 0, 0, 2] = True
    dense = oracle.make_causal_mask(L)[:, :, None, None] & pad
    Dv = nn.DeviceArray.from_numpy
    dq_, dk_, dv_, ddy = Dv(q, dtype), Dv(k, dtype), Dv(v, dtype), Dv(dy, dtype)
    mask = nn.make_causal_mask(dq_) & Dv(pad)
    assert isinstance(mask, nn.CausalAnd)
    y, a = nn.dot_product_attention(dq_, dk_, dv_, mask=mask, nheads=H, weights_dtype="f32", save_for_backward=saved)
    yr, ar = oracle.nnlib_attention_f32(q, k, v, None, dense, H, nthreads=4)
    assert rel_err(y.to_numpy(), yr) <= TOL[dtype]
    assert np.abs(a.to_numpy() - ar).max() <= TOL[dtype]
    assert np.count_nonzero(a.to_numpy()[~np.broadcast_to(dense, ar.shape)]) == 0
    y2, _ = nn.dot_product_attention(dq_, dk_, dv_, mask=mask, nheads=H, return_weights=False, save_for_backward=saved)
    assert rel_err(y2.to_numpy(), yr) <= TOL[dtype]
    got = nn.dot_product_attention_grad(ddy, dq_, dk_, dv_, y=y2, mask=mask, nheads=H)
    ref = oracle.attention_bwd_f64(q, k, v, dy, None, dense, H)
    for g, r_, name in zip(got[:3], ref[:3], ("dq", "dk", "dv")):
        err = np.abs(g.to_numpy() - r_).max() / max(np.abs(r_).max(), 0.05)
        assert err <= TOL[dtype], (name, err)


@pytest.mark.parametrize("dtype,D,H,Lq,Lkv,B,mask_kind,bias_kind,dropout", [
    ("bf16", 128, 2, 100, 2304, 1, None, None, None),
    ("f16", 64, 2, 130, 4096, 2, "random", None, None),        # dense mask tiles
    ("bf16", 96, 1, 64, 2500, 2, "random", None, None),        # unaligned: per-element path
    ("bf16", 64, 2, 200, 2304, 2, "lengths", None, None),      # context lengths: both kernel sets write their pairs' pieces
    ("f16", 128, 1, 70, 2048, 2, None, "full", None),          # bias and its gradient
    ("bf16", 64, 2, 100, 2304, 1, None, None, (0.2, 3)),
    ("f32", 64, 2, 100, 2304, 1, None, None, None),
    ("f32", 128, 1, 130, 2500, 2, "random", None, None),
    ("f32", 36, 2, 200, 2304, 2, "lengths", None, None),
    ("f32", 64, 1, 70, 2048, 2, None, "full", None),
])
def test_dq_split_over_the_keys(nn, oracle, dtype, D, H, Lq, Lkv, B, mask_kind, bias_kind, dropout):
    """Few queries, many keys, saved statistics: the dQ kernel's key range is cut into pieces whose Float32 partial sums a
    small kernel adds up."""
    bias_shape = (Lkv, Lq, H, B) if bias_kind == "full" else None
    _run(nn, oracle, dtype, D * H, D * H, Lq, Lkv, (B,), H, mask_kind=mask_kind, bias_shape=bias_shape,
         expect="flash32" if dtype == "f32" else "flash16", saved=True, dropout=dropout, seed=Lq + Lkv, scale=0.4)


@pytest.mark.parametrize("dtype,D", [("bf16", 128), ("f16", 64), ("f32", 64)])
@pytest.mark.parametrize("saved", [False, True])
def test_gradient_with_logits_that_climb_along_the_keys(nn, oracle, dtype, D, saved):
    """The forward kernels raise their running maximum lazily (only when a tile outgrows it by 2^8), so the statistics
    they save need not hold the true row maximum; the gradient kernels must get the same weights out of them.  Logits
    that climb by about 5 powers of two per 64-key tile (up to 40 at the last key) keep the saved maximum stale for
    most rows.

    Bounds.  Float32: 1e-4.  16-bit, dk and dv: 1e-2 when the gradient call computes the statistics itself.  With the
    statistics of the software-pipelined forward kernel the bound is 2e-2: that kernel multiplies q by log2(e)/sqrt(D)
    and rounds the product to the 16-bit type before QK^T (as the reference rounds q / sqrt(D), src/attention.jl:118),
    the gradient kernels scale the Float32 product instead, and the two sets of logits differ by up to
    |logit| * 2^-9 (bf16), which at logits of 40 powers of two is a per cent of a weight.  dq is a sum over keys of
    terms that cancel (each row of dS sums to zero and k is dominated by the ramp), so 16-bit rounding of dS shows
    in it: 3e-2."""
    rng = np.random.default_rng(5)
    H, L, B = 2, 512, 2
    E = D * H
    ramp = 5.0 * np.log(2.0) * np.arange(L) / 64.0
    q = round_to(rng.uniform(0.5, 1.5, (E, L, B)), dtype)
    k = round_to((ramp / np.sqrt(D))[None, :, None] + 0.3 * rng.standard_normal((E, L, B)), dtype)
    v, dy = (round_to(rng.standard_normal((E, L, B)), dtype) for _ in range(2))
    Dv = nn.DeviceArray.from_numpy
    dq_, dk_, dv_, ddy = Dv(q, dtype), Dv(k, dtype), Dv(v, dtype), Dv(dy, dtype)
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, nheads=H, return_weights=False, save_for_backward=saved)
    assert (getattr(y, "saved_stats", None) is not None) == saved
    got = nn.dot_product_attention_grad(ddy, dq_, dk_, dv_, y=y, nheads=H)
    assert nn.last_attention_bwd_kernel() == ("flash32" if dtype == "f32" else "flash16")
    ref = oracle.attention_bwd_f64(q, k, v, dy, None, None, H)
    if dtype == "f32":
        tols = (1e-4, 1e-4, 1e-4)
    else:
        tols = (3e-2, 2e-2, 2e-2) if saved else (3e-2, 1e-2, 1e-2)
    for g, r_, tol in zip(got[:3], ref[:3], tols):
        assert np.abs(g.to_numpy() - r_).max() / max(np.abs(r_).max(), 0.05) <= tol


_F32_GRAD_SCRIPT = """
import sys, numpy as np
sys.path.insert(0, %r)
import nnlib_amd as nn
d = np.load(sys.argv[1])
q, k, v, dy = (nn.DeviceArray.from_numpy(d[n], "f32") for n in ("q", "k", "v", "dy"))
mask = nn.make_causal_mask(q, dims=2) if int(d["causal"]) else None
y, _ = nn.dot_product_attention(q, k, v, nheads=int(d["H"]), mask=mask, return_weights=False, save_for_backward=bool(d["saved"]))
g = nn.dot_product_attention_grad(dy, q, k, v, y=y, mask=mask, nheads=int(d["H"]))
assert nn.last_attention_bwd_kernel() == "flash32"
np.savez(sys.argv[2], dq=g[0].to_numpy(), dk=g[1].to_numpy(), dv=g[2].to_numpy())
"""


@pytest.mark.parametrize("E,H,Lq,Lkv,causal,saved", [(256, 4, 300, 300, False, True), (256, 4, 257, 257, True, False),
                                                     (256, 2, 200, 330, False, False), (96, 1, 130, 130, True, True)],
                         ids=["D64-saved", "D64-causal", "D128-cross", "D96-causal-saved"])
def test_float32_gradient_through_bf16_planes_keeps_float32_accuracy(nn, oracle, tmp_path, E, H, Lq, Lkv, causal, saved):
    """Float32 gradient calls without bias / mask arrays run their products as six bf16 matrix instructions per Float32
    one (three planes per operand).  Against float64 on the same inputs every gradient must be as close as the Float32
    matrix instruction's, which a child process computes with MI355ATTN_F32_MFMA=1: values spread over 2^+-12 so that
    every plane carries weight."""
    import os, subprocess, sys
    rng = np.random.default_rng(E + Lq)
    spread = lambda shape: (rng.standard_normal(shape) * np.exp2(rng.integers(-12, 1, shape))).astype(np.float32)
    q, k, v, dy = spread((E, Lq, 2)), spread((E, Lkv, 2)), spread((E, Lkv, 2)), spread((E, Lq, 2))
    ref = oracle.attention_bwd_f64(q, k, v, dy, None, oracle.make_causal_mask(Lq) if causal else None, H, None)
    D = nn.DeviceArray.from_numpy
    dq_, dk_, dv_ = D(q, "f32"), D(k, "f32"), D(v, "f32")
    mask = nn.make_causal_mask(dq_, dims=2) if causal else None
    y, _ = nn.dot_product_attention(dq_, dk_, dv_, nheads=H, mask=mask, return_weights=False, save_for_backward=saved)
    got = nn.dot_product_attention_grad(D(dy, "f32"), dq_, dk_, dv_, y=y, mask=mask, nheads=H)
    assert nn.last_attention_bwd_kernel() == "flash32"
    # the same call on the Float32 matrix instruction, in a process of its own (the choice is made once per process)
    np.savez(tmp_path / "in.npz", q=q, k=k, v=v, dy=dy, H=H, causal=int(causal), saved=int(saved))
    env = dict(os.environ, MI355ATTN_F32_MFMA="1")
    pkg = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "nnlib.jl_amd")
    subprocess.run([sys.executable, "-c", _F32_GRAD_SCRIPT % pkg, str(tmp_path / "in.npz"), str(tmp_path / "out.npz")], env=env, check=True,
                   timeout=300)
    exact = np.load(tmp_path / "out.npz")
    for g, r, name in zip(got, ref, ("dq", "dk", "dv")):
        scale = np.abs(r).max()
        err, err_exact = np.abs(g.to_numpy() - r).max() / scale, np.abs(exact[name] - r).max() / scale
        print(name, err, err_exact)
        assert err < 5e-6 and err_exact < 5e-6, (name, err, err_exact)
        assert err < 4 * err_exact + 2e-7, (name, err, err_exact)


@pytest.mark.parametrize("saved", [False, True], ids=["own-stats", "saved-stats"])
@pytest.mark.parametrize("mask_kind,Lq,Lkv", [(None, 300, 330), ("causal", 300, 300), ("lengths", 257, 300), ("causal", 512, 512)],
                         ids=["cross", "causal", "lengths", "causal-512"])
def test_float32_gradient_with_256_query_workgroups(nn, oracle, mask_kind, Lq, Lkv, saved):
    """With enough (query tile, head, batch) work the Float32 dQ kernel runs 256 queries per workgroup on eight
    wavefronts (head dim 64 and below, no bias / mask arrays): query counts that end inside the first or the second
    half of the last workgroup, whose rows reach past the padded statistics planes."""
    _run(nn, oracle, "f32", 512, 512, Lq, Lkv, (16,), 8, mask_kind=mask_kind, saved=saved, scale=0.5, seed=Lq, expect="flash32")
    _run(nn, oracle, "f32", 256, 256, Lq, Lkv, (16,), 8, mask_kind=mask_kind, saved=saved, scale=0.5, seed=Lq + 1, expect="flash32")


@pytest.mark.parametrize("dtype,D,Dv", [("bf16", 128, 64), ("bf16", 64, 128), ("f16", 40, 96), ("f16", 256, 64), ("f32", 32, 64), ("f32", 128, 36)])
@pytest.mark.parametrize("mask_kind,saved", [(None, True), ("causal", False), ("random", True)])
def test_different_head_dims_for_qk_and_v(nn, oracle, dtype, D, Dv, mask_kind, saved):
    """q / k and v may have different head dims (src/attention.jl:55-78 only asks for divisibility by nheads and equal
    q / k dims).  The MFMA gradient kernels take one head dim: the library zero-pads the narrower side in its workspace
    and drops the padded gradient columns, and the logits keep the scale of the q / k head dim."""
    H = 2
    Lq = 150
    Lkv = Lq if mask_kind == "causal" else 210
    _run(nn, oracle, dtype, D * H, Dv * H, Lq, Lkv, (2,), H, mask_kind=mask_kind, saved=saved, scale=0.7, seed=D + Dv,
         expect="flash32" if dtype == "f32" else "flash16")
