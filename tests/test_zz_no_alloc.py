"""mi_attention_fwd_static: the forward call whose workspace is an array inside the library's device image, for
callers that cannot allocate device memory.  It runs the kernels of mi_attention_fwd, so its results must equal
that entry point's bit for bit.  Every case makes two calls in a row, the second on a smaller input, because all
calls share the one array and it keeps what the previous call left there."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def _desc(L, dtype, E, Lq, Lkv, B, H, q, k, v, out, weights=None, weights_f32=False, mask=None, mask_strides=None,
          bias=None, bias_strides=None, causal=False):
    code = {"f32": L.MI_F32, "f16": L.MI_F16, "bf16": L.MI_BF16}[dtype]
    d = L.mi_attn_desc()
    d.struct_size = ctypes.sizeof(L.mi_attn_desc)
    d.dtype = code
    d.weights_dtype = L.MI_F32 if weights_f32 else code
    d.E = d.Ev = E
    d.Lq, d.Lkv, d.H, d.B = Lq, Lkv, H, B
    d.causal = int(causal)
    d.q, d.k, d.v, d.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    if weights is not None:
        d.weights = weights.data_ptr()
    if mask is not None:
        d.mask = mask.data_ptr()
        d.mask_strides = (ctypes.c_int64 * 4)(*mask_strides)
    if bias is not None:
        d.bias = bias.data_ptr()
        d.bias_strides = (ctypes.c_int64 * 4)(*bias_strides)
    return d


def _both(nn, dtype, E, Lq, Lkv, B, H, seed, *, weights=False, key_mask=False, bias=False, expect_kernel, expect_workspace=True):
    """Runs the call through mi_attention_fwd (caller's workspace) and mi_attention_fwd_static on the same device
    buffers; returns nothing, asserts bit equality of outputs (and weights)."""
    L = nn._lib
    lib = L.load()
    g = torch.Generator(device="cuda").manual_seed(seed)
    t = TORCH[dtype]
    q = torch.randn(E * Lq * B, device="cuda", generator=g).to(t)
    k = torch.randn(E * Lkv * B, device="cuda", generator=g).to(t)
    v = torch.randn(E * Lkv * B, device="cuda", generator=g).to(t)
    mask = mstr = bs = bstr = None
    if key_mask:      # (Lkv, 1, 1, B): context lengths for the even batch elements, scattered keys for the odd ones
        m = torch.ones(B, Lkv, dtype=torch.uint8, device="cuda")
        for b in range(B):
            if b % 2 == 0:
                m[b, Lkv - 37 * (b + 1):] = 0
            else:
                m[b] = (torch.rand(Lkv, device="cuda", generator=g) < 0.7).to(torch.uint8)
                m[b, 0] = 1
        mask, mstr = m.reshape(-1), (1, 0, 0, Lkv)
    if bias:
        bs = (0.5 * torch.randn(Lkv * Lq * H * B, device="cuda", generator=g)).to(t)
        bstr = (1, Lkv, Lkv * Lq, Lkv * Lq * H)
    outs, ws_out = [], []
    for static in (False, True):
        out = torch.full((E * Lq * B,), float("nan"), device="cuda", dtype=t)
        w = torch.full((Lkv * Lq * H * B,), float("nan"), device="cuda", dtype=t) if weights else None
        d = _desc(L, dtype, E, Lq, Lkv, B, H, q, k, v, out, w, mask=mask, mask_strides=mstr, bias=bs, bias_strides=bstr)
        kern, ws = ctypes.c_int32(-1), ctypes.c_size_t(0)
        L.check(lib.mi_attention_plan(ctypes.byref(d), ctypes.byref(kern), ctypes.byref(ws)))
        assert L.KERNEL_NAMES[kern.value] == expect_kernel
        assert (ws.value > 0) == expect_workspace, ws.value
        assert ws.value <= L.MI_ATTN_STATIC_WORKSPACE_BYTES
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        if static:
            d.workspace, d.workspace_bytes = None, 0            # ignored by the static entry point
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            L.check(lib.mi_attention_fwd_static(ctypes.byref(d), stream))
            torch.cuda.synchronize()
            # neither through torch's allocator nor behind it: the driver's count of free device memory is unchanged
            assert torch.cuda.memory_allocated() == before
            assert torch.cuda.mem_get_info()[0] == free_before
        else:
            buf = torch.empty(max(ws.value, 1), dtype=torch.uint8, device="cuda")
            d.workspace, d.workspace_bytes = buf.data_ptr(), buf.numel()
            L.check(lib.mi_attention_fwd(ctypes.byref(d), stream))
        torch.cuda.synchronize()
        outs.append(out)
        ws_out.append(w)
    assert not torch.isnan(outs[0].float()).any()
    assert torch.equal(outs[0].view(torch.int16 if dtype != "f32" else torch.int32), outs[1].view(torch.int16 if dtype != "f32" else torch.int32))
    if weights:
        assert not torch.isnan(ws_out[0].float()).any()
        assert torch.equal(ws_out[0].view(torch.int16 if dtype != "f32" else torch.int32), ws_out[1].view(torch.int16 if dtype != "f32" else torch.int32))


def test_single_query_calls_then_a_smaller_one(nn):
    """Split-kv partials of the single-query kernels (and, with weights, the raw scores)."""
    _both(nn, "bf16", 1024, 1, 8192, 4, 8, 1, expect_kernel="decode")
    _both(nn, "bf16", 512, 1, 1500, 2, 4, 2, expect_kernel="decode")
    _both(nn, "f16", 1024, 1, 4096, 3, 8, 3, weights=True, expect_kernel="decode")
    _both(nn, "f16", 256, 1, 777, 1, 2, 4, weights=True, expect_kernel="decode")
    _both(nn, "f32", 512, 1, 4096, 4, 4, 5, expect_kernel="decode")
    _both(nn, "f32", 256, 1, 1000, 2, 4, 6, expect_kernel="decode")


def test_split_kv_calls_then_a_smaller_one(nn):
    """Few query tiles and many keys: (o, m, l) partials per key piece, merged by a second kernel."""
    _both(nn, "f16", 1024, 256, 8192, 2, 16, 7, bias=True, expect_kernel="flash16")
    _both(nn, "f16", 128, 100, 3000, 1, 2, 8, bias=True, expect_kernel="flash16")
    _both(nn, "f32", 128, 100, 3000, 1, 2, 9, expect_kernel="flash32")
    _both(nn, "f32", 64, 70, 2500, 1, 1, 10, expect_kernel="flash32")


def test_context_length_masks_then_a_smaller_one(nn):
    """Key-padding masks: one measured context length per (head, batch) pair goes through the workspace."""
    _both(nn, "bf16", 256, 300, 1100, 6, 2, 11, key_mask=True, expect_kernel="flash16")
    _both(nn, "bf16", 128, 140, 716, 3, 1, 12, key_mask=True, weights=True, expect_kernel="flash16")


def test_calls_without_a_workspace(nn):
    _both(nn, "bf16", 256, 520, 520, 2, 2, 13, expect_kernel="flash16", expect_workspace=False)
    _both(nn, "f32", 128, 96, 160, 2, 2, 14, weights=True, expect_kernel="flash32", expect_workspace=False)


def test_key_split_plan_too_large_for_the_builtin_workspace_stays_on_the_pipelined_kernel(nn):
    """512 queries against 2048 keys on 32 heads of 128: mi_attention_fwd cuts the keys into 4 pieces and asks for 34 MB of
    partial results, more than the built-in array holds; the entry point without caller workspace runs the same call on
    the software-pipelined kernel, which needs none.  Two different kernels, so the outputs agree to the 16-bit bound,
    not bit for bit; a smaller call follows."""
    L = nn._lib
    lib = L.load()
    for E, Lq, Lkv, B, H, seed in ((4096, 512, 2048, 1, 32, 21), (4096, 300, 2048, 1, 32, 22)):
        g = torch.Generator(device="cuda").manual_seed(seed)
        q, k, v = (torch.randn(E * n * B, device="cuda", generator=g).to(torch.bfloat16) for n in (Lq, Lkv, Lkv))
        outs = []
        for static in (False, True):
            out = torch.full((E * Lq * B,), float("nan"), device="cuda", dtype=torch.bfloat16)
            d = _desc(L, "bf16", E, Lq, Lkv, B, H, q, k, v, out, None)
            ws = ctypes.c_size_t(0)
            L.check(lib.mi_attention_workspace_size(ctypes.byref(d), ctypes.byref(ws)))
            assert (ws.value > L.MI_ATTN_STATIC_WORKSPACE_BYTES) == (Lq == 512)   # the smaller call's partial results fit
            stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            if static:
                torch.cuda.synchronize()
                before = torch.cuda.memory_allocated()
                L.check(lib.mi_attention_fwd_static(ctypes.byref(d), stream))
                assert torch.cuda.memory_allocated() == before
            else:
                buf = torch.empty(ws.value, dtype=torch.uint8, device="cuda")
                d.workspace, d.workspace_bytes = buf.data_ptr(), buf.numel()
                L.check(lib.mi_attention_fwd(ctypes.byref(d), stream))
            torch.cuda.synchronize()
            outs.append(out.float())
        assert not torch.isnan(outs[0]).any() and not torch.isnan(outs[1]).any()
        assert float((outs[0] - outs[1]).abs().max() / outs[0].abs().max()) <= 1e-2


def test_call_beyond_the_builtin_workspace_is_refused(nn):
    L = nn._lib
    lib = L.load()
    E, H, Lkv = 4096, 32, 4096
    B = 8
    while True:       # grow the batch until the plan asks for more than the built-in array holds
        d = L.mi_attn_desc()
        d.struct_size = ctypes.sizeof(L.mi_attn_desc)
        d.dtype = d.weights_dtype = L.MI_BF16
        d.E = d.Ev = E
        d.Lq, d.Lkv, d.H, d.B = 1, Lkv, H, B
        d.q = d.k = d.v = d.out = 0x1000          # planning reads no memory
        ws = ctypes.c_size_t(0)
        L.check(lib.mi_attention_workspace_size(ctypes.byref(d), ctypes.byref(ws)))
        if ws.value > L.MI_ATTN_STATIC_WORKSPACE_BYTES:
            break
        B *= 2
        assert B <= 4096
    q = torch.zeros(E * B, device="cuda", dtype=torch.bfloat16)
    kv = torch.zeros(E * Lkv * B, device="cuda", dtype=torch.bfloat16)
    out = torch.full((E * B,), 7.0, device="cuda", dtype=torch.bfloat16)
    d.q, d.k, d.v, d.out = q.data_ptr(), kv.data_ptr(), kv.data_ptr(), out.data_ptr()
    rc = lib.mi_attention_fwd_static(ctypes.byref(d), None)
    assert rc == L.MI_EWORKSPACE
    assert "built-in" in L.last_error()
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())               # nothing was launched


def test_static_call_inside_a_captured_graph(nn):
    """Stream capture refuses allocation and synchronisation: the static entry point must record cleanly, and every
    replay must reproduce the eager result bit for bit (replayed several times with eager work and synchronisations
    in between).  Split-kv call: partial results go through the built-in workspace and a merge kernel."""
    L = nn._lib
    lib = L.load()
    dtype, E, Lq, Lkv, B, H = "f16", 512, 128, 4096, 2, 8
    t = TORCH[dtype]
    g = torch.Generator(device="cuda").manual_seed(21)
    q = torch.randn(E * Lq * B, device="cuda", generator=g).to(t)
    k = torch.randn(E * Lkv * B, device="cuda", generator=g).to(t)
    v = torch.randn(E * Lkv * B, device="cuda", generator=g).to(t)
    eager = torch.empty(E * Lq * B, device="cuda", dtype=t)
    d = _desc(L, dtype, E, Lq, Lkv, B, H, q, k, v, eager)
    kern, ws = ctypes.c_int32(-1), ctypes.c_size_t(0)
    L.check(lib.mi_attention_plan(ctypes.byref(d), ctypes.byref(kern), ctypes.byref(ws)))
    assert ws.value > 0                       # the call does use scratch memory
    L.check(lib.mi_attention_fwd_static(ctypes.byref(d), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    out = torch.zeros_like(eager)
    dg = _desc(L, dtype, E, Lq, Lkv, B, H, q, k, v, out)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        L.check(lib.mi_attention_fwd_static(ctypes.byref(dg), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    for rep in range(3):
        out.fill_(float("nan"))
        other = (q.float() * (rep + 1)).sum()     # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.isfinite(other)
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), rep
