"""The C ABI without a GPU: the library loads, exports what include/mi355attn.h declares, and its
host-side validation returns the documented status codes."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi355attn.h")


@pytest.fixture(scope="module")
def L():
    from nnlib_amd import _lib
    return _lib


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", src)))


def test_header_symbols_are_exported_and_bound(L):
    names = _declared_functions()
    assert len(names) >= 25
    lib = ctypes.CDLL(L.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(L.SIGNATURES) == names, "python binding and header disagree"


def test_struct_layout_matches_header(L):
    # 6 x int32, 6 x int64, 6 pointers, 4 + 4 strides, workspace pointer + size, dropout (float, pad, u64), stats
    assert ctypes.sizeof(L.mi_attn_desc) == 6 * 4 + 6 * 8 + 5 * 8 + 8 + 32 + 8 + 32 + 8 + 8 + 16 + 8
    assert ctypes.sizeof(L.mi_attn_bwd_desc) == 8 + ctypes.sizeof(L.mi_attn_desc) + 8 * 8
    assert L.load().mi_version() == 100


def _desc(L, **kw):
    d = L.mi_attn_desc()
    d.struct_size = ctypes.sizeof(L.mi_attn_desc)
    d.dtype, d.weights_dtype = L.MI_F32, L.MI_F32
    d.E = d.Ev = 8
    d.Lq, d.Lkv, d.H, d.B = 3, 4, 2, 1
    d.q = d.k = d.v = d.out = 0x1000          # never dereferenced by the planner
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def _plan(L, d):
    kern, ws = ctypes.c_int32(-1), ctypes.c_size_t(0)
    rc = L.load().mi_attention_plan(ctypes.byref(d), ctypes.byref(kern), ctypes.byref(ws))
    return rc, kern.value, ws.value


def test_plan_validation_status_codes(L):
    assert _plan(L, _desc(L))[0] == L.MI_OK
    assert _plan(L, _desc(L, H=3))[0] == L.MI_ESHAPE                 # src/attention.jl:55
    assert "divisible" in L.last_error()
    assert _plan(L, _desc(L, H=0))[0] == L.MI_ESHAPE
    assert _plan(L, _desc(L, dtype=7))[0] == L.MI_EDTYPE
    assert _plan(L, _desc(L, struct_size=12))[0] == L.MI_EINVAL
    assert _plan(L, _desc(L, causal=1))[0] == L.MI_ESHAPE            # Lq != Lkv
    assert _plan(L, _desc(L, causal=1, Lq=4))[0] == L.MI_OK
    assert _plan(L, _desc(L, out=None))[0] == L.MI_EINVAL            # nothing to compute
    assert _plan(L, _desc(L, out=None, weights=0x1000))[0] == L.MI_OK
    assert _plan(L, _desc(L, weights=0x1000, dtype=L.MI_F16, weights_dtype=L.MI_BF16))[0] == L.MI_EDTYPE
    assert _plan(L, _desc(L, q=None))[0] == L.MI_EINVAL
    assert L.load().mi_attention_plan(None, None, None) == L.MI_EINVAL
    with pytest.raises(L.ArgumentError):
        L.check(L.MI_ESHAPE)
    with pytest.raises(L.DimensionMismatch):
        L.check(L.MI_ESHAPE, L.DimensionMismatch)


def test_plan_kernel_selection(L):
    K = L.KERNEL_NAMES
    big = dict(E=4096, Ev=4096, H=32, Lq=4096, Lkv=4096, B=2)
    assert K[_plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, **big))[1]] == "flash16"
    assert K[_plan(L, _desc(L, **big))[1]] == "flash32"
    assert K[_plan(L, _desc(L, **big, flags=L.MI_ATTN_FORCE_GENERIC))[1]] == "generic"
    assert K[_plan(L, _desc(L))[1]] == "flash32"                     # head dim 4: zero-padded into the 64-wide tiles
    assert K[_plan(L, _desc(L, E=12, Ev=12))[1]] == "generic"        # head dim 6: rows are not whole 16-byte chunks
    assert K[_plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, **dict(big, E=3072, Ev=2560)))[1]] == "flash16"   # 96 / 80
    assert K[_plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, **dict(big, E=3200, Ev=3200)))[1]] == "generic"   # 100
    assert K[_plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, **dict(big, E=8192, Ev=6144)))[1]] == "flash16"   # 256 / 192
    assert K[_plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, **dict(big, E=8448, Ev=8448)))[1]] == "generic"   # 264
    rc, kern, ws = _plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, E=4096, Ev=4096, H=32, Lq=1,
                                  Lkv=32768, B=16))
    assert rc == L.MI_OK and K[kern] == "decode" and ws > 0
    # misaligned base pointer: the vector kernels are not eligible
    assert K[_plan(L, _desc(L, dtype=L.MI_BF16, weights_dtype=L.MI_BF16, **dict(big, q=0x1002)))[1]] == "generic"


def test_plan_workspace_for_key_padding_masks(L):
    """A mask without bias that does not depend on the query is measured on the device first (context lengths, one
    Int32 per (head, batch) pair): the planner asks for that buffer, for 16-bit and Float32 calls, forward and gradient."""
    big = dict(E=4096, Ev=4096, H=32, Lq=4096, Lkv=4096, B=2)
    strides = (ctypes.c_int64 * 4)(1, 0, 0, 4096)                    # (Lkv, 1, 1, B)
    lens_bytes = 32 * 2 * 4
    for dt in (L.MI_BF16, L.MI_F32):
        d = _desc(L, dtype=dt, weights_dtype=dt, mask=0x2000, **big)
        d.mask_strides = strides
        rc, kern, ws = _plan(L, d)
        assert rc == L.MI_OK and ws == lens_bytes, (dt, ws)
        dense = _desc(L, dtype=dt, weights_dtype=dt, mask=0x2000, **big)
        dense.mask_strides = (ctypes.c_int64 * 4)(1, 4096, 0, 0)     # depends on the query: no lengths
        # 16-bit calls pack it for the software-pipelined kernel: 16 bytes per query and group of 128 keys
        assert _plan(L, dense)[2] == (32 * 4096 * 16 if dt == L.MI_BF16 else 0)
        b = L.mi_attn_bwd_desc()
        b.struct_size = ctypes.sizeof(L.mi_attn_bwd_desc)
        b.fwd = d
        b.dout = b.dq = b.dk = b.dv = 0x3000
        kern, ws = ctypes.c_int32(-1), ctypes.c_size_t(0)
        assert L.load().mi_attention_bwd_plan(ctypes.byref(b), ctypes.byref(kern), ctypes.byref(ws)) == L.MI_OK
        stats_bytes = 4 * 3 * 2 * 32 * 4096
        assert ws.value == stats_bytes + lens_bytes, (dt, ws.value)   # statistics planes (none saved here), then the lengths


def test_host_side_argument_checks_of_other_entry_points(L):
    lib = L.load()
    assert lib.mi_softmax_dim1(9, None, None, 4, 4, None) == L.MI_EDTYPE
    assert lib.mi_softmax_dim1(L.MI_F32, None, None, -1, 4, None) == L.MI_EINVAL
    assert lib.mi_softmax_dim1(L.MI_F32, None, None, 0, 4, None) == L.MI_OK       # empty: nothing to do
    assert lib.mi_softmax_dim1(L.MI_F32, None, None, 4, 4, None) == L.MI_EINVAL   # null pointers
    g = lambda *a: lib.mi_batched_gemm(*a)
    assert g(L.MI_F32, b"X", b"N", 2, 2, 2, 1.0, 1, 2, 4, 1, 2, 4, 0.0, 1, 2, 4, 1, None) == L.MI_EINVAL
    assert g(L.MI_F32, b"N", b"N", 2, 2, 2, 1.0, 1, 1, 4, 1, 2, 4, 0.0, 1, 2, 4, 1, None) == L.MI_ESHAPE  # lda < m
    assert g(L.MI_F32, b"N", b"N", -2, 2, 2, 1.0, 1, 2, 4, 1, 2, 4, 0.0, 1, 2, 4, 1, None) == L.MI_ESHAPE
    assert g(L.MI_F32, b"N", b"N", 2, 2, 2, 1.0, 1, 2, 4, 1, 2, 4, 0.0, 1, 2, 0, 3, None) == L.MI_ESHAPE   # C broadcast
    assert g(L.MI_F32, b"N", b"N", 0, 2, 2, 1.0, None, 1, 0, None, 2, 0, 0.0, None, 1, 0, 1, None) == L.MI_OK
    assert g(5, b"N", b"N", 2, 2, 2, 1.0, 1, 2, 4, 1, 2, 4, 0.0, 1, 2, 4, 1, None) == L.MI_EDTYPE
    assert lib.mi_randn_fill(None, L.MI_F32, 4, 1, 0, 1.0, None) == L.MI_EINVAL
    assert lib.mi_randn_fill(None, L.MI_F32, 0, 1, 0, 1.0, None) == L.MI_OK
    assert lib.mi_make_causal_mask(None, 4, None) == L.MI_EINVAL
    assert lib.mi_event_elapsed_ms(None, None, None) == L.MI_EINVAL
    assert lib.mi_malloc(None, 16) == L.MI_EINVAL
    assert lib.mi_free(None) == L.MI_OK


def test_host_mirror_shape_errors_without_gpu(L):
    """The Python mirror raises the reference's exception types before any device work."""
    import numpy as np
    import torch
    from nnlib_amd import DeviceArray, dot_product_attention, batched_mul, ArgumentError, DimensionMismatch

    def fake(*dims, dtype="f32"):
        return DeviceArray(torch.empty(1), dims, dtype)      # CPU storage: never reaches a kernel

    with pytest.raises(ArgumentError, match="divisible"):
        dot_product_attention(fake(6, 3, 1), fake(6, 4, 1), fake(6, 4, 1), nheads=4)
    with pytest.raises(ArgumentError, match="Batch dimensions"):
        dot_product_attention(fake(6, 3, 2), fake(6, 4, 1), fake(6, 4, 1))
    with pytest.raises(ArgumentError, match="query and key"):
        dot_product_attention(fake(6, 3, 1), fake(4, 4, 1), fake(6, 4, 1))
    with pytest.raises(ArgumentError, match="key and value"):
        dot_product_attention(fake(6, 3, 1), fake(6, 4, 1), fake(6, 5, 1))
    with pytest.raises(DimensionMismatch, match="batch size mismatch"):      # test/batchedmul.jl:76-78
        batched_mul(fake(2, 2, 2), fake(2, 2, 10))


def test_promote_type_table():
    """Element type of batched_mul(A, B): Julia's promote_type for the pairs test/batchedmul.jl:41-73 exercises."""
    from nnlib_amd.ops import promote_type as P
    want = {("f64", "f32"): "f64", ("f64", "f64"): "f64", ("i64", "f64"): "f64", ("i64", "f32"): "f32", ("i64", "i32"): "i64",
            ("i32", "i32"): "i32", ("c128", "c64"): "c128", ("c128", "f32"): "c128", ("c128", "i64"): "c128", ("c64", "f64"): "c128",
            ("c64", "f32"): "c64", ("c64", "i64"): "c64", ("f16", "f32"): "f32", ("bf16", "f16"): "f32", ("f32", "f32"): "f32"}
    for (a, b), t in want.items():
        assert P(a, b) == t and P(b, a) == t, (a, b)
