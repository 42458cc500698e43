"""ctypes front end of the C oracle (``nnlib_oracle.c``) plus an independent numpy statement.

TEST INFRASTRUCTURE ONLY.  Nothing under the product package imports this module; it is used
by ``tests/``, by the smoke check and by the benchmark's CPU-baseline leg.

Arrays follow the Julia convention of the reference: an array of Julia size ``(E, L, B)`` is a
numpy array of shape ``(E, L, B)`` in Fortran (column-major) memory order.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile the C oracle next to its source (gcc, a second or two)."""
    so = os.path.join(_HERE, "libnnlib_oracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libnnlib_oracle.so")
        if not os.path.exists(so):
            build()
        L = ctypes.CDLL(so)
        i64, f32, f64, vp, ci = ctypes.c_int64, ctypes.c_float, ctypes.c_double, ctypes.c_void_p, ctypes.c_int
        L.orc_batched_gemm_f32.argtypes = [ci, ci, i64, i64, i64, f32, vp, i64, i64, i64, vp, i64, i64, i64,
                                           f32, vp, i64, i64, i64, ci]
        L.orc_batched_gemm_f32.restype = None
        L.orc_batched_gemm_f64.argtypes = [ci, ci, i64, i64, i64, f64, vp, i64, i64, vp, i64, i64, f64, vp,
                                           i64, i64, i64]
        L.orc_batched_gemm_f64.restype = None
        L.orc_softmax_dim1_f32.argtypes = [vp, vp, i64, i64]
        L.orc_softmax_dim1_f32.restype = None
        L.orc_softmax_dim1_f64.argtypes = [vp, vp, i64, i64]
        L.orc_softmax_dim1_f64.restype = None
        L.orc_make_causal_mask.argtypes = [vp, i64]
        L.orc_make_causal_mask.restype = None
        L.orc_nnlib_attention_f32.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, vp, ci]
        L.orc_nnlib_attention_f32.restype = None
        L.orc_attention_f64.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, vp]
        L.orc_attention_f64.restype = None
        L.orc_attention_bwd_f64.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, vp, vp, vp]
        L.orc_attention_bwd_f64.restype = None
        for suf in ("f32", "f64"):
            getattr(L, "orc_softmax_nd_" + suf).argtypes = [ci, vp, vp, i64, i64, i64]
            getattr(L, "orc_logsumexp_" + suf).argtypes = [vp, vp, i64, i64, i64]
            getattr(L, "orc_softmax_bwd_" + suf).argtypes = [ci, vp, vp, vp, i64, i64, i64]
            getattr(L, "orc_logsumexp_bwd_" + suf).argtypes = [vp, vp, vp, i64, i64, i64]
            for n in ("orc_softmax_nd_", "orc_logsumexp_", "orc_softmax_bwd_", "orc_logsumexp_bwd_"):
                getattr(L, n + suf).restype = None
        L.orc_set_sgemm.argtypes = [vp]
        L.orc_set_sgemm.restype = None
        L.orc_has_sgemm.restype = ci
        _LIB = L
    return _LIB


def use_host_blas(enable=True):
    """Run the Float32 GEMM slices of ``batched_gemm`` / ``nnlib_attention_f32`` with the host's BLAS ``sgemm_``, as
    the reference does (src/gemm.jl:141-149), instead of the oracle's own kernel.  The routine is the one SciPy
    ships (``scipy.linalg.cython_blas``: OpenBLAS), pinned to one BLAS thread as src/gemm.jl:152-155 pins it inside
    its threaded loop.  Used by the benchmark's CPU baseline only; parity tests keep the oracle's own kernel.
    Returns a description of the BLAS in use, or None when none could be bound (the own kernel stays)."""
    L = lib()
    if not enable:
        L.orc_set_sgemm(None)
        return None
    try:
        from scipy.linalg import cython_blas
        cap = cython_blas.__pyx_capi__["sgemm"]
        api = ctypes.pythonapi
        api.PyCapsule_GetName.restype, api.PyCapsule_GetName.argtypes = ctypes.c_char_p, [ctypes.py_object]
        api.PyCapsule_GetPointer.restype, api.PyCapsule_GetPointer.argtypes = ctypes.c_void_p, [ctypes.py_object, ctypes.c_char_p]
        fn = api.PyCapsule_GetPointer(cap, api.PyCapsule_GetName(cap))
        if not fn:
            return None
        desc = "SciPy's BLAS sgemm_"
        try:
            import threadpoolctl
            threadpoolctl.threadpool_limits(1, user_api="blas")
            info = [i for i in threadpoolctl.threadpool_info() if i.get("user_api") == "blas"]
            if info:
                desc = f"{info[0].get('internal_api', 'blas')} {info[0].get('version', '')} sgemm_ (SciPy's), 1 BLAS thread"
        except Exception:
            pass
        L.orc_set_sgemm(fn)
        return desc
    except Exception:
        L.orc_set_sgemm(None)
        return None


def _f(a, dt):
    return np.asfortranarray(np.asarray(a, dtype=dt))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def broadcast_strides(shape, target_ndim=4):
    """Element strides (column-major) of an array broadcast against a ``target_ndim``-D tensor.

    Dimensions of extent 1 (or missing trailing dimensions) get stride 0, which is how
    Julia broadcasting treats them (reference src/attention.jl:131,137)."""
    shape = tuple(shape) + (1,) * (target_ndim - len(shape))
    out, acc = [], 1
    for n in shape:
        out.append(0 if n == 1 else acc)
        acc *= n
    return (ctypes.c_int64 * target_ndim)(*out)


def _flatten3(x):
    """(F, L, batch...) -> (F, L, prod(batch)) as the N-D method does (src/attention.jl:43)."""
    x = np.asarray(x)
    return x.reshape(x.shape[0], x.shape[1], -1, order="F")


def make_causal_mask(length):
    m = np.zeros((length, length), dtype=np.uint8, order="F")
    lib().orc_make_causal_mask(_ptr(m), length)
    return m.astype(bool)


def softmax_dim1(x, dtype=np.float32):
    x = _f(x, dtype)
    rows = x.shape[0] if x.ndim else 1
    cols = x.size // max(rows, 1)
    y = np.empty_like(x, order="F")
    fn = lib().orc_softmax_dim1_f32 if dtype == np.float32 else lib().orc_softmax_dim1_f64
    fn(_ptr(x), _ptr(y), rows, cols)
    return y


_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _mix64(z):
    """splitmix64 finaliser on uint64 arrays (wraps modulo 2^64)."""
    with np.errstate(over="ignore"):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def dropout_keep_mask(shape, p, seed):
    """Keep decisions (column-major linear index order) of the library's dropout stream: the published
    definition restated in numpy: bits(g) = mix64(mix64(seed ^ stream*C) + g*G) serves the four elements
    i = 4g .. 4g+3, u(i) = (bits(i >> 2) >> 16*(i & 3)) & 0xFFFF, keep = u >= ceil(p * 2^16).  The product's
    kernels must reproduce exactly this mask."""
    n = int(np.prod(shape, dtype=np.int64))
    i = np.arange(n, dtype=np.uint64)
    with np.errstate(over="ignore"):
        key = _mix64(np.array([seed], dtype=np.uint64) ^ (np.uint64(0x64726F70) * np.uint64(0xD1342543DE82EF95)))
        bits = _mix64(key + (i >> np.uint64(2)) * np.uint64(0x9E3779B97F4A7C15))
    thresh = min(max(int(np.ceil(np.float32(p).astype(np.float64) * 65536.0)), 0), 65536)
    keep = ((bits >> (np.uint64(16) * (i & np.uint64(3)))) & np.uint64(0xFFFF)).astype(np.int64) >= thresh
    return keep.reshape(shape, order="F")


def reduction_geometry(shape, dims):
    """(inner, len, outer, kept shape) of a reduction over ``dims`` (1-based dimension, tuple of adjacent
    dimensions, or None for Julia's ``:``) of a column-major array."""
    shape = tuple(shape)
    if dims is None:
        return 1, int(np.prod(shape, dtype=np.int64)), 1, ()
    ds = sorted(set(dims if isinstance(dims, (tuple, list)) else (dims,)))
    assert ds == list(range(ds[0], ds[-1] + 1))
    nd = len(shape)
    padded = shape + (1,) * max(0, ds[-1] - nd)       # dimensions past ndims have extent 1 in Julia
    lo, hi = ds[0] - 1, ds[-1]
    prod = lambda t: int(np.prod(t, dtype=np.int64)) if t else 1
    kept = (padded[:lo] + (1,) * (hi - lo) + padded[hi:])[:nd]
    return prod(padded[:lo]), prod(padded[lo:hi]), prod(padded[hi:]), kept


def _suffix(dtype):
    return "f32" if dtype == np.float32 else "f64"


def softmax(x, dims=1, dtype=np.float64, log=False):
    """softmax / logsoftmax over ``dims`` (src/softmax.jl:69-79, 137-147)."""
    x = _f(x, dtype)
    inner, n, outer, _ = reduction_geometry(x.shape, dims)
    y = np.empty_like(x, order="F")
    getattr(lib(), "orc_softmax_nd_" + _suffix(dtype))(int(log), _ptr(x), _ptr(y), inner, n, outer)
    return y


def logsoftmax(x, dims=1, dtype=np.float64):
    return softmax(x, dims, dtype, log=True)


def logsumexp(x, dims=None, dtype=np.float64):
    """logsumexp(x; dims) (src/softmax.jl:200-203); reduced dimensions are kept with extent 1."""
    x = _f(x, dtype)
    inner, n, outer, kept = reduction_geometry(x.shape, dims)
    y = np.empty(kept, dtype=dtype, order="F")
    getattr(lib(), "orc_logsumexp_" + _suffix(dtype))(_ptr(x), _ptr(y), inner, n, outer)
    return y


def grad_logsumexp(dy, x, dims=None, dtype=np.float64):
    """Pullback of logsumexp(x; dims) (rrule, src/softmax.jl:205-212): dy has the size of the reduced result."""
    x = _f(x, dtype)
    inner, n, outer, kept = reduction_geometry(x.shape, dims)
    dy = _f(np.asarray(dy, dtype=dtype).reshape(kept if kept else (1,), order="F"), dtype)
    dx = np.empty_like(x, order="F")
    getattr(lib(), "orc_logsumexp_bwd_" + _suffix(dtype))(_ptr(dy), _ptr(x), _ptr(dx), inner, n, outer)
    return dx


def grad_softmax(dy, y, dims=1, dtype=np.float64, log=False):
    """∇softmax / ∇logsoftmax given the forward result y (src/softmax.jl:107-110, 175-177)."""
    dy, y = _f(dy, dtype), _f(y, dtype)
    inner, n, outer, _ = reduction_geometry(y.shape, dims)
    dx = np.empty_like(y, order="F")
    getattr(lib(), "orc_softmax_bwd_" + _suffix(dtype))(int(log), _ptr(dy), _ptr(y), _ptr(dx), inner, n, outer)
    return dx


def grad_logsoftmax(dy, y, dims=1, dtype=np.float64):
    return grad_softmax(dy, y, dims, dtype, log=True)


def per_slice_product(A, B, adjA=False, adjB=False, transA=False, transB=False):
    """The reference's own oracle for batched_mul (bmm_test / bmm_adjtest, test/batchedmul.jl:6-28): the
    ordinary matrix product slice by slice, in double precision (complex128 for complex inputs); a batch
    extent of 1 is shared by every slice.  adj = conjugate transpose of each slice, trans = transpose."""
    A, B = np.asarray(A), np.asarray(B)
    wide = np.complex128 if (np.iscomplexobj(A) or np.iscomplexobj(B)) else np.float64
    A, B = A.astype(wide), B.astype(wide)
    op = lambda X, adj, tr: X.conj().T if adj else (X.T if tr else X)
    nb = max(A.shape[2], B.shape[2])
    out = [op(A[:, :, i if A.shape[2] > 1 else 0], adjA, transA) @ op(B[:, :, i if B.shape[2] > 1 else 0], adjB, transB)
           for i in range(nb)]
    return np.stack(out, axis=2)


def batched_gemm(A, B, transA=False, transB=False, alpha=1.0, beta=0.0, C=None, dtype=np.float32, nthreads=1):
    """3-D column-major batched GEMM; a batch extent of 1 on A or B broadcasts."""
    A, B = _f(A, dtype), _f(B, dtype)
    m, ka = (A.shape[1], A.shape[0]) if transA else (A.shape[0], A.shape[1])
    kb, n = (B.shape[1], B.shape[0]) if transB else (B.shape[0], B.shape[1])
    assert ka == kb
    batch = max(A.shape[2], B.shape[2])
    if C is None:
        C = np.zeros((m, n, batch), dtype=dtype, order="F")
    else:
        C = _f(C, dtype).copy(order="F")
    sA = 0 if A.shape[2] == 1 else A.shape[0] * A.shape[1]
    sB = 0 if B.shape[2] == 1 else B.shape[0] * B.shape[1]
    if dtype == np.float32:
        lib().orc_batched_gemm_f32(int(transA), int(transB), m, n, ka, alpha, _ptr(A), A.shape[0], sA, A.size,
                                   _ptr(B), B.shape[0], sB, B.size, beta, _ptr(C), m, m * n, batch, nthreads)
    else:
        lib().orc_batched_gemm_f64(int(transA), int(transB), m, n, ka, alpha, _ptr(A), A.shape[0], sA,
                                   _ptr(B), B.shape[0], sB, beta, _ptr(C), m, m * n, batch)
    return C


def _attention(q, k, v, bias, mask, nheads, dtype, want_out, nthreads):
    bshape = tuple(np.shape(q)[2:])
    q3, k3 = _f(_flatten3(q), dtype), _f(_flatten3(k), dtype)
    v3 = _f(_flatten3(v), dtype) if v is not None else None
    E, Lq, B = q3.shape
    Lkv = k3.shape[1]
    Ev = v3.shape[0] if v3 is not None else E
    H = nheads
    bs = ms = None
    if bias is not None:
        bias = _f(bias, dtype)
        bs = broadcast_strides(bias.shape)
    if mask is not None:
        mask = np.asfortranarray(np.asarray(mask).astype(np.uint8))
        ms = broadcast_strides(mask.shape)
    alpha = np.empty((Lkv, Lq, H, B), dtype=dtype, order="F")
    out = np.empty((Ev, Lq, B), dtype=dtype, order="F") if want_out else None
    if dtype == np.float32:
        lib().orc_nnlib_attention_f32(_ptr(q3), _ptr(k3), _ptr(v3), _ptr(bias), bs, _ptr(mask), ms,
                                      E, Ev, Lq, Lkv, H, B, _ptr(out), _ptr(alpha), nthreads)
    else:
        lib().orc_attention_f64(_ptr(q3), _ptr(k3), _ptr(v3), _ptr(bias), bs, _ptr(mask), ms,
                                E, Ev, Lq, Lkv, H, B, _ptr(out), _ptr(alpha))
    alpha = alpha.reshape((Lkv, Lq, H) + bshape, order="F")
    if want_out:
        out = out.reshape((Ev, Lq) + bshape, order="F")
    return out, alpha


def nnlib_attention_f32(q, k, v, bias=None, mask=None, nheads=1, nthreads=1):
    """The reference's op sequence in Float32 (src/attention.jl:52-127). Returns (x, alpha)."""
    return _attention(q, k, v, bias, mask, nheads, np.float32, True, nthreads)


def attention_f64(q, k, v, bias=None, mask=None, nheads=1):
    """Defining formula in double precision. Returns (x, alpha)."""
    return _attention(q, k, v, bias, mask, nheads, np.float64, True, 1)


def scores4_f64(q4, k4, bias=None, mask=None):
    """dot_product_attention_scores on 4-D (D, H, L, B) inputs (src/attention.jl:112-127)."""
    q4, k4 = np.asarray(q4), np.asarray(k4)
    D, H, Lq, B = q4.shape
    q3 = q4.reshape(D * H, Lq, B, order="F")
    k3 = k4.reshape(D * H, k4.shape[2], B, order="F")
    return _attention(q3, k3, None, bias, mask, H, np.float64, False, 1)[1]


def attention_bwd_f64(q, k, v, dout, bias=None, mask=None, nheads=1, dweights=None, keep_scale=None):
    """Gradient of dot_product_attention with respect to q, k, v and bias, given the cotangent ``dout``
    of the output (and optionally ``dweights`` of the returned weights): the reverse of the op chain of
    src/attention.jl:86-127.  ``keep_scale``: the (Lkv, Lq, H, B) factor a dropout ``fdrop`` multiplied the
    weights by (0 or 1/(1-p)).  Returns (dq, dk, dv, dbias); dbias has the shape of ``bias`` (None without)."""
    f8 = np.float64
    bshape = tuple(np.shape(q)[2:])
    q3, k3, v3, do3 = (_f(_flatten3(a), f8) for a in (q, k, v, dout))
    E, Lq, B = q3.shape
    Lkv, Ev, H = k3.shape[1], v3.shape[0], nheads
    _, alpha = _attention(q, k, v, bias, mask, nheads, f8, True, 1)
    alpha = _f(alpha.reshape(Lkv, Lq, H, B, order="F"), f8)
    dq, dk, dv = (np.empty(a.shape, dtype=f8, order="F") for a in (q3, k3, v3))
    dw = None if dweights is None else _f(np.asarray(dweights).reshape(Lkv, Lq, H, B, order="F"), f8)
    ks = None if keep_scale is None else _f(np.asarray(keep_scale).reshape(Lkv, Lq, H, B, order="F"), f8)
    db = bs = None
    if bias is not None:
        db = np.zeros(np.shape(bias), dtype=f8, order="F")
        bs = broadcast_strides(db.shape)
    lib().orc_attention_bwd_f64(_ptr(q3), _ptr(k3), _ptr(v3), _ptr(alpha), _ptr(do3), _ptr(dw), _ptr(ks), bs,
                                E, Ev, Lq, Lkv, H, B, _ptr(dq), _ptr(dk), _ptr(dv), _ptr(db))
    return (dq.reshape(np.shape(q), order="F"), dk.reshape(np.shape(k), order="F"),
            dv.reshape(np.shape(v), order="F"), db)


def numpy_attention_bwd(q, k, v, dout, bias=None, mask=None, nheads=1, dweights=None, keep_scale=None):
    """Independent einsum statement of the same gradient (no C involved)."""
    f8 = np.float64
    q3, k3, v3, do3 = (_flatten3(np.asarray(a, dtype=f8)) for a in (q, k, v, dout))
    E, Lq, B = q3.shape
    Lkv, Ev, H = k3.shape[1], v3.shape[0], nheads
    D, Dv = E // H, Ev // H
    _, alpha = numpy_attention(q, k, v, bias, mask, nheads)
    alpha = alpha.reshape(Lkv, Lq, H, B, order="F")
    q4, k4 = q3.reshape(D, H, Lq, B, order="F"), k3.reshape(D, H, Lkv, B, order="F")
    v4, do4 = v3.reshape(Dv, H, Lkv, B, order="F"), do3.reshape(Dv, H, Lq, B, order="F")
    da = np.einsum("dhjb,dhib->jihb", v4, do4)
    if dweights is not None:
        da = da + np.asarray(dweights, dtype=f8).reshape(Lkv, Lq, H, B, order="F")
    g = 1.0 if keep_scale is None else np.asarray(keep_scale, dtype=f8).reshape(Lkv, Lq, H, B, order="F")
    dv4 = np.einsum("jihb,dhib->dhjb", alpha * g, do4)
    da = da * g
    dl = alpha * (da - (alpha * da).sum(axis=0, keepdims=True))
    c = 1.0 / np.sqrt(f8(D))
    dq4 = c * np.einsum("jihb,dhjb->dhib", dl, k4)
    dk4 = c * np.einsum("jihb,dhib->dhjb", dl, q4)
    db = None
    if bias is not None:
        bshape = tuple(np.shape(bias)) + (1,) * (4 - np.ndim(bias))
        axes = tuple(a for a in range(4) if bshape[a] == 1)
        db = dl.sum(axis=axes, keepdims=True).reshape(np.shape(bias), order="F")
    return (dq4.reshape(np.shape(q), order="F"), dk4.reshape(np.shape(k), order="F"),
            dv4.reshape(np.shape(v), order="F"), db)


# ---------------------------------------------------------------------------------------------
# Independent numpy statement (no C involved): used to cross-check the C oracle itself.
# ---------------------------------------------------------------------------------------------

def numpy_attention(q, k, v, bias=None, mask=None, nheads=1):
    """x[d,h,i,b] = sum_j softmax_j(sum_d k[d,h,j,b] q[d,h,i,b]/sqrt(D) + bias, masked) v[d,h,j,b]
    evaluated with einsum in float64 on Julia-shaped arrays."""
    bshape = tuple(np.shape(q)[2:])
    q3, k3, v3 = (_flatten3(np.asarray(a, dtype=np.float64)) for a in (q, k, v))
    E, Lq, B = q3.shape
    Lkv, Ev, H = k3.shape[1], v3.shape[0], nheads
    D, Dv = E // H, Ev // H
    q4 = q3.reshape(D, H, Lq, B, order="F")
    k4 = k3.reshape(D, H, Lkv, B, order="F")
    v4 = v3.reshape(Dv, H, Lkv, B, order="F")
    logits = np.einsum("dhjb,dhib->jihb", k4, q4 / np.sqrt(np.float64(D)))
    if bias is not None:
        b = np.asarray(bias, dtype=np.float64)
        logits = logits + b.reshape(b.shape + (1,) * (4 - b.ndim))
    if mask is not None:
        m = np.asarray(mask, dtype=bool)
        logits = np.where(m.reshape(m.shape + (1,) * (4 - m.ndim)), logits, -np.inf)
    with np.errstate(invalid="ignore", over="ignore"):
        mx = logits.max(axis=0, keepdims=True)
        e = np.where(np.isposinf(mx), np.where(np.isposinf(logits), 1.0, 0.0), np.exp(logits - mx))
        alpha = e / e.sum(axis=0, keepdims=True)
    x = np.einsum("jihb,dhjb->dhib", alpha, v4).reshape(Ev, Lq, B, order="F")
    return x.reshape((Ev, Lq) + bshape, order="F"), alpha.reshape((Lkv, Lq, H) + bshape, order="F")
