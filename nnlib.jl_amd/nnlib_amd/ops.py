"""Python mirror of the reference's operator interface for the attention path.

Same names, argument meaning and error behaviour as NNlib.jl (citations are paths in the
NNlib.jl source tree).  Every function marshals arguments and calls the C ABI
(``include/mi355attn.h``); all arithmetic happens in the HIP kernels.
"""
import ctypes

import numpy as np
import torch

from . import _lib
from ._lib import ArgumentError, DimensionMismatch
from .array import BatchedTranspose, CausalAnd, CausalMask, DeviceArray, batched_transpose

__all__ = ["dot_product_attention", "dot_product_attention_scores", "make_causal_mask", "softmax", "softmax_",
           "logsoftmax", "logsoftmax_", "logsumexp", "grad_softmax", "grad_softmax_", "grad_logsoftmax",
           "grad_logsoftmax_", "batched_mul", "batched_mul_", "batched_mul_pullback", "last_attention_kernel", "last_attention_workspace",
           "dot_product_attention_grad", "last_attention_bwd_kernel", "Dropout", "dropout", "batched_vec"]

_last_kernel = None
_last_workspace = 0
_workspace = None


def identity(x):
    return x


class Dropout:
    """``fdrop = Dropout(p, seed)``: the reference's ``x -> dropout(x, p)`` (src/dropout.jl:38-53) with a
    reproducible counter-based stream.  ``dot_product_attention`` recognises it and applies the dropout
    inside the attention kernel; called on an array it runs the standalone kernel, with the same keep
    decisions for the same seed."""

    def __init__(self, p, seed=0):
        if not 0 <= p <= 1:
            raise ArgumentError("dropout expects a probability 0 <= p <= 1")      # src/dropout.jl:43
        self.p, self.seed = float(p), int(seed)

    def __call__(self, x):
        return dropout(x, self.p, seed=self.seed)


def dropout(x, p, *, seed=0, dims=None):
    """dropout(A, p; dims = :)  (src/dropout.jl:38-53): zero with probability p, else scale by 1/(1-p)."""
    x = _contig(x, "x")
    if x.dtype == "bool":
        raise ArgumentError("dropout needs a floating-point array")
    out = DeviceArray.empty(x.dims, x.dtype)
    if dims is not None:
        ds = {int(d) for d in (dims if isinstance(dims, (tuple, list)) else (dims,))}
        if not ds or min(ds) < 1:
            raise ArgumentError(f"dims must be positive dimension numbers, got {dims}")
        if x.ndim > 8:
            raise ArgumentError("dropout along dims takes arrays of up to 8 dimensions")
        mask = sum(1 << (d - 1) for d in ds if d <= x.ndim)
        sizes = (ctypes.c_int64 * max(x.ndim, 1))(*x.dims)
        _lib.check(_lib.load().mi_dropout_dims(x.code, x.ptr, out.ptr, x.ndim, sizes, mask, float(p), int(seed), _stream()))
        return out
    _lib.check(_lib.load().mi_dropout(x.code, x.ptr, out.ptr, x.length, float(p), int(seed), _stream()))
    return out


def last_attention_kernel():
    """Name of the kernel family the most recent attention call dispatched to."""
    return _lib.KERNEL_NAMES.get(_last_kernel)


def last_attention_workspace():
    """Workspace bytes the library asked for in the most recent attention call (non-zero: a split key range)."""
    return _last_workspace


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _get_workspace(nbytes):
    global _workspace
    if nbytes == 0:
        return None, 0
    if _workspace is None or _workspace.numel() < nbytes:
        _workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    return _workspace, _workspace.numel()


def _broadcast_strides(x, target, what):
    """Element strides of ``x`` against the 4-D score tensor ``target`` = (kv, q, H, B); 0 where
    ``x`` has extent 1.  Julia broadcasting raises DimensionMismatch otherwise."""
    dims = tuple(x.dims) + (1,) * (4 - len(x.dims))
    strides = tuple(x.strides) + (0,) * (4 - len(x.strides))
    if len(dims) > 4 and any(d != 1 for d in dims[4:]):
        raise DimensionMismatch(f"{what} of size {x.dims} is not broadcastable to {target}")
    out = []
    for d, s, t in zip(dims[:4], strides[:4], target):
        if d == 1:
            out.append(0)
        elif d == t:
            out.append(s)
        else:
            raise DimensionMismatch(f"arrays could not be broadcast to a common size: {what} has size {x.dims}, "
                                    f"attention scores have size {target}")
    return out


def _fill_desc(d, q, k, v, bias, mask, H, B, E, Ev, Lq, Lkv, flags, fdrop=None):
    """Forward-call part of a descriptor: element type, sizes, inputs, bias / mask strides."""
    d.struct_size = ctypes.sizeof(_lib.mi_attn_desc)
    if fdrop is not None:
        d.dropout_p, d.dropout_seed = fdrop.p, fdrop.seed
    d.dtype = d.weights_dtype = q.code_f64
    d.flags = flags
    d.E, d.Ev, d.Lq, d.Lkv, d.H, d.B = E, Ev, Lq, Lkv, H, B
    d.q, d.k = q.ptr, k.ptr
    d.v = v.ptr if v is not None else None
    target = (Lkv, Lq, H, B)
    if bias is not None:
        if bias.dtype != q.dtype:
            raise ArgumentError(f"bias must have the element type of q ({q.dtype}), got {bias.dtype}")
        st = _broadcast_strides(bias, target, "bias")
        d.bias = bias.ptr
        d.bias_strides = (ctypes.c_int64 * 4)(*st)
    d.causal = 0
    if isinstance(mask, (CausalMask, CausalAnd)):
        if mask.length != Lkv or mask.length != Lq:
            raise DimensionMismatch(f"arrays could not be broadcast to a common size: mask has size {(mask.length, mask.length)}, "
                                    f"attention scores have size {target}")
        d.causal = 1
        mask = mask.array if isinstance(mask, CausalAnd) else None   # causal .& array: the flag and the array together
    if mask is not None:
        if mask.dtype != "bool":
            raise ArgumentError("mask must be a Bool array")
        st = _broadcast_strides(mask, target, "mask")
        d.mask = mask.ptr
        d.mask_strides = (ctypes.c_int64 * 4)(*st)


def _attention_call(q, k, v, bias, mask, H, B, E, Ev, Lq, Lkv, want_out, want_weights, weights_dtype, flags,
                    fdrop=None, save_stats=False):
    """One mi_attention_fwd call on flattened (F, L, B) operands."""
    global _last_kernel, _last_workspace
    lib = _lib.load()
    d = _lib.mi_attn_desc()
    _fill_desc(d, q, k, v, bias, mask, H, B, E, Ev, Lq, Lkv, flags, fdrop)
    out = DeviceArray.empty((Ev, Lq, B), q.dtype) if want_out else None
    wdt = weights_dtype or q.dtype
    alpha = DeviceArray.empty((Lkv, Lq, H, B), wdt) if want_weights else None
    d.out = out.ptr if out is not None else None
    d.weights = alpha.ptr if alpha is not None else None
    d.weights_dtype = alpha.code_f64 if alpha is not None else q.code_f64
    kernel, ws = ctypes.c_int32(0), ctypes.c_size_t(0)
    _lib.check(lib.mi_attention_plan(ctypes.byref(d), ctypes.byref(kernel), ctypes.byref(ws)))
    stats = None
    if save_stats and out is not None and kernel.value in (_lib.KERNEL_FLASH16, _lib.KERNEL_FLASH32):
        # softmax row statistics for dot_product_attention_grad (what an AD rule keeps for its pullback)
        nb = ctypes.c_size_t(0)
        _lib.check(lib.mi_attention_stats_size(ctypes.byref(d), ctypes.byref(nb)))
        stats = DeviceArray.empty((nb.value // 4,), "f32")
        d.stats = stats.ptr
        _lib.check(lib.mi_attention_plan(ctypes.byref(d), ctypes.byref(kernel), ctypes.byref(ws)))   # saving them rules out split-kv
    wbuf, wsize = _get_workspace(ws.value)
    if wbuf is not None:
        d.workspace, d.workspace_bytes = wbuf.data_ptr(), wsize
    _lib.check(lib.mi_attention_fwd(ctypes.byref(d), _stream()))
    _last_kernel = kernel.value
    _last_workspace = ws.value
    if stats is not None:
        out.saved_stats = stats
    return out, alpha


def _contig(x, name):
    if not isinstance(x, DeviceArray):
        raise ArgumentError(f"{name} must be a DeviceArray")
    if not x.is_contiguous():
        raise ArgumentError(f"{name} must be a dense column-major array")
    return x


def _check_qkv(q, k, v, nheads):
    """The argument checks of src/attention.jl:40-78; returns (B, E, Ev, Lq, Lkv, batch dims)."""
    q, k, v = _contig(q, "q"), _contig(k, "k"), _contig(v, "v")
    if not (q.ndim == k.ndim == v.ndim) or q.ndim < 2:
        raise ArgumentError("query, key and value must have the same number of dimensions (at least 2)")
    if not (q.dtype == k.dtype == v.dtype) or q.dtype == "bool":
        raise ArgumentError("query, key and value must share a floating-point element type")
    bq, bk, bv = q.dims[2:], k.dims[2:], v.dims[2:]
    if not (bq == bk == bv):                                     # src/attention.jl:42, :63
        raise ArgumentError("Batch dimensions have to be the same.")
    B = int(np.prod(bq, dtype=np.int64)) if bq else 1
    E, Lq, Lkv, Ev = q.dims[0], q.dims[1], k.dims[1], v.dims[0]
    if E % nheads or k.dims[0] % nheads or Ev % nheads:          # src/attention.jl:55
        raise ArgumentError("First dimension in query, key and value must be divisible by `nheads`.\n"
                            f"Instead:\n- size(q): {q.dims}\n- size(k): {k.dims}\n- size(v): {v.dims}\n- nheads: {nheads}")
    if E != k.dims[0]:                                           # src/attention.jl:69
        raise ArgumentError("First dimension in query and key has to be the same. Instead:\n"
                            f"- size(q): {q.dims}\n- size(k): {k.dims}")
    if Lkv != v.dims[1]:                                         # src/attention.jl:74
        raise ArgumentError("Second dimension in key and value has to be the same. Instead:\n"
                            f"- size(k): {k.dims}\n- size(v): {v.dims}")
    return B, E, Ev, Lq, Lkv, tuple(bq)


def dot_product_attention(q, k, v, bias=None, *, fdrop=identity, mask=None, nheads=1, return_weights=True,
                          weights_dtype=None, save_for_backward=False, _flags=0):
    """dot_product_attention(query, key, value, [bias]; [fdrop, mask, nheads])  (src/attention.jl:40-84).

    q (qk_dim, q_len, batch...), k (qk_dim, kv_len, batch...), v (v_dim, kv_len, batch...).
    Returns ``(x, alpha)``: x (v_dim, q_len, batch...), alpha (kv_len, q_len, nheads, batch...).

    Beyond the reference: ``return_weights=False`` skips materialising alpha (``None`` is returned
    in its place), ``weights_dtype="f32"`` asks for Float32 weights from 16-bit inputs, and
    ``save_for_backward=True`` keeps the softmax row statistics on the returned ``x`` (attribute
    ``saved_stats``) so that ``dot_product_attention_grad(..., y=x)`` need not recompute them."""
    B, E, Ev, Lq, Lkv, bq = _check_qkv(q, k, v, nheads)
    if fdrop is identity or isinstance(fdrop, Dropout):
        x, alpha = _attention_call(q, k, v, bias, mask, nheads, B, E, Ev, Lq, Lkv, True, return_weights,
                                   weights_dtype, _flags, fdrop if isinstance(fdrop, Dropout) else None, save_for_backward)
    else:
        # alpha handed back is post-fdrop (src/attention.jl:126); the value product then runs as a
        # batched GEMM on the caller-visible weights, as src/attention.jl:96-98 does.
        _, alpha = _attention_call(q, k, None, bias, mask, nheads, B, E, Ev, Lq, Lkv, False, True, weights_dtype,
                                   _flags)
        alpha = fdrop(alpha)
        x = _weights_times_values(alpha, v, nheads, B, Ev, Lq, Lkv)
    stats = getattr(x, "saved_stats", None)
    x = x.reshape((Ev, Lq) + tuple(bq))
    if stats is not None:
        x.saved_stats = stats
    if alpha is not None:
        alpha = alpha.reshape((Lkv, Lq, nheads) + tuple(bq))
    return x, alpha


_last_bwd_kernel = None


def last_attention_bwd_kernel():
    """Name of the kernel family the most recent attention gradient call dispatched to."""
    return _lib.KERNEL_NAMES.get(_last_bwd_kernel)


def dot_product_attention_grad(dy, q, k, v, bias=None, *, y=None, dalpha=None, mask=None, nheads=1, fdrop=identity,
                               _flags=0):
    """Pullback of ``dot_product_attention(q, k, v, bias; fdrop, mask, nheads)`` for ``fdrop = identity`` or
    a ``Dropout(p, seed)`` (the same object the forward call got, so that the keep decisions repeat):
    given the cotangent ``dy`` of the output (and optionally ``dalpha`` of the returned weights) it
    returns ``(dq, dk, dv, dbias)``; ``dbias`` is ``None`` without a bias and has the bias's size
    otherwise (Float32).  The reference gets the same values from AD through src/attention.jl:86-127
    (rrule of batched_mul, src/batched/batchedmul.jl:96-110; _∇softmax!, src/softmax.jl:107-110; the
    pullback of dropout multiplies by the mask it drew, src/dropout.jl:38-53).
    ``y`` is the forward result, which the MFMA kernels need; without it (and without ``dalpha``) the library
    recomputes it with one forward call where those kernels can take the gradient."""
    global _last_bwd_kernel
    B, E, Ev, Lq, Lkv, bq = _check_qkv(q, k, v, nheads)
    dy = _contig(dy, "dy")
    if dy.dims != (Ev, Lq) + bq or dy.dtype != q.dtype:
        raise DimensionMismatch(f"dy must have the size and element type of the output {(Ev, Lq) + bq}, got {dy.dims}")
    lib = _lib.load()
    d = _lib.mi_attn_bwd_desc()
    d.struct_size = ctypes.sizeof(_lib.mi_attn_bwd_desc)
    if fdrop is not identity and not isinstance(fdrop, Dropout):
        raise ArgumentError("the fused gradient takes fdrop = identity or a Dropout(p, seed)")
    _fill_desc(d.fwd, q, k, v, bias, mask, nheads, B, E, Ev, Lq, Lkv, _flags, fdrop if isinstance(fdrop, Dropout) else None)
    if y is not None:
        y = _contig(y, "y")
        if y.dims != dy.dims or y.dtype != q.dtype:
            raise DimensionMismatch("y must have the size and element type of dy")
        d.fwd.out = y.ptr
        if getattr(y, "saved_stats", None) is not None and dalpha is None:
            d.fwd.stats = y.saved_stats.ptr
    d.dout = dy.ptr
    if dalpha is not None:
        dalpha = _contig(dalpha, "dalpha")
        if dalpha.dims != (Lkv, Lq, nheads) + bq or dalpha.dtype != q.dtype:
            raise DimensionMismatch(f"dalpha must have size {(Lkv, Lq, nheads) + bq} and the element type of q")
        d.dweights = dalpha.ptr
    dq, dk, dv = DeviceArray.empty(q.dims, q.dtype), DeviceArray.empty(k.dims, q.dtype), DeviceArray.empty(v.dims, q.dtype)
    d.dq, d.dk, d.dv = dq.ptr, dk.ptr, dv.ptr
    dbias = None
    if bias is not None:
        dbias = DeviceArray.zeros(bias.dims, "f32")
        d.dbias = dbias.ptr
    kernel, ws = ctypes.c_int32(0), ctypes.c_size_t(0)
    # without the forward result the library recomputes it where its MFMA kernels can take the gradient (the plan's
    # workspace has room for it)
    _lib.check(lib.mi_attention_bwd_plan(ctypes.byref(d), ctypes.byref(kernel), ctypes.byref(ws)))
    wbuf, wsize = _get_workspace(ws.value)
    if wbuf is not None:
        d.workspace, d.workspace_bytes = wbuf.data_ptr(), wsize
    _lib.check(lib.mi_attention_bwd(ctypes.byref(d), _stream()))
    _last_bwd_kernel = kernel.value
    return dq, dk, dv, dbias


def _weights_times_values(alpha, v, H, B, Ev, Lq, Lkv):
    """x[d,h,i,b] = sum_j alpha[j,i,h,b] v[d,h,j,b] as strided batched GEMMs over heads, one per batch
    (no permuted copies: a head of v is a (Dv, Lkv) matrix with column stride Ev)."""
    if alpha.dtype != v.dtype:
        raise ArgumentError("fdrop must keep the element type of the attention weights")
    lib = _lib.load()
    Dv = Ev // H
    out = DeviceArray.empty((Ev, Lq, B), v.dtype)
    es = v.itemsize
    for b in range(B):
        if v.dtype == "f64":
            _lib.check(lib.mi_batched_gemm_f64(b"N", b"N", Dv, Lq, Lkv, 1.0, v.ptr + es * b * Ev * Lkv, Ev, Dv,
                                               alpha.ptr + es * b * Lkv * Lq * H, Lkv, Lkv * Lq, 0.0,
                                               out.ptr + es * b * Ev * Lq, Ev, Dv, H, _stream()), DimensionMismatch)
            continue
        _lib.check(lib.mi_batched_gemm(v.code, b"N", b"N", Dv, Lq, Lkv, 1.0,
                                       v.ptr + es * b * Ev * Lkv, Ev, Dv,
                                       alpha.ptr + es * b * Lkv * Lq * H, Lkv, Lkv * Lq, 0.0,
                                       out.ptr + es * b * Ev * Lq, Ev, Dv, H, _stream()), DimensionMismatch)
    return out


def dot_product_attention_scores(q, k, bias=None, *, fdrop=identity, mask=None, weights_dtype=None, _flags=0):
    """dot_product_attention_scores(query, key, [bias]; [fdrop, mask])  (src/attention.jl:112-127).
    Inputs are 4-D (num_features / nheads, nheads, sequence_length, batch_size)."""
    q, k = _contig(q, "q"), _contig(k, "k")
    if q.ndim != 4 or k.ndim != 4:
        raise ArgumentError("dot_product_attention_scores expects 4-D (D, nheads, L, batch) arrays")
    if q.dtype != k.dtype:
        raise ArgumentError("query and key must share an element type")
    D, H, Lq, B = q.dims
    if k.dims[0] != D or k.dims[1] != H or k.dims[3] != B:
        raise DimensionMismatch(f"query {q.dims} and key {k.dims} disagree in feature, head or batch size")
    Lkv = k.dims[2]
    fused = fdrop if isinstance(fdrop, Dropout) else None
    _, alpha = _attention_call(q, k, None, bias, mask, H, B, D * H, D * H, Lq, Lkv, False, True, weights_dtype, _flags,
                               fused)
    return alpha if fused is not None else fdrop(alpha)


def make_causal_mask(x, *, dims=2):
    """make_causal_mask(x; dims=2)  (src/attention.jl:149-153): square mask of side size(x, dims) with
    m[i, j] = i <= j.  Returned lazily (see CausalMask); ``.materialize()`` gives the dense Bool array."""
    return CausalMask(x.size(dims))


# ---- softmax family --------------------------------------------------------------------------------

def _reduction_geometry(dims_of_x, dims):
    """(inner, len, outer, kept) for a reduction over ``dims`` of a column-major array: ``dims`` is a
    1-based dimension, a tuple of adjacent dimensions, or ``None`` for Julia's ``:``.  ``kept`` is the
    size of the reduced result (extent 1 along ``dims``, as Julia's ``sum(x; dims)`` keeps them)."""
    size = tuple(dims_of_x)
    if dims is None:
        n = int(np.prod(size, dtype=np.int64)) if size else 1
        return 1, n, 1, ()
    ds = sorted({int(d) for d in (dims if isinstance(dims, (tuple, list)) else (dims,))})
    if not ds or ds[0] < 1:
        raise ArgumentError(f"dims must be positive dimension numbers, got {dims}")
    ds = [d for d in ds if d <= len(size)]       # trailing singleton dimensions reduce to themselves
    if not ds:
        return int(np.prod(size, dtype=np.int64)) if size else 1, 1, 1, size
    if ds != list(range(ds[0], ds[-1] + 1)):   # callers route such sets through _nonadjacent_plan first
        raise ArgumentError(f"dims = {dims}: a single kernel call reduces over a run of adjacent dimensions")
    lo, hi = ds[0] - 1, ds[-1]
    prod = lambda t: int(np.prod(t, dtype=np.int64)) if t else 1
    kept = size[:lo] + (1,) * (hi - lo) + size[hi:]
    return prod(size[:lo]), prod(size[lo:hi]), prod(size[hi:]), kept


def _dims_call(x, dims):
    """Arguments of the `*_dims` entry points for a reduction of ``x`` over ``dims`` (a 1-based dimension, a tuple of
    dimensions, adjacent or not, or ``None`` for Julia's ``:``): (ndim, sizes, mask, workspace pointer, workspace
    bytes, size of the reduced result).  The library permutes sets that are not runs of adjacent dimensions."""
    size = tuple(x.dims)
    if len(size) > 8:
        raise ArgumentError("the softmax family takes arrays of up to 8 dimensions")
    if dims is None:
        ds, kept = list(range(1, len(size) + 1)), ()
    else:
        ds = sorted({int(d) for d in (dims if isinstance(dims, (tuple, list)) else (dims,))})
        if not ds or ds[0] < 1:
            raise ArgumentError(f"dims must be positive dimension numbers, got {dims}")
        kept = tuple(1 if (i + 1) in ds else d for i, d in enumerate(size))
    mask = sum(1 << (d - 1) for d in ds if d <= len(size))
    sizes = (ctypes.c_int64 * max(len(size), 1))(*size)
    nb = ctypes.c_size_t(0)
    _lib.check(_lib.load().mi_softmax_dims_workspace(x.code_f64, len(size), sizes, mask, ctypes.byref(nb)))
    wbuf, wsize = _get_workspace(nb.value)
    return len(size), sizes, mask, (wbuf.data_ptr() if wbuf is not None else None), wsize, kept


def _assign(out, y):
    """out .= y for two dense arrays of one size and element type."""
    out.storage[out.offset:out.offset + out.length].copy_(y.storage[y.offset:y.offset + y.length])
    return out


def _number_error(name):
    # src/softmax.jl:213-218
    return ArgumentError(f"`{name}(x)` called with a number, but it expects an array. Usually this is because a layer "
                         f"like `Dense(3,4,softmax)` is broadcasting it like an activation function; `{name}` needs to "
                         "be outside the layer.")


def _float(x):
    """``float.(x)``: integer arrays become Float64 (what ``similar(x, float(T))`` makes of them, src/softmax.jl:56);
    floating-point arrays are returned as they are."""
    if x.dtype not in ("i32", "i64"):
        return x
    x = _contig(x, "x")
    out = DeviceArray.empty(x.dims, "f64")
    _lib.check(_lib.load().mi_convert(out.ptr, _lib.MI_F64, x.ptr, x.code_any, x.length, _stream()))
    return out


def _softmax_like(name, op, out, x, dims):
    if not isinstance(x, DeviceArray) or not isinstance(out, DeviceArray):
        raise _number_error(name)
    x, out = _contig(_float(x), "x"), _contig(out, "out")
    if out.dims != x.dims:
        raise DimensionMismatch(f"output size {out.dims} differs from input size {x.dims}")
    if x.dtype == "bool" or out.dtype != x.dtype:
        raise ArgumentError(f"{name} needs floating-point input and output of one element type (integer input: Float64 output)")
    nd, sizes, mask, ws, wsize, _ = _dims_call(x, dims)
    _lib.check(_lib.load().mi_softmax_dims(op, x.code_f64, x.ptr, out.ptr, nd, sizes, mask, ws, wsize, _stream()))
    return out


def _float_dtype(x):
    return "f64" if x.dtype in ("i32", "i64") else x.dtype


def softmax(x, *, dims=1):
    """softmax(x; dims=1)  (src/softmax.jl:56).  ``dims=None`` is Julia's ``dims=:``."""
    if not isinstance(x, DeviceArray):
        raise _number_error("softmax")
    return softmax_(DeviceArray.empty(x.dims, _float_dtype(x)), x, dims=dims)


def softmax_(out, x=None, *, dims=1):
    """softmax!(out, x; dims=1) and softmax!(x; dims=1)  (src/softmax.jl:64-66)."""
    return _softmax_like("softmax!", _lib.MI_SOFTMAX, out, out if x is None else x, dims)


def logsoftmax(x, *, dims=1):
    """logsoftmax(x; dims=1)  (src/softmax.jl:133)."""
    if not isinstance(x, DeviceArray):
        raise _number_error("logsoftmax")
    return logsoftmax_(DeviceArray.empty(x.dims, _float_dtype(x)), x, dims=dims)


def logsoftmax_(out, x=None, *, dims=1):
    """logsoftmax!(out, x; dims=1) and logsoftmax!(x; dims=1)  (src/softmax.jl:141-143)."""
    return _softmax_like("logsoftmax!", _lib.MI_LOGSOFTMAX, out, out if x is None else x, dims)


def logsumexp(x, *, dims=None):
    """logsumexp(x; dims=:)  (src/softmax.jl:200-203).  With ``dims=None`` the result is a 0-d
    DeviceArray holding the scalar; otherwise the reduced dimensions are kept with extent 1."""
    if not isinstance(x, DeviceArray):
        raise _number_error("logsumexp")
    x = _contig(_float(x), "x")
    if x.dtype == "bool":
        raise ArgumentError("logsumexp needs a floating-point array")
    nd, sizes, mask, ws, wsize, kept = _dims_call(x, dims)
    out = DeviceArray.empty(kept, x.dtype)
    _lib.check(_lib.load().mi_logsumexp_dims(x.code_f64, x.ptr, out.ptr, nd, sizes, mask, ws, wsize, _stream()))
    return out


def grad_logsumexp(dy, x, *, dims=None, lse=None):
    """Pullback of ``logsumexp(x; dims)`` (rrule at src/softmax.jl:205-212): ``dy`` has the size of the reduced
    result; ``lse`` is that result when the caller kept it (recomputed otherwise)."""
    if not isinstance(x, DeviceArray) or not isinstance(dy, DeviceArray):
        raise _number_error("logsumexp")
    x, dy = _contig(x, "x"), _contig(dy, "dy")
    if lse is None:
        lse = logsumexp(x, dims=dims)
    lse = _contig(lse, "lse")
    nd, sizes, mask, ws, wsize, kept = _dims_call(x, dims)
    n_out = int(np.prod(kept, dtype=np.int64)) if kept else 1
    if dy.length != n_out or lse.length != n_out or not (dy.dtype == lse.dtype == x.dtype):
        raise DimensionMismatch(f"dy and lse must have the size {kept} of logsumexp(x; dims) and the element type of x")
    dx = DeviceArray.empty(x.dims, x.dtype)
    _lib.check(_lib.load().mi_logsumexp_bwd_dims(x.code_f64, dy.ptr, x.ptr, lse.ptr, dx.ptr, nd, sizes, mask, ws, wsize, _stream()))
    return dx


def _softmax_grad(name, op, dx, dy, y, dims):
    dy, y, dx = _contig(dy, "dy"), _contig(y, "y"), _contig(dx, "dx")
    if not (dy.dims == y.dims == dx.dims):
        raise DimensionMismatch(f"{name}: dx {dx.dims}, dy {dy.dims} and y {y.dims} must have one size")
    if y.dtype == "bool" or not (dy.dtype == y.dtype == dx.dtype):
        raise ArgumentError(f"{name} needs one floating-point element type for dx, dy and y")
    nd, sizes, mask, ws, wsize, _ = _dims_call(y, dims)
    _lib.check(_lib.load().mi_softmax_bwd_dims(op, y.code_f64, dy.ptr, y.ptr, dx.ptr, nd, sizes, mask, ws, wsize, _stream()))
    return dx


def grad_softmax(dy, y, *, dims=1):
    """∇softmax(dy, y; dims=1)  (src/softmax.jl:87-98): gradient of softmax given its RESULT y."""
    return _softmax_grad("∇softmax", _lib.MI_SOFTMAX, DeviceArray.empty(y.dims, y.dtype), dy, y, dims)


def grad_softmax_(dx, dy, y, *, dims=1):
    """∇softmax!(dx, dy, y; dims=1)  (src/softmax.jl:105-110)."""
    return _softmax_grad("∇softmax!", _lib.MI_SOFTMAX, dx, dy, y, dims)


def grad_logsoftmax(dy, y, *, dims=1):
    """∇logsoftmax(dy, y; dims=1)  (src/softmax.jl:155-166)."""
    return _softmax_grad("∇logsoftmax", _lib.MI_LOGSOFTMAX, DeviceArray.empty(y.dims, y.dtype), dy, y, dims)


def grad_logsoftmax_(dx, dy, y, *, dims=1):
    """∇logsoftmax!(dx, dy, y; dims=1)  (src/softmax.jl:173-177)."""
    return _softmax_grad("∇logsoftmax!", _lib.MI_LOGSOFTMAX, dx, dy, y, dims)


# ---- batched_mul ---------------------------------------------------------------------------------

def _blas_layout(X, name):
    """('N' | 'T', leading dimension, batch stride) from strides, the decision table of
    _batched_try_gemm! (src/batched/batchedmul.jl:272-294); layouts BLAS cannot address raise as
    ext/NNlibAMDGPUExt/batched_mul.jl:1-9 does."""
    s1, s2, s3 = X.strides
    if s2 == 1 and X.dims[0] > 1:
        flag, ld = b"T", s1
    elif s1 == 1:
        flag, ld = b"N", s2
    elif s2 == 1:
        flag, ld = b"T", s1
    else:
        raise ArgumentError(f"Unsupported array layout for batched mul.\n- Size: {X.dims}\n- Strides: {X.strides}")
    rows = X.dims[0] if flag == b"N" else X.dims[1]
    return flag, max(ld, rows, 1), s3


def batched_mul_(C, A, B, alpha=1.0, beta=0.0):
    """batched_mul!(C, A, B, alpha=1, beta=0)  (src/batched/batchedmul.jl:238-254)."""
    if not (C.ndim == A.ndim == B.ndim) or C.ndim < 3:
        raise DimensionMismatch("batched_mul! needs arrays of equal dimensionality (at least 3)")
    if C.ndim > 3:
        bs = C.dims[2:]
        if A.dims[2:] != bs:
            raise DimensionMismatch("batch size of A must match C")      # :246
        if B.dims[2:] != bs:
            raise DimensionMismatch("batch size of B must match C")      # :247
        C3 = C.reshape(C.dims[0], C.dims[1], -1)
        batched_mul_(C3, A.reshape(A.dims[0], A.dims[1], -1), B.reshape(B.dims[0], B.dims[1], -1), alpha, beta)
        return C
    if "bool" in (A.dtype, B.dtype, C.dtype):
        raise ArgumentError("batched_mul! needs numeric arrays")
    if A.dtype == B.dtype == C.dtype == "c64":
        return _batched_mul_complex(C, A, B, alpha, beta)
    if not (A.dtype == B.dtype == C.dtype) or A.dtype not in ("f32", "f16", "bf16", "f64"):
        # element types that differ, integers, ComplexF64: batched_mul_generic! (src/batched/batchedmul.jl:306-325)
        return _batched_mul_generic(C, A, B, alpha, beta)
    if A.dtype == "f64" and not (_is_blas_layout(A) and _is_blas_layout(B) and (C.strides[0] == 1 or C.dims[0] == 1 or C.strides[1] == 1)):
        return _batched_mul_generic(C, A, B, alpha, beta)
    nb = C.dims[2]
    if A.dims[2] not in (nb, 1):
        raise DimensionMismatch("batch size mismatch: A != C")            # src/gemm.jl:99
    if B.dims[2] not in (nb, 1):
        raise DimensionMismatch("batch size mismatch: B != C")            # src/gemm.jl:100
    m, ka = A.dims[0], A.dims[1]
    kb, n = B.dims[0], B.dims[1]
    if ka != kb or m != C.dims[0] or n != C.dims[1]:                      # src/gemm.jl:106-108
        raise DimensionMismatch(f"A1 has size ({m},{ka}), B1 has size ({kb},{n}), C1 has size {C.dims[:2]}")
    if C.strides[0] != 1 and C.strides[1] == 1 and C.dims[0] > 1:
        # C is a lazily transposed / permuted array: compute C' = B' * A' into its parent layout
        # (_batched_try_gemm!, src/batched/batchedmul.jl:268-270: "transposing C = A * B into C' = B' * A'")
        batched_mul_(batched_transpose(C), batched_transpose(B), batched_transpose(A), alpha, beta)
        return C
    tA, lda, sA = _blas_layout(A, "A")
    tB, ldb, sB = _blas_layout(B, "B")
    if C.strides[0] != 1 and C.dims[0] > 1:   # the stride of an extent-1 dimension addresses nothing
        raise ArgumentError(f"Unsupported array layout for batched mul.\n- Size: {C.dims}\n- Strides: {C.strides}")
    sA = 0 if A.dims[2] == 1 else sA                                     # src/gemm.jl:117-118
    sB = 0 if B.dims[2] == 1 else sB
    if A.dtype == "f64":     # dgemm_ in the reference (src/gemm.jl:27-32)
        _lib.check(_lib.load().mi_batched_gemm_f64(tA, tB, m, n, ka, float(alpha), A.ptr, lda, sA, B.ptr, ldb, sB, float(beta),
                                                   C.ptr, max(C.strides[1], m, 1), C.strides[2], nb, _stream()), DimensionMismatch)
        return C
    _lib.check(_lib.load().mi_batched_gemm(C.code, tA, tB, m, n, ka, float(alpha), A.ptr, lda, sA, B.ptr, ldb, sB,
                                           float(beta), C.ptr, max(C.strides[1], m, 1), C.strides[2], nb, _stream()),
               DimensionMismatch)
    return C


def _is_blas_layout(X):
    """One of the first two strides is 1 (or addresses nothing): 'N' or 'T' for a BLAS call."""
    return X.strides[0] == 1 or X.strides[1] == 1 or X.dims[0] == 1 or X.dims[1] == 1


# Julia's promote_type for the element types batched_mul meets (test/batchedmul.jl:41-73): the result of
# batched_mul(A, B) has this element type, and batched_mul_generic! computes in it.
_REAL_RANK = {"i32": 0, "i64": 1, "f16": 2, "bf16": 2, "f32": 3, "f64": 4}


def promote_type(a, b):
    if a == b:
        return a
    cplx = a in ("c64", "c128") or b in ("c64", "c128")
    ra = {"c64": "f32", "c128": "f64"}.get(a, a)
    rb = {"c64": "f32", "c128": "f64"}.get(b, b)
    if ra == rb:
        real = ra
    elif {ra, rb} == {"f16", "bf16"}:
        real = "f32"
    else:
        hi, lo = (ra, rb) if _REAL_RANK[ra] >= _REAL_RANK[rb] else (rb, ra)
        real = hi          # an integer joins any float; the wider float wins; Int32 with Int64 gives Int64
    if cplx:
        if real in ("i32", "i64"):          # Complex{Int} does not occur here: the complex side fixes the float type
            real = "f32"
        return "c128" if real == "f64" else "c64"
    return real


def _batched_mul_generic(C, A, B, alpha, beta):
    """batched_mul_generic! (src/batched/batchedmul.jl:306-325): any numeric element types and any strides; the
    arithmetic is that of C's element type, which must be what A's and B's promote to."""
    if C.conj:
        raise ArgumentError("batched_mul! cannot write into a batched_adjoint")
    want = promote_type(A.dtype, B.dtype)
    if promote_type(want, C.dtype) != C.dtype:
        raise ArgumentError(f"batched_mul!: cannot store the product of {A.dtype} and {B.dtype} arrays into a {C.dtype} array")
    if C.dtype in ("f16", "bf16"):
        # Float16 / BFloat16 times an integer array promotes to the 16-bit type (Julia's promote_type); the generic kernel
        # has no 16-bit accumulator type, so the product is formed in Float32 and rounded once into C
        if not C.is_contiguous():
            raise ArgumentError("batched_mul!: a 16-bit result of mixed element types must be a dense array")
        lib = _lib.load()
        tmp = DeviceArray.empty(C.dims, "f32")
        if beta != 0:
            _lib.check(lib.mi_convert(tmp.ptr, _lib.MI_F32, C.ptr, C.code, C.length, _stream()))
        _batched_mul_generic(tmp, A, B, alpha, beta)
        _lib.check(lib.mi_convert(C.ptr, C.code, tmp.ptr, _lib.MI_F32, C.length, _stream()))
        return C
    nb = C.dims[2]
    if A.dims[2] not in (nb, 1):
        raise DimensionMismatch("batch size mismatch: A != C")            # src/batched/batchedmul.jl:307-308
    if B.dims[2] not in (nb, 1):
        raise DimensionMismatch("batch size mismatch: B != C")
    m, ka = A.dims[0], A.dims[1]
    kb, n = B.dims[0], B.dims[1]
    if ka != kb or m != C.dims[0] or n != C.dims[1]:
        raise DimensionMismatch(f"A1 has size ({m},{ka}), B1 has size ({kb},{n}), C1 has size {C.dims[:2]}")
    al, be = complex(alpha), complex(beta)
    sA = 0 if A.dims[2] == 1 else A.strides[2]
    sB = 0 if B.dims[2] == 1 else B.strides[2]
    _lib.check(_lib.load().mi_batched_mul_generic(C.code_any, A.code_any, B.code_any, m, n, ka, al.real, al.imag,
                                                  A.ptr, A.strides[0], A.strides[1], sA, int(A.conj),
                                                  B.ptr, B.strides[0], B.strides[1], sB, int(B.conj), be.real, be.imag,
                                                  C.ptr, C.strides[0], C.strides[1], C.strides[2], nb, _stream()),
               DimensionMismatch)
    return C


def _batched_mul_complex(C, A, B, alpha, beta):
    """ComplexF32 operands: one strided kernel takes 'N', 'T', 'C' (a batched_adjoint) and every permuted
    layout of A, B and C (src/batched/batchedmul.jl:261-296 and the generic fallback :306-325)."""
    if C.conj:
        raise ArgumentError("batched_mul! cannot write into a batched_adjoint")
    nb = C.dims[2]
    if A.dims[2] not in (nb, 1):
        raise DimensionMismatch("batch size mismatch: A != C")            # src/gemm.jl:99
    if B.dims[2] not in (nb, 1):
        raise DimensionMismatch("batch size mismatch: B != C")            # src/gemm.jl:100
    m, ka = A.dims[0], A.dims[1]
    kb, n = B.dims[0], B.dims[1]
    if ka != kb or m != C.dims[0] or n != C.dims[1]:                      # src/gemm.jl:106-108
        raise DimensionMismatch(f"A1 has size ({m},{ka}), B1 has size ({kb},{n}), C1 has size {C.dims[:2]}")
    al, be = complex(alpha), complex(beta)
    sA = 0 if A.dims[2] == 1 else A.strides[2]                            # src/gemm.jl:117-118
    sB = 0 if B.dims[2] == 1 else B.strides[2]
    _lib.check(_lib.load().mi_batched_mul_c32(m, n, ka, al.real, al.imag, A.ptr, A.strides[0], A.strides[1], sA, int(A.conj),
                                              B.ptr, B.strides[0], B.strides[1], sB, int(B.conj), be.real, be.imag,
                                              C.ptr, C.strides[0], C.strides[1], C.strides[2], nb, _stream()),
               DimensionMismatch)
    return C


def _copy_if_faster(X):
    """_copy_if_faster (src/batched/batchedmul.jl:76-83) widened to every layout the GEMM kernel cannot
    address (neither of the first two strides is 1): such views are materialised; the reference would
    hand them to batched_mul_generic!, with the same result."""
    s1, s2, s3 = X.strides
    if (s3 == 1 and s1 != 1 and X.dims[2] > 1) or (s1 != 1 and s2 != 1 and X.dims[0] > 1 and X.dims[1] > 1):
        return X.copy()
    return X


def batched_mul(A, B):
    """batched_mul(A, B)  (src/batched/batchedmul.jl:47-60, 140-164): C[:,:,k...] = A[:,:,k...] * B[:,:,k...];
    a 3-D operand with batch extent 1 is shared by every batch, and so is a plain (or lazily
    transposed) matrix on either side.  Lazy views (batched_transpose, permuted) are accepted."""
    if not isinstance(A, DeviceArray) or not isinstance(B, DeviceArray):
        raise ArgumentError("batched_mul expects DeviceArrays")
    if A.ndim == 3 and B.ndim == 2:            # _semi_batched_mul, src/batched/batchedmul.jl:143-150
        return batched_mul(A, B.with_trailing(1))
    if A.ndim == 2 and B.ndim == 3:            # src/batched/batchedmul.jl:152-164
        return batched_mul(A.with_trailing(1), B)
    if A.ndim != B.ndim or A.ndim < 3:
        raise DimensionMismatch("batched_mul needs two arrays of equal dimensionality (at least 3)")
    if A.ndim > 3:
        bs = A.dims[2:]
        assert bs == B.dims[2:], "batch size has to be the same for the two arrays."   # :49
        z = batched_mul(A.reshape(A.dims[0], A.dims[1], -1), B.reshape(B.dims[0], B.dims[1], -1))
        return z.reshape((z.dims[0], z.dims[1]) + tuple(bs))
    if not (A.dims[2] == B.dims[2] or A.dims[2] == 1 or B.dims[2] == 1):
        raise DimensionMismatch("batch size mismatch: A != B")                          # :57-58
    if "bool" in (A.dtype, B.dtype):
        raise ArgumentError("batched_mul needs numeric arrays")
    T = promote_type(A.dtype, B.dtype)                         # src/batched/batchedmul.jl:65: promote_type of the eltypes
    C = DeviceArray.empty((A.dims[0], B.dims[1], max(A.dims[2], B.dims[2])), T)
    if A.dtype == B.dtype and T in ("f32", "f16", "bf16", "f64"):
        return batched_mul_(C, _copy_if_faster(A), _copy_if_faster(B))
    return batched_mul_(C, A, B)          # the complex and generic kernels address every strided layout themselves


def batched_vec(A, B):
    """batched_vec(A, B)  (src/batched/batchedmul.jl:166-218): C[:,k...] = A[:,:,k...] * B[:,k...]; a vector
    ``B`` is shared by every batch."""
    if not isinstance(A, DeviceArray) or not isinstance(B, DeviceArray):
        raise ArgumentError("batched_vec expects DeviceArrays")
    if A.ndim == 3 and B.ndim == 1:                                                    # :217-218
        return batched_mul(A, B.reshape(B.dims[0], 1, 1)).reshape(A.dims[0], A.dims[2])
    if A.ndim != B.ndim + 1:                                                           # :198-199
        raise DimensionMismatch(f"batched_vec requires ndims(A) == ndims(B) + 1, got ndims(A)={A.ndim} and ndims(B)={B.ndim}")
    if A.dims[2:] != B.dims[1:]:                                                       # :200-201
        raise DimensionMismatch(f"batch dimensions must match: size(A)[3:end]={A.dims[2:]} != size(B)[2:end]={B.dims[1:]}")
    if not B.is_contiguous():
        B = B.copy()                                                                   # :213-215: a transposed B is copied
    C = batched_mul(A, B.reshape((B.dims[0], 1) + B.dims[1:]))
    return C.reshape((C.dims[0],) + C.dims[2:])


def batched_mul_pullback(A, B, dC):
    """The pullback of ``batched_mul(A, B)`` (rrule at src/batched/batchedmul.jl:96-110):
    ``dA = dC * B'`` and ``dB = A' * dC`` per slice; an operand whose batch extent is 1 was shared by
    every slice, so its gradient is the sum over slices."""
    from .array import batched_adjoint
    if A.ndim != 3 or B.ndim != 3 or dC.ndim != 3:
        raise DimensionMismatch("batched_mul_pullback expects 3-D arrays")
    nb = dC.dims[2]

    def summed(X, make):
        if X.dims[2] != 1 or nb == 1:
            return make(None)
        # sum over slices: accumulate slice by slice into one (m, n, 1) result with beta = 1
        out = DeviceArray.zeros(X.dims, X.dtype)
        for b in range(nb):
            make((out, b))
        return out

    def slice3(X, b):
        return DeviceArray(X.storage, X.dims[:2] + (1,), X.dtype, X.strides, X.offset + (b * X.strides[2] if X.dims[2] > 1 else 0))

    def dA_of(acc):
        if acc is None:
            return batched_mul(dC, batched_adjoint(B))
        out, b = acc
        return batched_mul_(out, slice3(dC, b), batched_adjoint(slice3(B, b)), 1.0, 1.0)

    def dB_of(acc):
        if acc is None:
            return batched_mul(batched_adjoint(A), dC)
        out, b = acc
        return batched_mul_(out, batched_adjoint(slice3(A, b)), slice3(dC, b), 1.0, 1.0)

    return summed(A, dA_of), summed(B, dB_of)
