"""Julia-shaped device arrays for the Python mirror of the NNlib attention API.

A ``DeviceArray`` has a Julia ``size`` tuple and column-major memory, exactly as the arrays the
reference operates on; element ``(i1, i2, ...)`` is at ``i1 + i2*size[0] + ...``.  PyTorch is used
only as the owner of the device allocation (and for host<->device copies).
"""
import numpy as np
import torch

from . import _lib

_TORCH = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "bool": torch.uint8, "c64": torch.complex64,
          "f64": torch.float64, "c128": torch.complex128, "i32": torch.int32, "i64": torch.int64}
_CODE = {"f32": _lib.MI_F32, "f16": _lib.MI_F16, "bf16": _lib.MI_BF16}
# element type codes of the batched_mul entry points, which also take Float64, integers and complex numbers
_CODE_ANY = dict(_CODE, f64=_lib.MI_F64, c64=_lib.MI_C64, c128=_lib.MI_C128, i32=_lib.MI_I32, i64=_lib.MI_I64)
_NP = {"f32": np.float32, "f16": np.float16, "bf16": np.float32, "c64": np.complex64, "f64": np.float64, "c128": np.complex128,
       "i32": np.int32, "i64": np.int64}
# Default element type for a host array.  NumPy's default float is Float64 where the Julia code this mirrors has
# Float32 arrays: a float64 host array becomes Float32 unless dtype="f64" is asked for.  Integers and complex128 keep
# their width (complex128 -> ComplexF64: nothing is narrowed silently).
_NP2NAME = {np.dtype(np.float32): "f32", np.dtype(np.float16): "f16", np.dtype(np.bool_): "bool",
            np.dtype(np.uint8): "bool", np.dtype(np.complex64): "c64", np.dtype(np.complex128): "c128",
            np.dtype(np.int32): "i32", np.dtype(np.int64): "i64"}
COMPLEX = ("c64", "c128")


def _require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("nnlib_amd needs a GPU (torch.cuda.is_available() is False); there is no CPU path")


class DeviceArray:
    """Column-major array in device memory.

    ``dims`` is the Julia size; ``strides`` are element strides (Julia ``strides``), which lets
    ``batched_transpose`` and friends be lazy views like the reference's wrappers
    (src/batched/batchedadjtrans.jl:23-92)."""

    def __init__(self, storage, dims, dtype, strides=None, offset=0):
        self.storage = storage          # 1-D torch tensor that owns the memory
        self.dims = tuple(int(d) for d in dims)
        self.dtype = dtype              # "f32" | "f16" | "bf16" | "bool"; batched_mul also takes "f64", "i32", "i64", "c64", "c128"
        self.conj = False               # set by batched_adjoint of a complex array: elements read conjugated
        if strides is None:
            strides, acc = [], 1
            for d in self.dims:
                strides.append(acc)
                acc *= d
        self.strides = tuple(int(s) for s in strides)
        self.offset = int(offset)       # in elements

    # ---- construction --------------------------------------------------------------------
    @classmethod
    def empty(cls, dims, dtype="f32"):
        _require_gpu()
        n = int(np.prod(dims, dtype=np.int64)) if len(dims) else 1
        return cls(torch.empty(max(n, 1), dtype=_TORCH[dtype], device="cuda"), dims, dtype)

    @classmethod
    def zeros(cls, dims, dtype="f32"):
        a = cls.empty(dims, dtype)
        a.storage.zero_()
        return a

    @classmethod
    def from_numpy(cls, a, dtype=None):
        """``a`` is indexed like the Julia array (any memory order). ``dtype`` may narrow it
        ("bf16" rounds to nearest even from the array's float values)."""
        _require_gpu()
        a = np.asarray(a)
        if dtype is None:
            if a.dtype not in _NP2NAME:
                a = a.astype(np.float32)
            dtype = _NP2NAME[a.dtype]
        if dtype == "bool":
            flat = np.ascontiguousarray(a.astype(np.uint8).ravel(order="F"))
            t = torch.from_numpy(flat).cuda()
        elif dtype in ("c64", "c128", "f64", "i32", "i64"):
            t = torch.from_numpy(np.ascontiguousarray(a.astype(_NP[dtype]).ravel(order="F"))).cuda()
        else:
            src = a.astype(np.float32) if a.dtype not in (np.float32, np.float16) else a
            flat = np.ascontiguousarray(src.ravel(order="F"))
            t = torch.from_numpy(flat).cuda().to(_TORCH[dtype])
        if t.numel() == 0:
            t = torch.empty(1, dtype=_TORCH[dtype], device="cuda")
        return cls(t, a.shape, dtype)

    @classmethod
    def from_torch(cls, t, dims, dtype):
        """Wrap an existing 1-D (or contiguous) device tensor whose memory already is column-major ``dims``."""
        return cls(t.reshape(-1), dims, dtype)

    # ---- views ---------------------------------------------------------------------------
    @property
    def ndim(self):
        return len(self.dims)

    def size(self, d=None):
        return self.dims if d is None else (self.dims[d - 1] if d <= len(self.dims) else 1)

    @property
    def length(self):
        return int(np.prod(self.dims, dtype=np.int64)) if self.dims else 1

    def is_contiguous(self):
        acc = 1
        for d, s in zip(self.dims, self.strides):
            if d != 1 and s != acc:
                return False
            acc *= d
        return True

    def reshape(self, *dims):
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        if -1 in dims:
            known = int(np.prod([d for d in dims if d != -1], dtype=np.int64))
            dims = tuple(self.length // max(known, 1) if d == -1 else d for d in dims)
        assert self.is_contiguous(), "reshape needs a contiguous array"
        assert int(np.prod(dims, dtype=np.int64)) == self.length, "reshape must keep the element count"
        out = DeviceArray(self.storage, dims, self.dtype, None, self.offset)
        out.conj = self.conj
        return out

    def permuted(self, *perm):
        """Lazy ``PermutedDimsArray(A, perm)`` (1-based ``perm`` as in Julia): same memory, permuted
        size and strides."""
        if len(perm) == 1 and isinstance(perm[0], (tuple, list)):
            perm = tuple(perm[0])
        assert sorted(perm) == list(range(1, self.ndim + 1)), "perm must be a permutation of 1:ndims"
        out = DeviceArray(self.storage, [self.dims[p - 1] for p in perm], self.dtype,
                          [self.strides[p - 1] for p in perm], self.offset)
        out.conj = self.conj
        return out

    def with_trailing(self, n):
        """Same memory viewed with ``n`` extra trailing dimensions of extent 1 (``reshape(A, size(A)..., 1)``
        for views whose strides must be kept)."""
        out = DeviceArray(self.storage, self.dims + (1,) * n, self.dtype, self.strides + (self.length,) * n, self.offset)
        out.conj = self.conj
        return out

    def copy(self):
        """Dense column-major copy (``copy(X)`` / ``permutedims``): materialises a lazy view of up to 8 dims."""
        assert self.ndim <= 8, "copy of a strided view is built for up to 8 dimensions"
        out = DeviceArray.empty(self.dims, self.dtype)
        if self.ndim <= 3:
            d = self.dims + (1,) * (3 - self.ndim)
            s = self.strides + (0,) * (3 - self.ndim)
            _lib.check(_lib.load().mi_strided_copy(out.ptr, self.ptr, self.itemsize, d[0], d[1], d[2], s[0], s[1], s[2], None))
        else:
            import ctypes
            sizes, strides = (ctypes.c_int64 * self.ndim)(*self.dims), (ctypes.c_int64 * self.ndim)(*self.strides)
            _lib.check(_lib.load().mi_strided_copy_nd(out.ptr, self.ptr, self.itemsize, self.ndim, sizes, strides, None))
        if self.conj:
            out.storage.copy_(torch.conj_physical(out.storage))
        return out

    @property
    def itemsize(self):
        return self.storage.element_size()

    @property
    def ptr(self):
        return self.storage.data_ptr() + self.offset * self.itemsize

    @property
    def code(self):
        if self.dtype not in _CODE:
            raise _lib.ArgumentError(f"this operation takes Float32, Float16 or BFloat16 arrays, got {self.dtype}")
        return _CODE[self.dtype]

    @property
    def code_f64(self):
        """Element type code for the entry points that also take Float64 (the softmax family, the attention forward)."""
        if self.dtype == "f64":
            return _lib.MI_F64
        return self.code

    @property
    def code_any(self):
        """Element type code for the batched_mul entry points (every numeric element type)."""
        if self.dtype not in _CODE_ANY:
            raise _lib.ArgumentError(f"batched_mul takes numeric arrays, got {self.dtype}")
        return _CODE_ANY[self.dtype]

    # ---- host copies ---------------------------------------------------------------------
    def to_numpy(self):
        """Julia-shaped numpy array (Fortran order). bf16 comes back as float32, bool as bool."""
        if self.conj:
            plain = DeviceArray(self.storage, self.dims, self.dtype, self.strides, self.offset)
            return np.conj(plain.to_numpy())
        if not self.is_contiguous():
            return self.copy().to_numpy()
        flat = self.storage[self.offset:self.offset + self.length]
        if self.dtype == "bf16":
            flat = flat.float()
        h = flat.cpu().numpy()
        if self.dtype == "bool":
            h = h.astype(bool)
        return h.reshape(self.dims, order="F")

    def __repr__(self):
        return f"DeviceArray{{{self.dtype}}}{self.dims}"


class BatchedTranspose(DeviceArray):
    """Lazy per-slice transpose of a 3-D array (src/batched/batchedadjtrans.jl:23-52)."""

    def __init__(self, parent):
        assert parent.ndim == 3, "batched_transpose expects a 3-D array"
        d, s = parent.dims, parent.strides
        super().__init__(parent.storage, (d[1], d[0], d[2]), parent.dtype, (s[1], s[0], s[2]), parent.offset)
        self.parent = parent
        self.conj = parent.conj


def batched_transpose(A):
    """batched_transpose(A) (src/batched/batchedadjtrans.jl:37-38); transposing twice unwraps."""
    return A.parent if type(A) is BatchedTranspose else BatchedTranspose(A)


def transpose(M):
    """Lazy transpose of a matrix (Julia's ``transpose(M)`` / ``M'`` for the real element types here)."""
    assert M.ndim == 2, "transpose expects a matrix"
    return M.permuted(2, 1)


def adjoint(M):
    """Lazy conjugate transpose of a matrix (``M'``); equals ``transpose`` for the real element types."""
    out = transpose(M)
    if M.dtype in COMPLEX:
        out.conj = not M.conj
    return out


class BatchedAdjoint(BatchedTranspose):
    """Lazy per-slice conjugate transpose of a complex 3-D array (src/batched/batchedadjtrans.jl:23-52)."""

    def __init__(self, parent):
        super().__init__(parent)
        self.conj = not parent.conj


def batched_adjoint(A):
    """batched_adjoint(A) (src/batched/batchedadjtrans.jl:50-51): the per-slice conjugate transpose; for the
    real element types it equals batched_transpose.  Taking it twice unwraps."""
    if A.dtype not in COMPLEX:
        return batched_transpose(A)
    return A.parent if isinstance(A, BatchedAdjoint) else BatchedAdjoint(A)


class CausalMask:
    """What ``make_causal_mask`` returns for device arrays: the (len, len) pattern
    ``m[i, j] = i <= j`` (src/attention.jl:145) kept symbolic so that the attention kernel can
    apply it from indices instead of reading len*len bytes.  ``materialize()`` gives the dense
    Bool array the reference would have produced."""

    def __init__(self, length):
        self.length = int(length)
        self.dims = (self.length, self.length)

    def size(self, d=None):
        return self.dims if d is None else (self.dims[d - 1] if d <= 2 else 1)

    def materialize(self):
        out = DeviceArray.empty(self.dims, "bool")
        _lib.check(_lib.load().mi_make_causal_mask(out.ptr, self.length, None))
        return out

    def to_numpy(self):
        return self.materialize().to_numpy()

    def __and__(self, other):
        """``make_causal_mask(x) .& padding`` in the reference materialises the product; here the causal half stays
        symbolic and the Bool array (e.g. a key-padding mask of size (kv_len, 1, 1, batch)) rides along, so that the
        kernels apply the causal pattern from indices and read only the array."""
        if isinstance(other, CausalAnd):
            return CausalAnd(self.length, other.array)
        if not isinstance(other, DeviceArray) or other.dtype != "bool":
            raise ArgumentError("a causal mask combines with a Bool DeviceArray")
        return CausalAnd(self.length, other)

    __rand__ = __and__


class CausalAnd:
    """Elementwise AND of the causal pattern with a Bool array, kept as the pair (see CausalMask.__and__)."""

    def __init__(self, length, array):
        self.length = int(length)
        self.array = array

    def materialize(self):
        raise ArgumentError("materialise the two halves separately: CausalMask(length).materialize() and .array")
