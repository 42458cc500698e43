"""ctypes binding of ``libmi355attn.so`` (the C ABI declared in ``include/mi355attn.h``).

There is no fallback: if the shared library is missing, importing the ops raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI355ATTN_LIB overrides the in-tree build (e.g. to load a library built with other flags)
LIB_PATH = os.environ.get("MI355ATTN_LIB") or os.path.normpath(os.path.join(_HERE, "..", "lib", "libmi355attn.so"))

MI_OK, MI_EINVAL, MI_EDTYPE, MI_ESHAPE, MI_EHIP, MI_ENOMEM, MI_EWORKSPACE = range(7)
MI_F32, MI_F16, MI_BF16, MI_F64, MI_C64, MI_C128, MI_I32, MI_I64 = range(8)
KERNEL_GENERIC, KERNEL_FLASH16, KERNEL_FLASH32, KERNEL_DECODE = 0, 1, 2, 3
KERNEL_NAMES = {0: "generic", 1: "flash16", 2: "flash32", 3: "decode"}
MI_ATTN_FORCE_GENERIC = 1
MI_ATTN_STATIC_WORKSPACE_BYTES = 32 << 20
MI_SOFTMAX, MI_LOGSOFTMAX = 0, 1

c_i32, c_i64, c_u64, c_f32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float
c_vp, c_sz = ctypes.c_void_p, ctypes.c_size_t


class mi_attn_desc(ctypes.Structure):
    _fields_ = [
        ("struct_size", c_i32), ("dtype", c_i32), ("weights_dtype", c_i32), ("causal", c_i32),
        ("flags", ctypes.c_uint32), ("reserved", c_i32),
        ("E", c_i64), ("Ev", c_i64), ("Lq", c_i64), ("Lkv", c_i64), ("H", c_i64), ("B", c_i64),
        ("q", c_vp), ("k", c_vp), ("v", c_vp), ("out", c_vp), ("weights", c_vp),
        ("bias", c_vp), ("bias_strides", c_i64 * 4),
        ("mask", c_vp), ("mask_strides", c_i64 * 4),
        ("workspace", c_vp), ("workspace_bytes", c_sz),
        ("dropout_p", c_f32), ("reserved2", ctypes.c_uint32), ("dropout_seed", c_u64),
        ("stats", c_vp),
    ]


class mi_attn_bwd_desc(ctypes.Structure):
    _fields_ = [
        ("struct_size", c_i32), ("reserved", c_i32), ("fwd", mi_attn_desc),
        ("dout", c_vp), ("dweights", c_vp), ("dq", c_vp), ("dk", c_vp), ("dv", c_vp), ("dbias", c_vp),
        ("workspace", c_vp), ("workspace_bytes", c_sz),
    ]


# name -> (restype, argtypes); every symbol include/mi355attn.h declares
SIGNATURES = {
    "mi_version": (c_i32, []),
    "mi_last_error_string": (ctypes.c_char_p, []),
    "mi_init": (c_i32, [c_i32]),
    "mi_device_count": (c_i32, [ctypes.POINTER(c_i32)]),
    "mi_device_name": (c_i32, [ctypes.c_char_p, c_sz]),
    "mi_malloc": (c_i32, [ctypes.POINTER(c_vp), c_sz]),
    "mi_free": (c_i32, [c_vp]),
    "mi_memcpy_h2d": (c_i32, [c_vp, c_vp, c_sz, c_vp]),
    "mi_memcpy_d2h": (c_i32, [c_vp, c_vp, c_sz, c_vp]),
    "mi_memcpy_d2d": (c_i32, [c_vp, c_vp, c_sz, c_vp]),
    "mi_fill_zero": (c_i32, [c_vp, c_sz, c_vp]),
    "mi_stream_create": (c_i32, [ctypes.POINTER(c_vp)]),
    "mi_stream_destroy": (c_i32, [c_vp]),
    "mi_stream_sync": (c_i32, [c_vp]),
    "mi_device_sync": (c_i32, []),
    "mi_event_create": (c_i32, [ctypes.POINTER(c_vp)]),
    "mi_event_destroy": (c_i32, [c_vp]),
    "mi_event_record": (c_i32, [c_vp, c_vp]),
    "mi_event_sync": (c_i32, [c_vp]),
    "mi_event_elapsed_ms": (c_i32, [c_vp, c_vp, ctypes.POINTER(c_f32)]),
    "mi_attention_plan": (c_i32, [ctypes.POINTER(mi_attn_desc), ctypes.POINTER(c_i32), ctypes.POINTER(c_sz)]),
    "mi_attention_workspace_size": (c_i32, [ctypes.POINTER(mi_attn_desc), ctypes.POINTER(c_sz)]),
    "mi_attention_fwd": (c_i32, [ctypes.POINTER(mi_attn_desc), c_vp]),
    "mi_attention_fwd_static": (c_i32, [ctypes.POINTER(mi_attn_desc), c_vp]),
    "mi_attention_stats_size": (c_i32, [ctypes.POINTER(mi_attn_desc), ctypes.POINTER(c_sz)]),
    "mi_attention_bwd_plan": (c_i32, [ctypes.POINTER(mi_attn_bwd_desc), ctypes.POINTER(c_i32), ctypes.POINTER(c_sz)]),
    "mi_attention_bwd": (c_i32, [ctypes.POINTER(mi_attn_bwd_desc), c_vp]),
    "mi_make_causal_mask": (c_i32, [c_vp, c_i64, c_vp]),
    "mi_dropout": (c_i32, [c_i32, c_vp, c_vp, c_i64, c_f32, c_u64, c_vp]),
    "mi_softmax_dim1": (c_i32, [c_i32, c_vp, c_vp, c_i64, c_i64, c_vp]),
    "mi_softmax": (c_i32, [c_i32, c_i32, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "mi_logsumexp": (c_i32, [c_i32, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "mi_softmax_bwd": (c_i32, [c_i32, c_i32, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "mi_softmax_dims_workspace": (c_i32, [c_i32, c_i32, ctypes.POINTER(c_i64), ctypes.c_uint32, ctypes.POINTER(c_sz)]),
    "mi_softmax_dims": (c_i32, [c_i32, c_i32, c_vp, c_vp, c_i32, ctypes.POINTER(c_i64), ctypes.c_uint32, c_vp, c_sz, c_vp]),
    "mi_logsumexp_dims": (c_i32, [c_i32, c_vp, c_vp, c_i32, ctypes.POINTER(c_i64), ctypes.c_uint32, c_vp, c_sz, c_vp]),
    "mi_softmax_bwd_dims": (c_i32, [c_i32, c_i32, c_vp, c_vp, c_vp, c_i32, ctypes.POINTER(c_i64), ctypes.c_uint32, c_vp, c_sz, c_vp]),
    "mi_logsumexp_bwd_dims": (c_i32, [c_i32, c_vp, c_vp, c_vp, c_vp, c_i32, ctypes.POINTER(c_i64), ctypes.c_uint32, c_vp, c_sz, c_vp]),
    "mi_batched_gemm": (c_i32, [c_i32, ctypes.c_char, ctypes.c_char, c_i64, c_i64, c_i64, c_f32, c_vp, c_i64, c_i64,
                                c_vp, c_i64, c_i64, c_f32, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "mi_dropout_dims": (c_i32, [c_i32, c_vp, c_vp, c_i32, ctypes.POINTER(c_i64), ctypes.c_uint32, c_f32, c_u64, c_vp]),
    "mi_logsumexp_bwd": (c_i32, [c_i32, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "mi_batched_gemm_f64": (c_i32, [ctypes.c_char, ctypes.c_char, c_i64, c_i64, c_i64, ctypes.c_double, c_vp, c_i64, c_i64,
                                    c_vp, c_i64, c_i64, ctypes.c_double, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "mi_batched_mul_generic": (c_i32, [c_i32, c_i32, c_i32, c_i64, c_i64, c_i64, ctypes.c_double, ctypes.c_double, c_vp, c_i64, c_i64, c_i64,
                                       c_i32, c_vp, c_i64, c_i64, c_i64, c_i32, ctypes.c_double, ctypes.c_double, c_vp, c_i64, c_i64,
                                       c_i64, c_i64, c_vp]),
    "mi_batched_mul_c32": (c_i32, [c_i64, c_i64, c_i64, c_f32, c_f32, c_vp, c_i64, c_i64, c_i64, c_i32, c_vp, c_i64, c_i64, c_i64,
                                   c_i32, c_f32, c_f32, c_vp, c_i64, c_i64, c_i64, c_i64, c_vp]),
    "mi_strided_copy": (c_i32, [c_vp, c_vp, c_i32, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_vp]),
    "mi_strided_copy_nd": (c_i32, [c_vp, c_vp, c_i32, c_i32, ctypes.POINTER(c_i64), ctypes.POINTER(c_i64), c_vp]),
    "mi_randn_fill": (c_i32, [c_vp, c_i32, c_i64, c_u64, c_u64, c_f32, c_vp]),
    "mi_bernoulli_fill": (c_i32, [c_vp, c_i64, c_u64, c_u64, c_f32, c_vp]),
    "mi_convert": (c_i32, [c_vp, c_i32, c_vp, c_i32, c_i64, c_vp]),
}


class MIError(RuntimeError):
    """A non-zero status from the library that has no closer reference exception."""

    def __init__(self, code, msg):
        super().__init__(f"mi355attn status {code}: {msg}")
        self.code = code


class ArgumentError(ValueError):
    """Mirror of Julia's ArgumentError, thrown by the reference at src/attention.jl:42,55-78."""


class DimensionMismatch(ValueError):
    """Mirror of Julia's DimensionMismatch, thrown by the reference at src/batched/batchedmul.jl:57-58."""


_lib = None


def load():
    """Load the shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C nnlib.jl_amd/csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no CPU fallback.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def last_error():
    return load().mi_last_error_string().decode("utf-8", "replace")


def check(rc, shape_exc=ArgumentError):
    """Map a status code onto the exception the reference would raise for the same condition."""
    if rc == MI_OK:
        return
    msg = last_error()
    if rc == MI_ESHAPE:
        raise shape_exc(msg)
    if rc in (MI_EINVAL, MI_EDTYPE):
        raise ArgumentError(msg)
    if rc == MI_ENOMEM:
        raise MemoryError(msg)
    raise MIError(rc, msg)
