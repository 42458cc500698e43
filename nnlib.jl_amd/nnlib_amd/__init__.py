"""Python mirror of NNlib.jl's attention-path operators on MI355X (gfx950).

Host-side stand-in for the Julia module: same operator names and semantics, column-major
Julia-shaped arrays, all computation behind the C ABI of ``libmi355attn.so``.
"""
from . import _lib
from ._lib import ArgumentError, DimensionMismatch, MIError
from .array import BatchedAdjoint, BatchedTranspose, CausalAnd, CausalMask, DeviceArray, adjoint, batched_adjoint, batched_transpose, transpose
from .ops import (Dropout, dropout, identity, batched_vec, batched_mul, batched_mul_, batched_mul_pullback, dot_product_attention, dot_product_attention_grad,
                  last_attention_bwd_kernel, dot_product_attention_scores, grad_logsoftmax, grad_logsumexp,
                  grad_logsoftmax_, grad_softmax, grad_softmax_, last_attention_kernel, last_attention_workspace, logsoftmax, logsoftmax_,
                  logsumexp, make_causal_mask, softmax, softmax_)

__all__ = ["identity", "grad_logsumexp", "BatchedAdjoint", "ArgumentError", "DimensionMismatch", "MIError", "DeviceArray", "BatchedTranspose", "CausalMask", "CausalAnd",
           "batched_adjoint", "batched_transpose", "batched_mul", "batched_mul_", "dot_product_attention",
           "dot_product_attention_scores", "last_attention_kernel", "last_attention_workspace", "make_causal_mask", "softmax", "softmax_",
           "logsoftmax", "logsoftmax_", "logsumexp", "grad_softmax", "grad_softmax_", "grad_logsoftmax",
           "grad_logsoftmax_", "batched_mul_pullback", "dot_product_attention_grad", "last_attention_bwd_kernel", "Dropout", "dropout", "batched_vec", "transpose", "adjoint"]
