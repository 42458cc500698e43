# NNlibMI355Ext -- makes NNlib's own generics dispatch to libmi355attn.so for MI355Attention.DeviceArray arguments.
#
# Loaded automatically when NNlib (and ChainRulesCore, which NNlib itself depends on) are in the session next to
# MI355Attention, the way NNlib's backends are wired (NNlib Project.toml:16-34, ext/NNlibAMDGPUExt/NNlibAMDGPUExt.jl).
# The same file works from inside NNlib's tree: add MI355Attention to NNlib's [weakdeps], `NNlibMI355Ext =
# "MI355Attention"` to its [extensions], and copy this file to NNlib's ext/.
#
# Only forwarding: every method hands its arguments to the MI355Attention method of the same name.
module NNlibMI355Ext

using NNlib
using ChainRulesCore
using MI355Attention
const M = MI355Attention
const DA = M.DeviceArray

# ---- attention: the overload no backend has today (src/attention.jl:40-84, 112-127, 149-153) ----------------------
NNlib.dot_product_attention(q::DA{T, N}, k::DA{T, N}, v::DA{T, N}, bias = nothing; kws...) where {T, N} =
    M.dot_product_attention(q, k, v, bias; kws...)
NNlib.dot_product_attention_scores(q::DA{T, 4}, k::DA{T, 4}, bias = nothing; kws...) where {T} =
    M.dot_product_attention_scores(q, k, bias; kws...)
NNlib.make_causal_mask(x::DA; dims::Int = 2) = M.make_causal_mask(x; dims)

# ---- batched_mul: the two backend hooks (src/batched/batchedmul.jl:256-298, ext/NNlibAMDGPUExt/batched_mul.jl:11-24)
# _batched_gemm! receives BLAS-style flags for arrays whose first stride is 1 after un-transposing: 'N', 'T', or 'C'
# (what src/batched/batchedmul.jl:268-270 passes for a BatchedAdjoint of a complex array)
_op(t::Char, X) = t == 'N' ? X : t == 'C' ? M.batched_adjoint(X) : M.batched_transpose(X)
NNlib._batched_gemm!(::Type{<:DA}, tA::Char, tB::Char, α::Number, A, B, β::Number, C) =
    M.batched_mul!(C, _op(tA, A), _op(tB, B), α, β)
# element types outside BlasFloat (Float16, BFloat16, integers) and mixed ones never reach _batched_gemm!
NNlib._batched_mul!(::Type{<:DA}, C, A, B, α::Number, β::Number) = M.batched_mul!(C, A, B, α, β)
NNlib.batched_mul(A::DA{<:Any, 3}, B::DA{<:Any, 3}) = M.batched_mul(A, B)
NNlib.batched_mul(A::DA{<:Any, 3}, B::DA{<:Any, 2}) = M.batched_mul(A, B)
NNlib.batched_mul(A::DA{<:Any, 2}, B::DA{<:Any, 3}) = M.batched_mul(A, B)
NNlib.batched_vec(A::DA, B::DA) = M.batched_vec(A, B)
NNlib.batched_transpose(A::DA{T, 3}) where {T} = M.batched_transpose(A)
NNlib.batched_adjoint(A::DA{T, 3}) where {T} = M.batched_adjoint(A)

# ---- softmax family (src/softmax.jl:56-79, 105-110, 133-147, 173-177, 200-203; hook position of
# ext/NNlibCUDACUDNNExt/softmax.jl:35-40) -----------------------------------------------------------------------------
NNlib.softmax!(out::DA{T}, x::DA{T}; dims = 1) where {T} = M.softmax!(out, x; dims)
NNlib.logsoftmax!(out::DA{T}, x::DA{T}; dims = 1) where {T} = M.logsoftmax!(out, x; dims)
NNlib.logsumexp(x::DA; dims = :) = M.logsumexp(x; dims)
NNlib.∇softmax!(dx::DA, dy::DA, y::DA; dims = 1) = M.∇softmax!(dx, dy, y; dims)
NNlib.∇logsoftmax!(dx::DA, dy::DA, y::DA; dims = 1) = M.∇logsoftmax!(dx, dy, y; dims)

# ---- dropout as fdrop (src/dropout.jl:38-53) ---------------------------------------------------------------------------
NNlib.dropout(x::DA, p::Real; dims = :, seed::Integer = 0) = M.dropout(x, p; dims, seed)

# ---- reverse mode: NNlib has no rule for attention (AD walks src/attention.jl:86-127); the fused pullback takes
# its place for device arrays.  The forward result is kept for the pullback; the library recomputes nothing. ---------
function ChainRulesCore.rrule(::typeof(NNlib.dot_product_attention), q::DA{T, 3}, k::DA{T, 3}, v::DA{T, 3}, bias = nothing;
                              mask = nothing, nheads = 1, fdrop = identity) where {T}
    stats = M.attention_stats(q, nheads)
    y, α = M.dot_product_attention(q, k, v, bias; mask, nheads, fdrop, stats)
    function attention_pullback(Δ)
        dy, dα = unthunk(Δ[1]), Δ[2]
        dq, dk, dv, dbias = M.∇dot_product_attention(dy, q, k, v, bias; y, mask, nheads, fdrop,
                                                     stats = dα isa AbstractZero ? stats : nothing,
                                                     dα = dα isa AbstractZero ? nothing : unthunk(dα))
        return (NoTangent(), dq, dk, dv, bias === nothing ? NoTangent() : dbias)
    end
    return (y, α), attention_pullback
end

function ChainRulesCore.rrule(::typeof(NNlib.batched_mul), A::DA{T, 3}, B::DA{T, 3}) where {T}
    batched_mul_pullback(Δ) = (NoTangent(), M.batched_mul_pullback(A, B, unthunk(Δ))...)
    return M.batched_mul(A, B), batched_mul_pullback
end

end # module
