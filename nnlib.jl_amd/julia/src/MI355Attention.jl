# MI355Attention.jl -- Julia host side of the MI355X attention library.
#
# Thin marshalling layer over the C ABI of libmi355attn.so (include/mi355attn.h).  It owns a
# column-major device array type and defines, for that type, the operators NNlib.jl exports for
# the attention path, with NNlib's signatures, return values and exception types:
#
#   dot_product_attention(q, k, v, [bias]; fdrop, mask, nheads)   NNlib src/attention.jl:40-84
#   dot_product_attention_scores(q, k, [bias]; fdrop, mask)        NNlib src/attention.jl:112-127
#   make_causal_mask(x; dims)                                      NNlib src/attention.jl:149-153
#   softmax(x; dims), softmax!(out, x; dims)                       NNlib src/softmax.jl:56-66
#   logsoftmax, logsoftmax!, logsumexp                             NNlib src/softmax.jl:133-147,200-203
#   ∇softmax, ∇softmax!, ∇logsoftmax, ∇logsoftmax!                 NNlib src/softmax.jl:87-110,155-177
#   batched_mul(A, B), batched_mul!(C, A, B, alpha, beta)          NNlib src/batched/batchedmul.jl:47-60,238-254
#   batched_transpose, batched_adjoint (ComplexF32: BatchedAdjoint) NNlib src/batched/batchedadjtrans.jl:37-52
#   batched_vec, matrix x 3-array forms of batched_mul             NNlib src/batched/batchedmul.jl:140-218
#   Dropout(p, seed) as fdrop, dropout(x, p)                       NNlib src/dropout.jl:38-53
#   ∇dot_product_attention, batched_mul_pullback                   what AD derives from src/attention.jl:86-127
#
# All arithmetic AND all planning (kernel choice, workspace sizes, recomputing a forward result the caller did not
# keep, permuting for reductions over dimensions that are not neighbours, element type promotion of mixed products)
# happen in the library: every function below checks sizes the way NNlib does, allocates outputs and workspace, and
# makes one ccall.  ext/NNlibMI355Ext.jl forwards NNlib's own generics to these methods when NNlib is loaded.
# This file has not been executed in the build environment (no Julia toolchain there); the Python mirror in
# nnlib_amd/ exercises the same entry points.
module MI355Attention

export DeviceArray, CausalMask, CausalAnd, dot_product_attention, dot_product_attention_scores, make_causal_mask,
       softmax, softmax!, logsoftmax, logsoftmax!, logsumexp, ∇logsumexp, ∇softmax, ∇softmax!, ∇logsoftmax, ∇logsoftmax!,
       batched_mul, batched_mul!, batched_vec, batched_transpose, batched_adjoint, batched_mul_pullback,
       Dropout, dropout, ∇dot_product_attention

const libmi = get(ENV, "MI355ATTN_LIB", joinpath(@__DIR__, "..", "..", "lib", "libmi355attn.so"))

# ---- status codes and element types (include/mi355attn.h) ----------------------------------------
const MI_OK, MI_EINVAL, MI_EDTYPE, MI_ESHAPE, MI_EHIP, MI_ENOMEM, MI_EWORKSPACE = Int32.(0:6)
const MI_F32, MI_F16, MI_BF16, MI_F64, MI_C64, MI_C128, MI_I32, MI_I64 = Int32.(0:7)

primitive type BFloat16 <: AbstractFloat 16 end     # storage only; use BFloat16s.jl for arithmetic
const MIFloat = Union{Float32, Float16, BFloat16}
dtype_code(::Type{Float32}) = MI_F32
dtype_code(::Type{Float16}) = MI_F16
dtype_code(::Type{BFloat16}) = MI_BF16
# element types only batched_mul takes
dtype_code(::Type{Float64}) = MI_F64
dtype_code(::Type{ComplexF32}) = MI_C64
dtype_code(::Type{ComplexF64}) = MI_C128
dtype_code(::Type{Int32}) = MI_I32
dtype_code(::Type{Int64}) = MI_I64
const MINumber = Union{MIFloat, Float64, ComplexF32, ComplexF64, Int32, Int64}
# the softmax family and the attention forward call also take Float64 (test/softmax.jl:4-29, test/attention.jl:17-34)
const MIFloat64 = Union{MIFloat, Float64}

last_error() = unsafe_string(ccall((:mi_last_error_string, libmi), Cstring, ()))

# Status -> the exception NNlib raises for the same condition (src/attention.jl:42,55-78 throw
# ArgumentError; src/batched/batchedmul.jl:57-58 and src/gemm.jl:106-108 throw DimensionMismatch).
function check(rc::Int32; shape_error = ArgumentError)
    rc == MI_OK && return nothing
    msg = last_error()
    rc == MI_ESHAPE && throw(shape_error(msg))
    (rc == MI_EINVAL || rc == MI_EDTYPE) && throw(ArgumentError(msg))
    rc == MI_ENOMEM && throw(OutOfMemoryError())
    error("mi355attn status $rc: $msg")
end

__init__() = check(ccall((:mi_init, libmi), Int32, (Int32,), Int32(0)))

# ---- device arrays ---------------------------------------------------------------------------------
# Column-major, like Array.  `strides` lets batched_transpose be a lazy view, as NNlib's
# BatchedTranspose is (src/batched/batchedadjtrans.jl:23-27).
mutable struct DeviceArray{T, N} <: AbstractArray{T, N}
    ptr::Ptr{Cvoid}
    dims::NTuple{N, Int}
    strides::NTuple{N, Int}
    owner::Any                      # `nothing` if this object owns ptr, else the parent array
    function DeviceArray{T, N}(ptr, dims, strides, owner) where {T, N}
        a = new{T, N}(ptr, dims, strides, owner)
        owner === nothing && finalizer(free!, a)
        a
    end
end

dense_strides(dims) = ntuple(i -> prod(dims[1:i-1]; init = 1), length(dims))

function DeviceArray{T}(::UndefInitializer, dims::Vararg{Int, N}) where {T, N}
    p = Ref{Ptr{Cvoid}}(C_NULL)
    check(ccall((:mi_malloc, libmi), Int32, (Ptr{Ptr{Cvoid}}, Csize_t), p, max(prod(dims), 1) * sizeof(T)))
    DeviceArray{T, N}(p[], dims, dense_strides(dims), nothing)
end
DeviceArray{T}(u::UndefInitializer, dims::Tuple) where {T} = DeviceArray{T}(u, dims...)

function free!(a::DeviceArray)
    # mi_free is hipFree: it may block until the device is idle, which is acceptable at GC time
    a.ptr == C_NULL || ccall((:mi_free, libmi), Int32, (Ptr{Cvoid},), a.ptr)
    a.ptr = C_NULL
    nothing
end

function DeviceArray(h::Array{T, N}) where {T <: Union{MINumber, Bool}, N}
    d = DeviceArray{T}(undef, size(h)...)
    check(ccall((:mi_memcpy_h2d, libmi), Int32, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), d.ptr, h, sizeof(h), C_NULL))
    d
end

function Base.Array(d::DeviceArray{T, N}) where {T, N}
    is_dense(d) || throw(ArgumentError("materialise a lazy transpose before copying to the host"))
    h = Array{T, N}(undef, d.dims)
    check(ccall((:mi_memcpy_d2h, libmi), Int32, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), h, d.ptr, sizeof(h), C_NULL))
    h
end

Base.size(a::DeviceArray) = a.dims
Base.strides(a::DeviceArray) = a.strides
Base.elsize(::Type{<:DeviceArray{T}}) where {T} = sizeof(T)
Base.unsafe_convert(::Type{Ptr{T}}, a::DeviceArray{T}) where {T} = convert(Ptr{T}, a.ptr)
Base.similar(a::DeviceArray, ::Type{T}, dims::Dims) where {T} = DeviceArray{T}(undef, dims...)
Base.getindex(::DeviceArray, I...) = error("scalar indexing of a DeviceArray is not supported; copy with Array(x)")
is_dense(a::DeviceArray) = a.strides == dense_strides(a.dims)

function Base.reshape(a::DeviceArray{T}, dims::Dims{N}) where {T, N}
    is_dense(a) || throw(ArgumentError("reshape needs a dense array"))
    prod(dims) == length(a) || throw(DimensionMismatch("new dimensions $dims must be consistent with array size $(length(a))"))
    DeviceArray{T, N}(a.ptr, dims, dense_strides(dims), a)
end

batched_transpose(a::DeviceArray{T, 3}) where {T} =
    DeviceArray{T, 3}(a.ptr, (a.dims[2], a.dims[1], a.dims[3]), (a.strides[2], a.strides[1], a.strides[3]), a)
batched_adjoint(a::DeviceArray{<:Real, 3}) = batched_transpose(a)

# Complex arrays: the per-slice conjugate transpose is a wrapper, outermost as in the reference
# (src/batched/batchedadjtrans.jl:23-52, src/batched/batchedmul.jl:234); the kernel reads it conjugated.
struct BatchedAdjoint{T <: Complex} <: AbstractArray{T, 3}
    parent::DeviceArray{T, 3}
end
batched_adjoint(a::DeviceArray{T, 3}) where {T <: Complex} = BatchedAdjoint{T}(a)
batched_adjoint(a::BatchedAdjoint) = a.parent
Base.size(a::BatchedAdjoint) = (size(a.parent, 2), size(a.parent, 1), size(a.parent, 3))
Base.getindex(::BatchedAdjoint, I...) = error("scalar indexing of a device array is not supported")

# ---- masks -----------------------------------------------------------------------------------------
# make_causal_mask on a device array returns this lazy stand-in for triu(trues(len, len)); the kernel
# applies m[i, j] = i <= j (src/attention.jl:145) from indices.  collect(m) gives the dense Bool matrix.
struct CausalMask <: AbstractMatrix{Bool}
    len::Int
end
Base.size(m::CausalMask) = (m.len, m.len)
Base.getindex(m::CausalMask, i::Int, j::Int) = i <= j
make_causal_mask(x::DeviceArray; dims::Int = 2) = CausalMask(size(x, dims))

# `make_causal_mask(x) .& padding` (a causal language model on a padded batch): the reference materialises the
# product; here the causal half stays symbolic and the Bool array rides along, so that the kernels apply the causal
# pattern from indices and read only the array (a key-padding mask of size (kv_len, 1, 1, batch) is then measured on
# the device and becomes per-sequence context lengths).
struct CausalAnd
    len::Int
    array::DeviceArray{Bool}
end
Base.Broadcast.broadcasted(::typeof(&), m::CausalMask, a::DeviceArray{Bool}) = CausalAnd(m.len, a)
Base.Broadcast.broadcasted(::typeof(&), a::DeviceArray{Bool}, m::CausalMask) = CausalAnd(m.len, a)
Base.Broadcast.materialize(m::CausalAnd) = m      # `.&` calls materialize on what broadcasted returned

# ---- attention -------------------------------------------------------------------------------------
# Mirror of `mi_attn_desc` (include/mi355attn.h); field order and sizes must match the header.
struct AttnDesc
    struct_size::Int32; dtype::Int32; weights_dtype::Int32; causal::Int32; flags::UInt32; reserved::Int32
    E::Int64; Ev::Int64; Lq::Int64; Lkv::Int64; H::Int64; B::Int64
    q::Ptr{Cvoid}; k::Ptr{Cvoid}; v::Ptr{Cvoid}; out::Ptr{Cvoid}; weights::Ptr{Cvoid}
    bias::Ptr{Cvoid}; bias_strides::NTuple{4, Int64}
    mask::Ptr{Cvoid}; mask_strides::NTuple{4, Int64}
    workspace::Ptr{Cvoid}; workspace_bytes::Csize_t
    dropout_p::Float32; reserved2::UInt32; dropout_seed::UInt64
    stats::Ptr{Cvoid}
end

# Mirror of `mi_attn_bwd_desc`.
struct AttnBwdDesc
    struct_size::Int32; reserved::Int32
    fwd::AttnDesc
    dout::Ptr{Cvoid}; dweights::Ptr{Cvoid}; dq::Ptr{Cvoid}; dk::Ptr{Cvoid}; dv::Ptr{Cvoid}; dbias::Ptr{Cvoid}
    workspace::Ptr{Cvoid}; workspace_bytes::Csize_t
end

# fdrop = Dropout(p, seed): NNlib's `x -> dropout(x, p)` (src/dropout.jl:38-53) with a reproducible
# counter-based stream.  dot_product_attention applies it inside the attention kernel; called on an
# array it runs the standalone kernel, with the same keep decisions for the same seed.
struct Dropout
    p::Float32
    seed::UInt64
    function Dropout(p::Real, seed::Integer = 0)
        0 <= p <= 1 || throw(ArgumentError("dropout expects a probability 0 <= p <= 1"))
        new(Float32(p), UInt64(seed))
    end
end
(d::Dropout)(x::DeviceArray) = dropout(x, d.p; seed = d.seed)
function dropout(x::DeviceArray{T, N}, p::Real; seed::Integer = 0, dims = :) where {T <: MIFloat, N}
    0 <= p <= 1 || throw(ArgumentError("dropout expects a probability 0 <= p <= 1"))
    is_dense(x) || throw(ArgumentError("dropout needs a dense array"))
    y = similar(x, T, size(x))
    if dims isa Colon
        GC.@preserve x y check(ccall((:mi_dropout, libmi), Int32, (Int32, Ptr{Cvoid}, Ptr{Cvoid}, Int64, Float32, UInt64, Ptr{Cvoid}),
                                     dtype_code(T), x.ptr, y.ptr, length(x), Float32(p), UInt64(seed), C_NULL))
    else
        # one decision per index along dims, shared along the other dimensions (src/dropout.jl:38-53)
        N <= 8 || throw(ArgumentError("dropout along dims takes arrays of up to 8 dimensions"))
        mask = UInt32(sum(d -> 1 << (d - 1), filter(d -> d <= N, collect(dims)); init = 0))
        sizes = collect(Int64, size(x))
        GC.@preserve x y sizes check(ccall((:mi_dropout_dims, libmi), Int32,
                                           (Int32, Ptr{Cvoid}, Ptr{Cvoid}, Int32, Ptr{Int64}, UInt32, Float32, UInt64, Ptr{Cvoid}),
                                           dtype_code(T), x.ptr, y.ptr, Int32(N), sizes, mask, Float32(p), UInt64(seed), C_NULL))
    end
    y
end

# element strides of x against the (kv, q, head, batch) score tensor; 0 where x has extent 1
function broadcast_strides(x::DeviceArray, target::NTuple{4, Int}, what)
    ntuple(4) do i
        d = i <= ndims(x) ? size(x, i) : 1
        d == 1 ? Int64(0) : d == target[i] ? Int64(strides(x)[i]) :
            throw(DimensionMismatch("arrays could not be broadcast to a common size: $what has size $(size(x)), attention scores have size $target"))
    end
end

# (causal flag, mask pointer + strides, bias pointer + strides) of a call
function mask_and_bias(::Type{T}, bias, mask, target::NTuple{4, Int}) where {T}
    Lkv, Lq = target[1], target[2]
    causal, mptr, mstr = Int32(0), C_NULL, ntuple(_ -> Int64(0), 4)
    if mask isa CausalMask || mask isa CausalAnd
        (mask.len == Lkv == Lq) || throw(DimensionMismatch("arrays could not be broadcast to a common size: mask has size $((mask.len, mask.len)), attention scores have size $target"))
        causal = Int32(1)
        mask = mask isa CausalAnd ? mask.array : nothing      # causal .& array: the flag and the array together
    end
    if mask !== nothing
        mask isa DeviceArray{Bool} || throw(ArgumentError("mask must be a Bool DeviceArray or a CausalMask"))
        mptr, mstr = mask.ptr, broadcast_strides(mask, target, "mask")
    end
    bptr, bstr = C_NULL, ntuple(_ -> Int64(0), 4)
    if bias !== nothing
        bias isa DeviceArray{T} || throw(ArgumentError("bias must be a DeviceArray with the element type of q"))
        bptr, bstr = bias.ptr, broadcast_strides(bias, target, "bias")
    end
    causal, mptr, mstr, bptr, bstr
end

# `stats`: nothing, or a Float32 DeviceArray of mi_attention_stats_size bytes that receives the softmax
# row statistics for ∇dot_product_attention (written by the MFMA flash kernels, with or without bias, mask and dropout)
function attention_call(q::DeviceArray{T, 3}, k::DeviceArray{T, 3}, v, bias, mask, H::Int; want_out::Bool,
                        want_weights::Bool, fdrop::Union{Nothing, Dropout} = nothing, stats = nothing) where {T <: MIFloat64}
    E, Lq, B = size(q); Lkv = size(k, 2); Ev = v === nothing ? E : size(v, 1)
    causal, mptr, mstr, bptr, bstr = mask_and_bias(T, bias, mask, (Lkv, Lq, H, B))
    out = want_out ? DeviceArray{T}(undef, Ev, Lq, B) : nothing
    alpha = want_weights ? DeviceArray{T}(undef, Lkv, Lq, H, B) : nothing
    p, seed = fdrop === nothing ? (0f0, UInt64(0)) : (fdrop.p, fdrop.seed)
    mk(ws, wsbytes) = AttnDesc(Int32(sizeof(AttnDesc)), dtype_code(T), dtype_code(T), causal, UInt32(0), Int32(0),
                               E, Ev, Lq, Lkv, H, B, q.ptr, k.ptr, v === nothing ? C_NULL : v.ptr,
                               out === nothing ? C_NULL : out.ptr, alpha === nothing ? C_NULL : alpha.ptr,
                               bptr, bstr, mptr, mstr, ws, wsbytes, p, UInt32(0), seed, stats === nothing ? C_NULL : stats.ptr)
    need = Ref{Csize_t}(0)
    check(ccall((:mi_attention_workspace_size, libmi), Int32, (Ref{AttnDesc}, Ptr{Csize_t}), mk(C_NULL, 0), need))
    ws = need[] > 0 ? DeviceArray{UInt8}(undef, Int(need[])) : nothing
    GC.@preserve q k v bias mask out alpha ws stats begin
        check(ccall((:mi_attention_fwd, libmi), Int32, (Ref{AttnDesc}, Ptr{Cvoid}),
                    mk(ws === nothing ? C_NULL : ws.ptr, need[]), C_NULL))
    end
    out, alpha
end

function dot_product_attention(q::DeviceArray{T, N}, k::DeviceArray{T, N}, v::DeviceArray{T, N}, args...; kws...) where {T, N}
    batch_size = size(q)[3:end]
    batch_size == size(k)[3:end] == size(v)[3:end] || throw(ArgumentError("Batch dimensions have to be the same."))
    q, k, v = map(x -> reshape(x, (size(x, 1), size(x, 2), prod(size(x)[3:end]; init = 1))), (q, k, v))
    x, α = dot_product_attention(q, k, v, args...; kws...)
    x = reshape(x, (size(x, 1), size(x, 2), batch_size...))
    α === nothing || (α = reshape(α, (size(α)[1:3]..., batch_size...)))
    return x, α
end

# attention_stats(q, nheads): buffer for the `stats` keyword of dot_product_attention (forward, written)
# and ∇dot_product_attention (backward, read): saves the gradient its own pass over the keys
function attention_stats(q::DeviceArray{T, 3}, nheads::Int) where {T}
    DeviceArray{Float32}(undef, 3 * size(q, 3) * nheads * (cld(size(q, 2), 128) * 128))
end

# `return_weights = false` is this library's one addition: it skips materialising α and returns
# `nothing` in its place (the reference always returns α).
function dot_product_attention(q::DeviceArray{T, 3}, k::DeviceArray{T, 3}, v::DeviceArray{T, 3}, bias = nothing;
                               fdrop = identity, mask = nothing, nheads = 1, return_weights = true, stats = nothing) where {T <: MIFloat64}
    all(size.((q, k, v), 1) .% nheads .== 0) || throw(ArgumentError("First dimension in query, key and value must be divisible by `nheads`.\nInstead:\n- size(q): $(size(q))\n- size(k): $(size(k))\n- size(v): $(size(v))\n- nheads: $nheads"))
    size(q, 3) == size(k, 3) == size(v, 3) || throw(ArgumentError("Batch dimensions have to be the same. Instead:\n- size(q): $(size(q))\n- size(k): $(size(k))\n- size(v): $(size(v))"))
    size(q, 1) == size(k, 1) || throw(ArgumentError("First dimension in query and key has to be the same. Instead:\n- size(q): $(size(q))\n- size(k): $(size(k))"))
    size(k, 2) == size(v, 2) || throw(ArgumentError("Second dimension in key and value has to be the same. Instead:\n- size(k): $(size(k))\n- size(v): $(size(v))"))
    if fdrop === identity || fdrop isa Dropout
        return attention_call(q, k, v, bias, mask, nheads; want_out = true, want_weights = return_weights,
                              fdrop = fdrop isa Dropout ? fdrop : nothing, stats)
    end
    # any other fdrop acts on the weights the caller sees (src/attention.jl:126): scores -> fdrop -> PV
    _, α = attention_call(q, k, nothing, bias, mask, nheads; want_out = false, want_weights = true)
    α = fdrop(α)
    return weights_times_values(α, v, nheads), α
end

function dot_product_attention_scores(q::DeviceArray{T, 4}, k::DeviceArray{T, 4}, bias = nothing;
                                      fdrop = identity, mask = nothing) where {T <: MIFloat64}
    D, H, Lq, B = size(q)
    (size(k, 1), size(k, 2), size(k, 4)) == (D, H, B) || throw(DimensionMismatch("query $(size(q)) and key $(size(k)) disagree in feature, head or batch size"))
    _, α = attention_call(reshape(q, (D * H, Lq, B)), reshape(k, (D * H, size(k, 3), B)), nothing, bias, mask, H;
                          want_out = false, want_weights = true, fdrop = fdrop isa Dropout ? fdrop : nothing)
    return fdrop isa Dropout ? α : fdrop(α)
end

# Pullback of dot_product_attention(q, k, v, bias; fdrop, mask, nheads) for fdrop = identity or the
# Dropout(p, seed) the forward call got (the keep decisions repeat): returns (dq, dk, dv, dbias) for the
# cotangent dy of the output (and optionally dα of the returned weights).
# NNlib gets these from AD through src/attention.jl:86-127 (rrule of batched_mul,
# src/batched/batchedmul.jl:96-110; _∇softmax!, src/softmax.jl:107-110; the pullback of dropout
# multiplies by the mask it drew, src/dropout.jl:38-53).  `y` is the forward result, which the MFMA kernels
# need; without it (and without dα) the library recomputes it where those kernels can take the gradient.
# A ChainRulesCore.rrule for DeviceArray arguments is three lines
# on top of this function: call the forward, close over (q, k, v, bias, y), return this pullback.
function ∇dot_product_attention(dy::DeviceArray{T, 3}, q::DeviceArray{T, 3}, k::DeviceArray{T, 3}, v::DeviceArray{T, 3},
                                bias = nothing; y = nothing, dα = nothing, mask = nothing, nheads = 1, stats = nothing,
                                fdrop::Union{typeof(identity), Dropout} = identity) where {T <: MIFloat}
    E, Lq, B = size(q); Lkv = size(k, 2); Ev = size(v, 1)
    size(dy) == (Ev, Lq, B) || throw(DimensionMismatch("dy must have the size of the output $((Ev, Lq, B)), got $(size(dy))"))
    causal, mptr, mstr, bptr, bstr = mask_and_bias(T, bias, mask, (Lkv, Lq, nheads, B))
    dq, dk, dv = similar(q, T, size(q)), similar(k, T, size(k)), similar(v, T, size(v))
    dbias = bias === nothing ? nothing : DeviceArray{Float32}(undef, size(bias)...)
    dbias === nothing || check(ccall((:mi_fill_zero, libmi), Int32, (Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), dbias.ptr, sizeof(Float32) * length(dbias), C_NULL))
    p, seed = fdrop isa Dropout ? (fdrop.p, fdrop.seed) : (0f0, UInt64(0))
    fwd_desc(yptr) = AttnDesc(Int32(sizeof(AttnDesc)), dtype_code(T), dtype_code(T), causal, UInt32(0), Int32(0), E, Ev, Lq, Lkv, nheads, B,
                              q.ptr, k.ptr, v.ptr, yptr, C_NULL, bptr, bstr, mptr, mstr, C_NULL, 0, p, UInt32(0), seed, stats === nothing ? C_NULL : stats.ptr)
    # y === nothing: the library recomputes the forward result where its MFMA kernels can take the gradient; the
    # workspace mi_attention_bwd_plan asks for has room for it
    fwd = fwd_desc(y === nothing ? C_NULL : y.ptr)
    mk(ws, wsbytes) = AttnBwdDesc(Int32(sizeof(AttnBwdDesc)), Int32(0), fwd, dy.ptr, dα === nothing ? C_NULL : dα.ptr, dq.ptr, dk.ptr,
                                  dv.ptr, dbias === nothing ? C_NULL : dbias.ptr, ws, wsbytes)
    need = Ref{Csize_t}(0)
    check(ccall((:mi_attention_bwd_plan, libmi), Int32, (Ref{AttnBwdDesc}, Ptr{Int32}, Ptr{Csize_t}), mk(C_NULL, 0), C_NULL, need))
    ws = need[] > 0 ? DeviceArray{UInt8}(undef, Int(need[])) : nothing
    GC.@preserve dy q k v bias mask y dα dq dk dv dbias ws stats begin
        check(ccall((:mi_attention_bwd, libmi), Int32, (Ref{AttnBwdDesc}, Ptr{Cvoid}), mk(ws === nothing ? C_NULL : ws.ptr, need[]), C_NULL))
    end
    dq, dk, dv, dbias
end

# x[d,h,i,b] = sum_j α[j,i,h,b] v[d,h,j,b]: one strided batched GEMM over heads per batch element
function weights_times_values(α::DeviceArray{T, 4}, v::DeviceArray{T, 3}, H::Int) where {T}
    Ev, Lkv, B = size(v); Lq = size(α, 2); Dv = Ev ÷ H
    out = DeviceArray{T}(undef, Ev, Lq, B)
    for b in 0:B-1
        gemm!('N', 'N', Dv, Lq, Lkv, 1f0, v.ptr + sizeof(T) * b * Ev * Lkv, Ev, Dv,
              α.ptr + sizeof(T) * b * Lkv * Lq * H, Lkv, Lkv * Lq, 0f0, out.ptr + sizeof(T) * b * Ev * Lq, Ev, Dv, H, T)
    end
    out
end

# ---- softmax family (NNlib src/softmax.jl) ---------------------------------------------------------
const MI_SOFTMAX, MI_LOGSOFTMAX = Int32(0), Int32(1)

# dims (an integer, a tuple of dimensions, adjacent or not, or :) as the bit mask of the *_dims entry points, the
# sizes as a host vector, and a workspace of the size the library asks for (0 bytes for a run of adjacent dimensions)
function dims_call(x::DeviceArray{T, N}, dims) where {T, N}
    N <= 8 || throw(ArgumentError("the softmax family takes arrays of up to 8 dimensions"))
    ds = dims isa Colon ? collect(1:N) : collect(Int, dims)
    (isempty(ds) || minimum(ds) < 1) && throw(ArgumentError("dims must be positive dimension numbers, got $dims"))
    mask = UInt32(sum(d -> UInt32(1) << (d - 1), filter(d -> d <= N, unique(ds)); init = UInt32(0)))
    sizes = collect(Int64, size(x))
    need = Ref{Csize_t}(0)
    check(ccall((:mi_softmax_dims_workspace, libmi), Int32, (Int32, Int32, Ptr{Int64}, UInt32, Ptr{Csize_t}),
                dtype_code(T), Int32(N), sizes, mask, need))
    ws = need[] > 0 ? DeviceArray{UInt8}(undef, Int(need[])) : nothing
    sizes, mask, ws, need[]
end
wsptr(ws) = ws === nothing ? C_NULL : ws.ptr

function softmax_like!(op::Int32, out::DeviceArray{T, N}, x::DeviceArray{T, N}, dims) where {T <: MIFloat64, N}
    size(out) == size(x) || throw(DimensionMismatch("output size $(size(out)) differs from input size $(size(x))"))
    sizes, mask, ws, wsb = dims_call(x, dims)
    GC.@preserve out x sizes ws check(ccall((:mi_softmax_dims, libmi), Int32,
        (Int32, Int32, Ptr{Cvoid}, Ptr{Cvoid}, Int32, Ptr{Int64}, UInt32, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
        op, dtype_code(T), x.ptr, out.ptr, Int32(N), sizes, mask, wsptr(ws), wsb, C_NULL))
    out
end

# float.(x) for an integer array: Float64, what `similar(x, float(T))` is in src/softmax.jl:56
function to_float64(x::DeviceArray{T, N}) where {T <: Union{Int32, Int64}, N}
    out = similar(x, Float64, size(x))
    GC.@preserve out x check(ccall((:mi_convert, libmi), Int32, (Ptr{Cvoid}, Int32, Ptr{Cvoid}, Int32, Int64, Ptr{Cvoid}),
                                  out.ptr, MI_F64, x.ptr, dtype_code(T), length(x), C_NULL))
    out
end
softmax(x::DeviceArray{<:Union{Int32, Int64}}; dims = 1) = softmax(to_float64(x); dims)
logsoftmax(x::DeviceArray{<:Union{Int32, Int64}}; dims = 1) = logsoftmax(to_float64(x); dims)
logsumexp(x::DeviceArray{<:Union{Int32, Int64}}; dims = :) = logsumexp(to_float64(x); dims)
softmax(x::DeviceArray{T}; dims = 1) where {T <: MIFloat64} = softmax!(similar(x, T, size(x)), x; dims)
softmax!(x::DeviceArray; dims = 1) = softmax!(x, x; dims)
softmax!(out::DeviceArray{T}, x::DeviceArray{T}; dims = 1) where {T <: MIFloat64} = softmax_like!(MI_SOFTMAX, out, x, dims)

logsoftmax(x::DeviceArray{T}; dims = 1) where {T <: MIFloat64} = logsoftmax!(similar(x, T, size(x)), x; dims)
logsoftmax!(x::DeviceArray; dims = 1) = logsoftmax!(x, x; dims)
logsoftmax!(out::DeviceArray{T}, x::DeviceArray{T}; dims = 1) where {T <: MIFloat64} = softmax_like!(MI_LOGSOFTMAX, out, x, dims)

# logsumexp(x; dims = :) returns a scalar for dims = : (one device-to-host copy), else an array that
# keeps the reduced dimensions with extent 1, as NNlib's does (src/softmax.jl:200-203).
function logsumexp(x::DeviceArray{T, N}; dims = :) where {T <: MIFloat64, N}
    sizes, mask, ws, wsb = dims_call(x, dims)
    kept = dims isa Colon ? () : ntuple(d -> d in dims ? 1 : size(x, d), N)
    out = similar(x, T, kept)
    GC.@preserve out x sizes ws check(ccall((:mi_logsumexp_dims, libmi), Int32,
        (Int32, Ptr{Cvoid}, Ptr{Cvoid}, Int32, Ptr{Int64}, UInt32, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
        dtype_code(T), x.ptr, out.ptr, Int32(N), sizes, mask, wsptr(ws), wsb, C_NULL))
    dims isa Colon ? Array(out)[] : out
end

# Pullback of logsumexp (rrule at src/softmax.jl:205-212): dy and lse are device arrays with the size of the
# reduced result (for dims = : a 0-dimensional or one-element array holding the cotangent / the result).
function ∇logsumexp(dy::DeviceArray{T}, x::DeviceArray{T, N}, lse::DeviceArray{T}; dims = :) where {T <: MIFloat64, N}
    sizes, mask, ws, wsb = dims_call(x, dims)
    n_out = dims isa Colon ? 1 : prod(d -> d in dims ? 1 : size(x, d), 1:N; init = 1)
    length(dy) == length(lse) == n_out || throw(DimensionMismatch("dy and lse must have the size of logsumexp(x; dims)"))
    dx = similar(x, T, size(x))
    GC.@preserve dy x lse dx sizes ws check(ccall((:mi_logsumexp_bwd_dims, libmi), Int32,
        (Int32, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Int32, Ptr{Int64}, UInt32, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
        dtype_code(T), dy.ptr, x.ptr, lse.ptr, dx.ptr, Int32(N), sizes, mask, wsptr(ws), wsb, C_NULL))
    dx
end

function softmax_grad!(op::Int32, dx::DeviceArray{T, N}, dy::DeviceArray{T, N}, y::DeviceArray{T, N}, dims) where {T <: MIFloat64, N}
    size(dx) == size(dy) == size(y) || throw(DimensionMismatch("dx, dy and y must have one size"))
    sizes, mask, ws, wsb = dims_call(y, dims)
    GC.@preserve dx dy y sizes ws check(ccall((:mi_softmax_bwd_dims, libmi), Int32,
        (Int32, Int32, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Int32, Ptr{Int64}, UInt32, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
        op, dtype_code(T), dy.ptr, y.ptr, dx.ptr, Int32(N), sizes, mask, wsptr(ws), wsb, C_NULL))
    dx
end
∇softmax!(dx::DeviceArray, dy::DeviceArray, y::DeviceArray; dims = 1) = softmax_grad!(MI_SOFTMAX, dx, dy, y, dims)
∇softmax(dy::DeviceArray{T}, y::DeviceArray{T}; dims = 1) where {T} = ∇softmax!(similar(y, T, size(y)), dy, y; dims)
∇logsoftmax!(dx::DeviceArray, dy::DeviceArray, y::DeviceArray; dims = 1) = softmax_grad!(MI_LOGSOFTMAX, dx, dy, y, dims)
∇logsoftmax(dy::DeviceArray{T}, y::DeviceArray{T}; dims = 1) where {T} = ∇logsoftmax!(similar(y, T, size(y)), dy, y; dims)

# ---- batched_mul -----------------------------------------------------------------------------------
function gemm!(tA, tB, m, n, k, α, A, lda, sA, B, ldb, sB, β, C, ldc, sC, batch, ::Type{T}) where {T}
    check(ccall((:mi_batched_gemm, libmi), Int32,
                (Int32, Cchar, Cchar, Int64, Int64, Int64, Float32, Ptr{Cvoid}, Int64, Int64, Ptr{Cvoid}, Int64, Int64,
                 Float32, Ptr{Cvoid}, Int64, Int64, Int64, Ptr{Cvoid}),
                dtype_code(T), tA, tB, m, n, k, α, A, lda, sA, B, ldb, sB, β, C, ldc, sC, batch, C_NULL);
          shape_error = DimensionMismatch)
end

# ('N' | 'T', leading dimension) from strides: the table of _batched_try_gemm!, src/batched/batchedmul.jl:272-294
function blas_layout(X::DeviceArray{T, 3}) where {T}
    s1, s2, _ = strides(X)
    if s2 == 1 && size(X, 1) > 1
        'T', max(s1, size(X, 2), 1)
    elseif s1 == 1
        'N', max(s2, size(X, 1), 1)
    elseif s2 == 1
        'T', max(s1, size(X, 2), 1)
    else
        throw(ArgumentError("Unsupported array layout for batched mul.\n- Size: $(size(X))\n- Strides: $(strides(X))"))
    end
end

function batched_mul!(C::DeviceArray{T, 3}, A::DeviceArray{T, 3}, B::DeviceArray{T, 3}, α::Number = one(Float32),
                      β::Number = zero(Float32)) where {T <: MIFloat}
    size(A, 3) == size(C, 3) || size(A, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != C"))
    size(B, 3) == size(C, 3) || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: B != C"))
    m, ka = size(A, 1), size(A, 2); kb, n = size(B, 1), size(B, 2)
    (ka == kb && m == size(C, 1) && n == size(C, 2)) ||
        throw(DimensionMismatch("A1 has size ($m,$ka), B1 has size ($kb,$n), C1 has size $(size(C)[1:2])"))
    if strides(C)[1] != 1 && strides(C)[2] == 1 && size(C, 1) > 1
        # C is a lazily permuted array: C' = B' * A' (src/batched/batchedmul.jl:268-270)
        batched_mul!(batched_transpose(C), batched_transpose(B), batched_transpose(A), α, β)
        return C
    end
    (tA, lda), (tB, ldb) = blas_layout(A), blas_layout(B)
    (strides(C)[1] == 1 || size(C, 1) == 1) || throw(ArgumentError("Unsupported array layout for batched mul.\n- Size: $(size(C))\n- Strides: $(strides(C))"))
    sA = size(A, 3) == 1 ? 0 : strides(A)[3]          # src/gemm.jl:117-118
    sB = size(B, 3) == 1 ? 0 : strides(B)[3]
    GC.@preserve A B C gemm!(tA, tB, m, n, ka, Float32(α), A.ptr, lda, sA, B.ptr, ldb, sB, Float32(β), C.ptr,
                              max(strides(C)[2], m, 1), strides(C)[3], size(C, 3), T)
    C
end

# Float64 (dgemm_ in the reference, src/gemm.jl:27-32): the same call on the fp64 matrix cores
function batched_mul!(C::DeviceArray{Float64, 3}, A::DeviceArray{Float64, 3}, B::DeviceArray{Float64, 3}, α::Number = 1.0, β::Number = 0.0)
    blasable(X) = strides(X)[1] == 1 || strides(X)[2] == 1 || size(X, 1) == 1 || size(X, 2) == 1
    (blasable(A) && blasable(B) && strides(C)[1] == 1) || return generic_mul!(C, A, B, α, β)
    size(A, 3) == size(C, 3) || size(A, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != C"))
    size(B, 3) == size(C, 3) || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: B != C"))
    m, ka = size(A, 1), size(A, 2); kb, n = size(B, 1), size(B, 2)
    (ka == kb && m == size(C, 1) && n == size(C, 2)) ||
        throw(DimensionMismatch("A1 has size ($m,$ka), B1 has size ($kb,$n), C1 has size $(size(C)[1:2])"))
    (tA, lda), (tB, ldb) = blas_layout(A), blas_layout(B)
    GC.@preserve A B C check(ccall((:mi_batched_gemm_f64, libmi), Int32,
        (Cchar, Cchar, Int64, Int64, Int64, Float64, Ptr{Cvoid}, Int64, Int64, Ptr{Cvoid}, Int64, Int64, Float64, Ptr{Cvoid}, Int64, Int64, Int64, Ptr{Cvoid}),
        tA, tB, m, n, ka, Float64(α), A.ptr, lda, size(A, 3) == 1 ? 0 : strides(A)[3], B.ptr, ldb, size(B, 3) == 1 ? 0 : strides(B)[3],
        Float64(β), C.ptr, max(strides(C)[2], m, 1), strides(C)[3], size(C, 3), C_NULL); shape_error = DimensionMismatch)
    C
end

# batched_mul_generic! (src/batched/batchedmul.jl:306-325): element types that differ, integers, ComplexF64, layouts
# that are neither 'N' nor 'T'.  C's element type is promote_type of A's and B's; the library converts and computes in it.
const AnyArr = Union{DeviceArray{<:MINumber, 3}, BatchedAdjoint}
strided_operand(a::DeviceArray{T, 3}) where {T} = (a.ptr, strides(a)[1], strides(a)[2], strides(a)[3], Int32(0), dtype_code(T))
strided_operand(a::BatchedAdjoint{T}) where {T <: Complex} = (a.parent.ptr, strides(a.parent)[2], strides(a.parent)[1], strides(a.parent)[3], Int32(1), dtype_code(T))
function generic_mul!(C::DeviceArray{TC, 3}, A::AnyArr, B::AnyArr, α::Number = true, β::Number = false) where {TC <: MINumber}
    size(A, 3) == size(C, 3) || size(A, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != C"))
    size(B, 3) == size(C, 3) || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: B != C"))
    m, ka = size(A, 1), size(A, 2); kb, n = size(B, 1), size(B, 2)
    (ka == kb && m == size(C, 1) && n == size(C, 2)) ||
        throw(DimensionMismatch("A1 has size ($m,$ka), B1 has size ($kb,$n), C1 has size $(size(C)[1:2])"))
    (pa, ar, ac, ab, ca, da), (pb, br, bc, bb, cb, db) = strided_operand(A), strided_operand(B)
    al, be = ComplexF64(α), ComplexF64(β)
    GC.@preserve A B C check(ccall((:mi_batched_mul_generic, libmi), Int32,
        (Int32, Int32, Int32, Int64, Int64, Int64, Float64, Float64, Ptr{Cvoid}, Int64, Int64, Int64, Int32, Ptr{Cvoid}, Int64, Int64, Int64, Int32,
         Float64, Float64, Ptr{Cvoid}, Int64, Int64, Int64, Int64, Ptr{Cvoid}),
        dtype_code(TC), da, db, m, n, ka, real(al), imag(al), pa, ar, ac, size(A, 3) == 1 ? 0 : ab, ca, pb, br, bc, size(B, 3) == 1 ? 0 : bb, cb,
        real(be), imag(be), C.ptr, strides(C)[1], strides(C)[2], strides(C)[3], size(C, 3), C_NULL); shape_error = DimensionMismatch)
    C
end
batched_mul!(C::DeviceArray{TC, 3}, A::AnyArr, B::AnyArr, α::Number = true, β::Number = false) where {TC <: MINumber} = generic_mul!(C, A, B, α, β)
function batched_mul(A::AnyArr, B::AnyArr)
    size(A, 3) == size(B, 3) || size(A, 3) == 1 || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != B"))
    T = promote_type(eltype(A), eltype(B))                     # src/batched/batchedmul.jl:65
    batched_mul!(DeviceArray{T}(undef, size(A, 1), size(B, 2), max(size(A, 3), size(B, 3))), A, B)
end

# ComplexF32 (cgemm in the reference, src/gemm.jl:31): one strided kernel takes 'N', 'T', 'C' and every
# permuted layout of A, B and C (the cases of src/batched/batchedmul.jl:261-296 and the generic fallback :306-325)
const CArr = Union{DeviceArray{ComplexF32, 3}, BatchedAdjoint{ComplexF32}}
operand(a::DeviceArray{ComplexF32, 3}) = (a.ptr, strides(a)[1], strides(a)[2], strides(a)[3], Int32(0))
operand(a::BatchedAdjoint{ComplexF32}) = (a.parent.ptr, strides(a.parent)[2], strides(a.parent)[1], strides(a.parent)[3], Int32(1))
function batched_mul!(C::DeviceArray{ComplexF32, 3}, A::CArr, B::CArr, α::Number = true, β::Number = false)
    size(A, 3) == size(C, 3) || size(A, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != C"))
    size(B, 3) == size(C, 3) || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: B != C"))
    m, ka = size(A, 1), size(A, 2); kb, n = size(B, 1), size(B, 2)
    (ka == kb && m == size(C, 1) && n == size(C, 2)) ||
        throw(DimensionMismatch("A1 has size ($m,$ka), B1 has size ($kb,$n), C1 has size $(size(C)[1:2])"))
    (pa, ar, ac, ab, ca), (pb, br, bc, bb, cb) = operand(A), operand(B)
    al, be = ComplexF32(α), ComplexF32(β)
    GC.@preserve A B C check(ccall((:mi_batched_mul_c32, libmi), Int32,
        (Int64, Int64, Int64, Float32, Float32, Ptr{Cvoid}, Int64, Int64, Int64, Int32, Ptr{Cvoid}, Int64, Int64, Int64, Int32,
         Float32, Float32, Ptr{Cvoid}, Int64, Int64, Int64, Int64, Ptr{Cvoid}),
        m, n, ka, real(al), imag(al), pa, ar, ac, size(A, 3) == 1 ? 0 : ab, ca, pb, br, bc, size(B, 3) == 1 ? 0 : bb, cb,
        real(be), imag(be), C.ptr, strides(C)[1], strides(C)[2], strides(C)[3], size(C, 3), C_NULL); shape_error = DimensionMismatch)
    C
end
function batched_mul(A::CArr, B::CArr)
    size(A, 3) == size(B, 3) || size(A, 3) == 1 || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != B"))
    batched_mul!(DeviceArray{ComplexF32}(undef, size(A, 1), size(B, 2), max(size(A, 3), size(B, 3))), A, B)
end

# lazy PermutedDimsArray(A, perm) and matrix transpose: same memory, permuted size and strides
permuted(a::DeviceArray{T, N}, perm::NTuple{N, Int}) where {T, N} =
    DeviceArray{T, N}(a.ptr, ntuple(i -> a.dims[perm[i]], N), ntuple(i -> a.strides[perm[i]], N), a)
Base.transpose(a::DeviceArray{T, 2}) where {T} = permuted(a, (2, 1))
Base.adjoint(a::DeviceArray{T, 2}) where {T <: Real} = permuted(a, (2, 1))
with_batch(a::DeviceArray{T, 2}) where {T} = DeviceArray{T, 3}(a.ptr, (a.dims..., 1), (a.strides..., length(a)), a)

# dense copy of a lazy view of up to 3 dimensions (copy(X) in _copy_if_faster, src/batched/batchedmul.jl:76-83)
function Base.copy(a::DeviceArray{T, N}) where {T, N}
    N <= 3 || throw(ArgumentError("copy of a strided DeviceArray is built for up to 3 dimensions"))
    out = DeviceArray{T}(undef, size(a)...)
    d = (size(a)..., ntuple(_ -> 1, 3 - N)...); s = (strides(a)..., ntuple(_ -> 0, 3 - N)...)
    GC.@preserve a out check(ccall((:mi_strided_copy, libmi), Int32,
                                   (Ptr{Cvoid}, Ptr{Cvoid}, Int32, Int64, Int64, Int64, Int64, Int64, Int64, Ptr{Cvoid}),
                                   out.ptr, a.ptr, sizeof(T), d[1], d[2], d[3], s[1], s[2], s[3], C_NULL))
    out
end

# layouts the GEMM kernel cannot address are materialised first (the reference copies the stride(X,3) == 1
# case and hands the rest to batched_mul_generic!; the results are the same)
function copy_if_faster(X::DeviceArray{T, 3}) where {T}
    s1, s2, s3 = strides(X)
    ((s3 == 1 && s1 != 1 && size(X, 3) > 1) || (s1 != 1 && s2 != 1 && size(X, 1) > 1 && size(X, 2) > 1)) ? copy(X) : X
end

function batched_mul(A::DeviceArray{T, 3}, B::DeviceArray{T, 3}) where {T <: MIFloat}
    size(A, 3) == size(B, 3) || size(A, 3) == 1 || size(B, 3) == 1 || throw(DimensionMismatch("batch size mismatch: A != B"))
    batched_mul!(DeviceArray{T}(undef, size(A, 1), size(B, 2), max(size(A, 3), size(B, 3))), copy_if_faster(A), copy_if_faster(B))
end
# a matrix (plain or lazily transposed) on either side is shared by every batch (src/batched/batchedmul.jl:140-164)
batched_mul(A::DeviceArray{T, 3}, B::DeviceArray{T, 2}) where {T <: MIFloat} = batched_mul(A, with_batch(B))
batched_mul(A::DeviceArray{T, 2}, B::DeviceArray{T, 3}) where {T <: MIFloat} = batched_mul(with_batch(A), B)

# batched_vec (src/batched/batchedmul.jl:166-218)
function batched_vec(A::DeviceArray{T}, B::DeviceArray{T}) where {T <: MIFloat}
    ndims(A) == ndims(B) + 1 || throw(DimensionMismatch("batched_vec requires ndims(A) == ndims(B) + 1, got ndims(A)=$(ndims(A)) and ndims(B)=$(ndims(B))"))
    size(A)[3:end] == size(B)[2:end] || throw(DimensionMismatch("batch dimensions must match: size(A)[3:end]=$(size(A)[3:end]) != size(B)[2:end]=$(size(B)[2:end])"))
    Bd = is_dense(B) ? B : copy(B)
    C = batched_mul(A, reshape(Bd, (size(B, 1), 1, size(B)[2:end]...)))
    reshape(C, (size(C, 1), size(C)[3:end]...))
end
batched_vec(A::DeviceArray{T, 3}, b::DeviceArray{T, 1}) where {T <: MIFloat} =
    reshape(batched_mul(A, reshape(b, (length(b), 1, 1))), (size(A, 1), size(A, 3)))

# pullback of batched_mul (rrule at src/batched/batchedmul.jl:96-110); an operand with batch extent 1 was
# shared by every slice, so its gradient accumulates over slices (beta = 1)
function batched_mul_pullback(A::DeviceArray{T, 3}, B::DeviceArray{T, 3}, Δ::DeviceArray{T, 3}) where {T <: MIFloat}
    nb = size(Δ, 3)
    slice(X, b) = DeviceArray{T, 3}(X.ptr + sizeof(T) * (size(X, 3) > 1 ? b * strides(X)[3] : 0), (size(X, 1), size(X, 2), 1), strides(X), X)
    function grad(X, f)
        (size(X, 3) != 1 || nb == 1) && return f(Δ, A, B, nothing)
        out = DeviceArray{T}(undef, size(X)...)
        for b in 0:nb-1
            f(slice(Δ, b), slice(A, b), slice(B, b), (out, b == 0 ? 0f0 : 1f0))
        end
        out
    end
    dA = grad(A, (Δ, A, B, acc) -> acc === nothing ? batched_mul(Δ, batched_adjoint(B)) : batched_mul!(acc[1], Δ, batched_adjoint(B), 1f0, acc[2]))
    dB = grad(B, (Δ, A, B, acc) -> acc === nothing ? batched_mul(batched_adjoint(A), Δ) : batched_mul!(acc[1], batched_adjoint(A), Δ, 1f0, acc[2]))
    dA, dB
end

function batched_mul(x::DeviceArray{T, N}, y::DeviceArray{T, N}) where {T <: MIFloat, N}
    batch_size = size(x)[3:end]
    @assert batch_size == size(y)[3:end] "batch size has to be the same for the two arrays."
    z = batched_mul(reshape(x, (size(x, 1), size(x, 2), prod(batch_size))), reshape(y, (size(y, 1), size(y, 2), prod(batch_size))))
    reshape(z, (size(z, 1), size(z, 2), batch_size...))
end

end # module
