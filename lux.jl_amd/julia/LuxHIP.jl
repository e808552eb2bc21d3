# LuxHIP.jl -- Julia glue that puts libluxhip behind LuxLib's own device-dispatch points.
#
# Written against LuxLib v1.15 (lib/LuxLib of LuxDL/Lux.jl).  LuxLib's public API and its
# ChainRulesCore rrules stay untouched: this module only
#   * defines a device type and a dense array type whose memory libluxhip owns,
#   * adds methods on LuxLib.Impl's backend hooks (the same hooks LuxLibCUDAExt / LuxLibcuDNNExt
#     override: fused_dense!, matmul!, matmuladd!, bias_activation!, ∇activation, batchnorm,
#     conv!, ∇conv_data, ∇conv_filter, conv_bias_act), and
#   * adds whole-op methods + rrules where the reference has no device hook (layernorm,
#     groupnorm, batchnorm as cuDNNExt does).
#
# There is no Julia toolchain where this repository is built and tested, so this file is
# exercised nowhere yet; the Python mirror (lux.jl_amd/luxlib.py) drives the very same C ABI
# with the very same argument order and is what the parity tests run.  A CPU test parses every
# `ccall((:luxhip_...` below and checks symbol, argument count and C types against include/luxhip.h.
module LuxHIP

using LuxLib: LuxLib, Impl, Traits, Utils
using LuxLib.Traits: GPUBroadcastOp
using ChainRulesCore: ChainRulesCore, NoTangent, ProjectTo, @thunk
using NNlib: NNlib, DenseConvDims
using MLDataDevices: MLDataDevices, AbstractGPUDevice
using Static: True, False, StaticBool, known
using LinearAlgebra: Adjoint, Transpose
using Random: Random

const CRC = ChainRulesCore
const libluxhip = get(ENV, "LIBLUXHIP", joinpath(@__DIR__, "..", "libluxhip.so"))

# ---------------------------------------------------------------------------------------------
# status handling: 0 ok, -1 unsupported (caller falls back), anything else throws
# ---------------------------------------------------------------------------------------------
struct LuxHIPError <: Exception
    status::Cint
    msg::String
end
last_error() = unsafe_string(ccall((:luxhip_last_error, libluxhip), Cstring, ()))
@inline function check(status::Cint)
    status == 0 && return true
    status == -1 && return false                     # LUXHIP_UNSUPPORTED -> generic path
    throw(LuxHIPError(status, last_error()))
end

# ---------------------------------------------------------------------------------------------
# device + array
# ---------------------------------------------------------------------------------------------
struct LuxHIPDevice <: AbstractGPUDevice end

const STREAM = Ref{Ptr{Cvoid}}(C_NULL)
function __init__()
    check(ccall((:luxhip_init, libluxhip), Cint, (Cint,), 0))
    check(ccall((:luxhip_stream_create, libluxhip), Cint, (Ptr{Ptr{Cvoid}},), STREAM))
end
stream() = STREAM[]
synchronize() = check(ccall((:luxhip_stream_synchronize, libluxhip), Cint, (Ptr{Cvoid},), stream()))

const HIPFloat = Union{Float32,Core.BFloat16}
dtype_code(::Type{Float32}) = Cint(0)
dtype_code(::Type{Core.BFloat16}) = Cint(1)

"Dense column-major array in HBM whose buffer belongs to libluxhip's pooled allocator."
mutable struct HIPArray{T,N} <: DenseArray{T,N}
    ptr::Ptr{T}
    dims::Dims{N}
    owner::Any          # the HIPArray that owns the buffer (for reshapes) or `nothing`
    function HIPArray{T,N}(::UndefInitializer, dims::Dims{N}) where {T,N}
        p = Ref{Ptr{Cvoid}}(C_NULL)
        check(ccall((:luxhip_malloc, libluxhip), Cint, (Ptr{Ptr{Cvoid}}, Csize_t), p, max(prod(dims) * sizeof(T), 1)))
        a = new{T,N}(Ptr{T}(p[]), dims, nothing)
        finalizer(x -> ccall((:luxhip_free, libluxhip), Cint, (Ptr{Cvoid},), x.ptr), a)
        return a
    end
    HIPArray{T,N}(ptr::Ptr{T}, dims::Dims{N}, owner) where {T,N} = new{T,N}(ptr, dims, owner)
end
Base.size(a::HIPArray) = a.dims
Base.pointer(a::HIPArray) = a.ptr
Base.similar(a::HIPArray, ::Type{T}, dims::Dims{N}) where {T,N} = HIPArray{T,N}(undef, dims)
Base.reshape(a::HIPArray{T}, dims::Dims{N}) where {T,N} = HIPArray{T,N}(a.ptr, dims, something(a.owner, a))
Base.unsafe_convert(::Type{Ptr{T}}, a::HIPArray{T}) where {T} = a.ptr
function HIPArray(h::Array{T,N}) where {T<:HIPFloat,N}
    a = HIPArray{T,N}(undef, size(h))
    check(ccall((:luxhip_memcpy_h2d, libluxhip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), a.ptr, h, sizeof(h), stream()))
    return a
end
function Base.Array(a::HIPArray{T,N}) where {T,N}
    h = Array{T,N}(undef, size(a))
    check(ccall((:luxhip_memcpy_d2h, libluxhip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), h, a.ptr, sizeof(h), stream()))
    return h
end
MLDataDevices.get_device_type(::HIPArray) = LuxHIPDevice          # feeds internal_operation_mode (traits.jl:191-197)
MLDataDevices.get_device(::HIPArray) = LuxHIPDevice()

# A HIPArray supports neither scalar indexing nor Base broadcasting (no kernel compiler sits behind
# it): whatever libluxhip declines (status -1: an activation without a device kernel, an unsupported
# shape) cannot fall back to LuxLib's generic broadcast path on this array type.  Those cases raise
# this error, which names the way out: move the operands to the host (`Array(x)`) for that call.
struct HIPFallbackError <: Exception
    what::String
end
Base.showerror(io::IO, e::HIPFallbackError) = print(io, "LuxHIP: ", e.what, " is not handled by libluxhip (", last_error(),
    ") and HIPArray has no generic broadcast/indexing path to fall back to; run this call on host arrays (`Array(x)`)")
Base.getindex(::HIPArray, ::Int...) = throw(HIPFallbackError("scalar indexing"))
Base.setindex!(::HIPArray, _, ::Int...) = throw(HIPFallbackError("scalar indexing"))
Base.Broadcast.BroadcastStyle(::Type{<:HIPArray}) = throw(HIPFallbackError("broadcasting"))
function Base.copyto!(dst::HIPArray{T}, src::HIPArray{T}) where {T}
    length(dst) == length(src) || throw(DimensionMismatch("copyto!: lengths differ"))
    check(ccall((:luxhip_memcpy_d2d, libluxhip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}), dst.ptr, src.ptr,
        length(src) * sizeof(T), stream()))
    return dst
end

const HIPOp = GPUBroadcastOp{LuxHIPDevice}
optr(::Nothing) = C_NULL
optr(a::HIPArray) = Ptr{Cvoid}(pointer(a))

# activation ids of include/luxhip.h; `nothing` => no device kernel (arbitrary closures)
act_id(::typeof(identity)) = Cint(0)
act_id(::typeof(NNlib.relu)) = Cint(1)
act_id(::Union{typeof(tanh),typeof(NNlib.tanh_fast)}) = Cint(2)
act_id(::Union{typeof(NNlib.sigmoid),typeof(NNlib.sigmoid_fast)}) = Cint(3)
act_id(::typeof(NNlib.swish)) = Cint(4)
act_id(::typeof(NNlib.gelu)) = Cint(5)
act_id(::typeof(NNlib.softplus)) = Cint(6)
act_id(::typeof(NNlib.logsigmoid)) = Cint(7)
act_id(::typeof(NNlib.lisht)) = Cint(8)
act_id(::Any) = nothing

icn(x::AbstractArray{T,N}) where {T,N} = N == 1 ? (1, length(x), 1) : (prod(size(x)[1:(N - 2)]), size(x, N - 1), size(x, N))

# ---------------------------------------------------------------------------------------------
# dense: Impl.matmul!, Impl.matmuladd!, Impl.fused_dense!   (impl/matmul.jl:85-125, impl/dense.jl:46-69)
# ---------------------------------------------------------------------------------------------
unwrap(a::HIPArray) = (a, Cint(0))
unwrap(a::Union{Adjoint{<:Any,<:HIPArray},Transpose{<:Any,<:HIPArray}}) = (parent(a), Cint(1))   # prepare_transposed, ext/CUDAExt/cublaslt.jl:15-33

function gemm!(C::HIPArray{T,2}, A, B, bias) where {T<:HIPFloat}
    (Ap, tA), (Bp, tB) = unwrap(A), unwrap(B)
    M, N = size(C)
    K = size(A, 2)
    return check(ccall((:luxhip_matmul, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Int64),
        stream(), dtype_code(T), tA, tB, M, N, K, optr(Ap), max(1, stride(Ap, 2)), optr(Bp), max(1, stride(Bp, 2)),
        optr(bias), optr(C), max(1, stride(C, 2))))
end

function Impl.matmul!(C::HIPArray{T,2}, ::HIPOp, A::AbstractMatrix, B::AbstractMatrix) where {T<:HIPFloat}
    gemm!(C, A, B, nothing) || throw(HIPFallbackError("matmul!"))
    return nothing
end
# C = A * B .+ bias in one kernel (the reference's fallback is `C .= bias; mul!(C, A, B, 1, 1)`, impl/matmul.jl:80-82)
function Impl.matmuladd!(C::HIPArray{T,2}, ::HIPOp, A::AbstractMatrix, B::AbstractMatrix, bias::HIPArray{T,1}) where {T<:HIPFloat}
    gemm!(C, A, B, bias) || throw(HIPFallbackError("matmuladd!"))
    return nothing
end

function fused_dense_device!(y::HIPArray{T,2}, pre, act, W::HIPArray{T,2}, x::HIPArray{T,2}, b) where {T<:HIPFloat}
    id = act_id(act)
    id === nothing && return false
    M, K = size(W)
    N = size(x, 2)
    return check(ccall((:luxhip_fused_dense_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Int64, Ptr{Cvoid}),
        stream(), dtype_code(T), id, M, K, N, optr(W), max(1, stride(W, 2)), optr(x), max(1, stride(x, 2)), optr(b), optr(y),
        max(1, stride(y, 2)), optr(pre)))
end

# Activations without a device kernel (arbitrary closures, e.g. the `x -> x^3` of LuxLib's dense tests): the
# contraction and the bias run on the device with the identity, the closure is applied to a staged host copy.
# Slow (two PCIe transfers) and correct; rule branch 3 of the reference (impl/dense.jl:103-112) does the same with
# its generic broadcast.
function host_activation!(y::HIPArray{T,N}, σ::F) where {F,T<:HIPFloat,N}
    h = Array(y)
    h .= σ.(h)
    copyto!(y, HIPArray(h))
    return y
end
# (σ.(z), Δ -> Δ .* σ'.(z)) through the caller's AD on host arrays
function host_activation_rule(cfg, σ::F, z::HIPArray{T,N}) where {F,T<:HIPFloat,N}
    yh, back = CRC.rrule_via_ad(cfg, Base.Fix1(broadcast, σ), Array(z))
    return HIPArray(yh), Δ -> HIPArray(convert(Array{T,N}, CRC.unthunk(back(Array(CRC.unthunk(Δ)))[2])))
end

function Impl.fused_dense!(y::HIPArray{T,2}, opmode::HIPOp, act::F, W::HIPArray{T,2}, x::HIPArray{T,2},
        b::Union{Nothing,HIPArray{T,1}}) where {F,T<:HIPFloat}
    if act_id(act) === nothing
        fused_dense_device!(y, nothing, identity, W, x, b) || error(last_error())
        host_activation!(y, act)
    elseif !fused_dense_device!(y, nothing, act, W, x, b)
        # -1 (cublaslt.jl:359-402 warns and takes the unfused path): the product still runs on the device
        @warn "libluxhip cannot fuse this dense call; using matmul! followed by bias_activation!" maxlog = 1
        Impl.matmul!(y, opmode, W, x)
        Impl.bias_activation!(y, opmode, act, y, b)
    end
    return nothing
end

# rule branch 3 (impl/dense.jl:103-112) for closures: z = W x .+ b and its pullback on the device, σ on the host
function CRC.rrule(cfg::CRC.RuleConfig{>:CRC.HasReverseMode}, ::typeof(Impl.fused_dense), opmode::HIPOp, act::F, W::HIPArray{T,2},
        x::HIPArray{T,2}, b::Union{Nothing,HIPArray{T,1}}) where {F,T<:HIPFloat}
    act_id(act) === nothing || return CRC.rrule(Impl.fused_dense, opmode, act, W, x, b)
    z, ∇z = CRC.rrule(Impl.fused_dense, opmode, identity, W, x, b)
    y, ∇act = host_activation_rule(cfg, act, z)
    return y, Δ -> ∇z(∇act(Δ))
end

# rrule with the saved pre-activation for activations that need it (precedent: the cuBLASLt AUX
# output used by the gelu rrule, impl/dense.jl:116-134) and a single fused device pullback.
function CRC.rrule(::typeof(Impl.fused_dense), opmode::HIPOp, act::F, W::HIPArray{T,2}, x::HIPArray{T,2},
        b::Union{Nothing,HIPArray{T,1}}) where {F,T<:HIPFloat}
    id = act_id(act)
    id === nothing && throw(HIPFallbackError("the pullback of fused_dense with activation $(act)"))
    M, K = size(W)
    N = size(x, 2)
    y = similar(W, T, (M, N))
    pre = id in (4, 5, 6, 7, 8) ? similar(y) : nothing
    fused_dense_device!(y, pre, act, W, x, b) || error(last_error())
    𝒫W, 𝒫x, 𝒫b = ProjectTo(W), ProjectTo(x), ProjectTo(b)
    function ∇fused_dense_hip(Δ′)
        Δ = CRC.unthunk(Δ′)
        ∂W, ∂x = similar(W), similar(x)
        ∂b = b === nothing ? nothing : similar(b)
        dz = id == 0 ? nothing : similar(y)
        check(ccall((:luxhip_fused_dense_bwd, libluxhip), Cint,
            (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Int64, Ptr{Cvoid}, Int64,
                Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
            stream(), dtype_code(T), id, M, K, N, optr(Δ), optr(y), optr(pre), optr(W), max(1, stride(W, 2)), optr(x),
            max(1, stride(x, 2)), optr(dz), optr(∂W), optr(∂x), optr(∂b))) || error(last_error())
        return NoTangent(), NoTangent(), NoTangent(), 𝒫W(∂W), 𝒫x(∂x), b === nothing ? NoTangent() : 𝒫b(∂b)
    end
    return y, ∇fused_dense_hip
end

# ---------------------------------------------------------------------------------------------
# elementwise: Impl.bias_activation!, Impl.activation!, Impl.∇activation  (impl/bias_activation.jl:207-220,
# impl/activation.jl:113-141)
# ---------------------------------------------------------------------------------------------
function Impl.bias_activation!(y::HIPArray{T,N}, ::HIPOp, σ::F, x::HIPArray{T,N}, bias::Union{Nothing,HIPArray{T,1}}) where {F,T<:HIPFloat,N}
    id = act_id(σ)
    I, C, Nb = icn(x)
    ok = check(ccall((:luxhip_bias_activation_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), something(id, Cint(0)), I, C, Nb, optr(x), optr(bias), optr(y), C_NULL))
    ok || throw(HIPFallbackError("bias_activation! with activation $(σ)"))
    id === nothing && host_activation!(y, σ)        # a closure: the bias on the device, σ on a staged host copy
    return nothing
end
Impl.activation!(y::HIPArray{T,N}, op::HIPOp, σ::F, x::HIPArray{T,N}) where {F,T<:HIPFloat,N} =
    Impl.bias_activation!(y, op, σ, x, nothing)

function Impl.∇activation(::HIPOp, Δ::HIPArray{T,N}, out::HIPArray{T,N}, act::F, x) where {F,T<:HIPFloat,N}
    id = act_id(act)
    id === nothing && throw(HIPFallbackError("∇activation of $(act)"))
    ∂x = similar(out)
    pre = x isa HIPArray ? x : nothing
    check(ccall((:luxhip_bias_activation_bwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), id, length(out), 1, 1, optr(Δ), optr(out), optr(pre), optr(∂x), C_NULL)) || error(last_error())
    return ∂x
end

# ---------------------------------------------------------------------------------------------
# batchnorm: whole-op override + rrule (precedent ext/cuDNNExt/cuDNNExt.jl:26-54)
# ---------------------------------------------------------------------------------------------
function batchnorm_device(x::HIPArray{T,N}, γ, β, rμ, rσ², training::Bool, act, m, ϵ, save::Bool) where {T<:HIPFloat,N}
    I, C, Nb = icn(x)
    y = similar(x)
    upd = training && rμ !== nothing
    rμ′ = upd ? similar(rμ) : rμ
    rσ²′ = upd ? similar(rσ²) : rσ²
    μs = save ? HIPArray{Float32,1}(undef, (C,)) : nothing
    is = save ? HIPArray{Float32,1}(undef, (C,)) : nothing
    check(ccall((:luxhip_batchnorm_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint, Cdouble, Cdouble,
            Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), act_id(act), I, C, Nb, optr(x), optr(γ), optr(β), optr(rμ), optr(rσ²), Cint(training), Float64(m),
        Float64(ϵ), optr(y), upd ? optr(rμ′) : C_NULL, upd ? optr(rσ²′) : C_NULL, optr(μs), optr(is))) || error(last_error())
    return y, rμ′, rσ²′, μs, is
end

function Impl.batchnorm(x::HIPArray{T,N}, γ::Union{Nothing,HIPArray{T,1}}, β::Union{Nothing,HIPArray{T,1}},
        rμ::Union{Nothing,HIPArray{T,1}}, rσ²::Union{Nothing,HIPArray{T,1}}, training::StaticBool, act::F, m, ϵ) where {F,T<:HIPFloat,N}
    act_id(act) === nothing && throw(HIPFallbackError("batchnorm with activation $(act)"))
    y, rμ′, rσ²′, _, _ = batchnorm_device(x, γ, β, rμ, rσ², known(training), act, m, ϵ, false)
    return y, rμ′, rσ²′
end

function CRC.rrule(::typeof(Impl.batchnorm), x::HIPArray{T,N}, γ, β, rμ, rσ², training::StaticBool, act::F, m, ϵ) where {F,T<:HIPFloat,N}
    act_id(act) === nothing && throw(HIPFallbackError("the pullback of batchnorm with activation $(act)"))
    y, rμ′, rσ²′, μs, is = batchnorm_device(x, γ, β, rμ, rσ², known(training), act, m, ϵ, true)
    I, C, Nb = icn(x)
    from_batch = known(training) || rμ === nothing
    function ∇batchnorm_hip(Δ′)
        Δ = CRC.unthunk(first(CRC.unthunk(Δ′)))
        ∂x = similar(x)
        ∂γ = γ === nothing ? nothing : similar(γ)
        ∂β = β === nothing ? nothing : similar(β)
        check(ccall((:luxhip_batchnorm_bwd, libluxhip), Cint,
            (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint,
                Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
            stream(), dtype_code(T), act_id(act), I, C, Nb, optr(Δ), optr(x), optr(γ), optr(β), optr(μs), optr(is), Cint(from_batch),
            optr(∂x), optr(∂γ), optr(∂β))) || error(last_error())
        nt = NoTangent()
        return nt, ∂x, something(∂γ, nt), something(∂β, nt), nt, nt, nt, nt, nt, nt
    end
    return (y, rμ′, rσ²′), ∇batchnorm_hip
end

# ---------------------------------------------------------------------------------------------
# groupnorm: whole-op method + rrule  (impl/groupnorm.jl:5-22, 349-404; mean_var rrule impl/common_ops.jl:45-61)
# ---------------------------------------------------------------------------------------------
function groupnorm_device(x::HIPArray{T,N}, γ, β, groups::Int, act, ϵ, save::Bool) where {T<:HIPFloat,N}
    id = act_id(act)
    id === nothing && throw(HIPFallbackError("groupnorm with activation $(act)"))
    I, C, Nb = icn(x)
    y = similar(x)
    μs = save ? HIPArray{Float32,1}(undef, (groups * Nb,)) : nothing
    is = save ? HIPArray{Float32,1}(undef, (groups * Nb,)) : nothing
    check(ccall((:luxhip_groupnorm_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), id, I, C, groups, Nb, optr(x), optr(γ), optr(β), Float64(ϵ), optr(y), optr(μs), optr(is))) ||
        throw(HIPFallbackError("groupnorm"))
    return y, μs, is
end

Impl.groupnorm(x::HIPArray{T,N}, γ::Union{Nothing,HIPArray{T,1}}, β::Union{Nothing,HIPArray{T,1}}, groups::Int, act::F,
    ϵ) where {F,T<:HIPFloat,N} = first(groupnorm_device(x, γ, β, groups, act, ϵ, false))

function groupnorm_pullback(Δ::HIPArray{T,N}, x::HIPArray{T,N}, γ, β, groups::Int, id::Cint, μs, is) where {T<:HIPFloat,N}
    I, C, Nb = icn(x)
    ∂x = similar(x)
    ∂γ = γ === nothing ? nothing : similar(γ)
    ∂β = β === nothing ? nothing : similar(β)
    check(ccall((:luxhip_groupnorm_bwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid},
            Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), id, I, C, groups, Nb, optr(Δ), optr(x), optr(γ), optr(β), optr(μs), optr(is), optr(∂x), optr(∂γ),
        optr(∂β))) || error(last_error())
    return ∂x, ∂γ, ∂β
end

function CRC.rrule(::typeof(Impl.groupnorm), x::HIPArray{T,N}, γ::Union{Nothing,HIPArray{T,1}}, β::Union{Nothing,HIPArray{T,1}},
        groups::Int, act::F, ϵ) where {F,T<:HIPFloat,N}
    y, μs, is = groupnorm_device(x, γ, β, groups, act, ϵ, true)
    id = act_id(act)
    function ∇groupnorm_hip(Δ′)
        ∂x, ∂γ, ∂β = groupnorm_pullback(CRC.unthunk(Δ′), x, γ, β, groups, id, μs, is)
        nt = NoTangent()
        return nt, ∂x, something(∂γ, nt), something(∂β, nt), nt, nt, nt
    end
    return y, ∇groupnorm_hip
end

# ---------------------------------------------------------------------------------------------
# instancenorm (impl/normalization.jl:191-208): the groupnorm kernels with G = C; training with running
# statistics updates them in the same launch; inference with running statistics is the inference batchnorm
# ---------------------------------------------------------------------------------------------
function instancenorm_device(x::HIPArray{T,N}, γ, β, rμ, rσ², training::Bool, act, m, ϵ, save::Bool) where {T<:HIPFloat,N}
    id = act_id(act)
    id === nothing && throw(HIPFallbackError("instancenorm with activation $(act)"))
    I, C, Nb = icn(x)
    if !training && rμ !== nothing
        y, _, _, μs, is = batchnorm_device(x, γ, β, rμ, rσ², false, act, m, ϵ, save)
        return y, rμ, rσ², (:running, μs, is)
    end
    if training && rμ !== nothing && length(x) > 0
        y, rμ′, rσ²′ = similar(x), similar(rμ), similar(rσ²)
        μs, is = HIPArray{Float32,1}(undef, (C * Nb,)), HIPArray{Float32,1}(undef, (C * Nb,))
        check(ccall((:luxhip_instancenorm_fwd, libluxhip), Cint,
            (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid},
                Cdouble, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
            stream(), dtype_code(T), id, I, C, Nb, optr(x), optr(γ), optr(β), Float64(ϵ), optr(y), optr(μs), optr(is), Float64(m),
            optr(rμ), optr(rσ²), optr(rμ′), optr(rσ²′))) || throw(HIPFallbackError("instancenorm"))
        return y, rμ′, rσ²′, (:sample, μs, is)
    end
    y, μs, is = groupnorm_device(x, γ, β, C, act, ϵ, save)
    return y, rμ, rσ², (:sample, μs, is)
end

function Impl.instancenorm(x::HIPArray{T,N}, γ::Union{Nothing,HIPArray{T,1}}, β::Union{Nothing,HIPArray{T,1}},
        rμ::Union{Nothing,HIPArray{T,1}}, rσ²::Union{Nothing,HIPArray{T,1}}, training::StaticBool, act::F, m, ϵ) where {F,T<:HIPFloat,N}
    y, rμ′, rσ²′, _ = instancenorm_device(x, γ, β, rμ, rσ², known(training), act, m, ϵ, false)
    return y, rμ′, rσ²′
end

function CRC.rrule(::typeof(Impl.instancenorm), x::HIPArray{T,N}, γ, β, rμ, rσ², training::StaticBool, act::F, m, ϵ) where {F,T<:HIPFloat,N}
    y, rμ′, rσ²′, (kind, μs, is) = instancenorm_device(x, γ, β, rμ, rσ², known(training), act, m, ϵ, true)
    id = act_id(act)
    I, C, Nb = icn(x)
    function ∇instancenorm_hip(Δ′)
        Δ = CRC.unthunk(first(CRC.unthunk(Δ′)))
        nt = NoTangent()
        if kind === :running      # statistics are constants: only ∂x = ∂y γ′ and the parameter gradients
            ∂x = similar(x)
            ∂γ = γ === nothing ? nothing : similar(γ)
            ∂β = β === nothing ? nothing : similar(β)
            check(ccall((:luxhip_batchnorm_bwd, libluxhip), Cint,
                (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint,
                    Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
                stream(), dtype_code(T), id, I, C, Nb, optr(Δ), optr(x), optr(γ), optr(β), optr(μs), optr(is), Cint(0), optr(∂x),
                optr(∂γ), optr(∂β))) || error(last_error())
        else
            ∂x, ∂γ, ∂β = groupnorm_pullback(Δ, x, γ, β, C, id, μs, is)
        end
        return nt, ∂x, something(∂γ, nt), something(∂β, nt), nt, nt, nt, nt, nt, nt
    end
    return (y, rμ′, rσ²′), ∇instancenorm_hip
end

# ---------------------------------------------------------------------------------------------
# layernorm: the reference has no device hook (impl/layernorm.jl:3-14 is generic broadcasts), so the
# whole op gets a method + rrule.  Statistics run over a prefix 1:k of the dims ((L, R) view).  Parameters
# that span exactly those dims go into the same kernel; parameters that vary along one other run of dims
# (e.g. (1, 1, C, 1) with dims = Colon()) are applied by a second per-channel pass: the inference batchnorm
# kernel with mean 0, variance 1, ε = 0 on the (I, C, N) view, and its pullback yields their gradients.
# ---------------------------------------------------------------------------------------------
function layernorm_geometry(x::HIPArray{T,N}, γ, β, dims) where {T,N}
    d = Impl.compute_layernorm_dims(x, γ, β, dims)                      # throws like the reference (impl/layernorm.jl:16-35)
    d = d isa Colon ? (1:N) : d
    dv = sort!(collect(Int, d))
    dv == collect(1:length(dv)) || throw(HIPFallbackError("layernorm over the non-leading dims $(d)"))
    k = length(dv)
    L = prod(size(x)[1:k]; init=1)
    R = L == 0 ? 0 : length(x) ÷ L
    γ === nothing && return L, R, nothing
    pshape = (size(γ)..., ntuple(Returns(1), N - ndims(γ))...)         # expand_layernorm_dims (impl/layernorm.jl:37-51)
    pshape == (size(x)[1:k]..., ntuple(Returns(1), N - k)...) && return L, R, nothing
    varying = findall(!=(1), collect(pshape))
    a, b = isempty(varying) ? (N + 1, N) : (first(varying), last(varying))
    all(i -> pshape[i] == size(x, i), a:b) || throw(HIPFallbackError("layernorm parameters of shape $(size(γ)) with gaps between the dims they vary along"))
    return L, R, (prod(size(x)[1:(a - 1)]; init=1), prod(size(x)[a:b]; init=1), prod(size(x)[(b + 1):N]; init=1))
end

function layernorm_device(x::HIPArray{T,N}, γ, β, act, dims, ϵ, save::Bool) where {T<:HIPFloat,N}
    id = act_id(act)
    id === nothing && throw(HIPFallbackError("layernorm with activation $(act)"))
    L, R, view = layernorm_geometry(x, γ, β, dims)
    y = similar(x)
    μs = save ? HIPArray{Float32,1}(undef, (R,)) : nothing
    is = save ? HIPArray{Float32,1}(undef, (R,)) : nothing
    fused = view === nothing
    check(ccall((:luxhip_layernorm_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), fused ? id : Cint(0), L, R, optr(x), fused ? optr(γ) : C_NULL, fused ? optr(β) : C_NULL, Float64(ϵ),
        optr(y), optr(μs), optr(is))) || throw(HIPFallbackError("layernorm"))
    fused && return y, (μs, is, L, R, nothing, nothing)
    I, C, Nn = view
    x̂ = reshape(y, (I, C, Nn))
    zeros_c, ones_c = fill_like(γ, C, 0), fill_like(γ, C, 1)
    out, _, _, μa, ia = batchnorm_device(x̂, reshape(γ, (C,)), reshape(β, (C,)), zeros_c, ones_c, false, act, 0.1, 0.0, save)
    return reshape(out, size(x)), (μs, is, L, R, x̂, (μa, ia))
end
fill_like(a::HIPArray{T}, n::Integer, v) where {T} = HIPArray(fill(T(v), n))

Impl.layernorm(x::HIPArray{T,N}, γ::Union{Nothing,HIPArray{T}}, β::Union{Nothing,HIPArray{T}}, act::F, dims, ϵ) where {F,T<:HIPFloat,N} =
    first(layernorm_device(x, γ, β, act, dims, ϵ, false))

function CRC.rrule(::typeof(Impl.layernorm), x::HIPArray{T,N}, γ::Union{Nothing,HIPArray{T}}, β::Union{Nothing,HIPArray{T}}, act::F, dims,
        ϵ) where {F,T<:HIPFloat,N}
    y, (μs, is, L, R, x̂, affine) = layernorm_device(x, γ, β, act, dims, ϵ, true)
    id = act_id(act)
    function ∇layernorm_hip(Δ′)
        Δ = CRC.unthunk(Δ′)
        nt = NoTangent()
        ∂x = similar(x)
        ∂γ = γ === nothing ? nothing : similar(γ)
        ∂β = β === nothing ? nothing : similar(β)
        if affine === nothing
            check(ccall((:luxhip_layernorm_bwd, libluxhip), Cint,
                (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid},
                    Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
                stream(), dtype_code(T), id, L, R, optr(Δ), optr(x), optr(γ), optr(β), optr(μs), optr(is), optr(∂x), optr(∂γ),
                optr(∂β))) || error(last_error())
        else
            # second pass first: ∂x̂ and the parameter gradients from the per-channel pullback, then the normalisation's
            I, C, Nn = size(x̂)
            ∂x̂ = similar(x̂)
            check(ccall((:luxhip_batchnorm_bwd, libluxhip), Cint,
                (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Cint,
                    Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
                stream(), dtype_code(T), id, I, C, Nn, optr(Δ), optr(x̂), optr(γ), optr(β), optr(affine[1]), optr(affine[2]), Cint(0),
                optr(∂x̂), optr(∂γ), optr(∂β))) || error(last_error())
            check(ccall((:luxhip_layernorm_bwd, libluxhip), Cint,
                (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid},
                    Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
                stream(), dtype_code(T), Cint(0), L, R, optr(∂x̂), optr(x), C_NULL, C_NULL, optr(μs), optr(is), optr(∂x), C_NULL,
                C_NULL)) || error(last_error())
        end
        return nt, ∂x, something(∂γ, nt), something(∂β, nt), nt, nt, nt
    end
    return y, ∇layernorm_hip
end

# ---------------------------------------------------------------------------------------------
# conv: Impl.conv!, Impl.∇conv_data, Impl.∇conv_filter, Impl.conv_bias_act  (impl/conv.jl:29-166)
# ---------------------------------------------------------------------------------------------
struct ConvDimsC
    W::Int64; H::Int64; Cin::Int64; N::Int64; kW::Int64; kH::Int64; Cout::Int64
    stride_w::Int64; stride_h::Int64; pad_w_lo::Int64; pad_w_hi::Int64; pad_h_lo::Int64; pad_h_hi::Int64
    dil_w::Int64; dil_h::Int64; groups::Int64; flipkernel::Int64
end
function ConvDimsC(c::DenseConvDims{2}, N::Integer)
    (W, H), (kW, kH) = NNlib.input_size(c), NNlib.kernel_size(c)
    (sw, sh), (pwl, pwh, phl, phh), (dw, dh) = NNlib.stride(c), NNlib.padding(c), NNlib.dilation(c)
    return ConvDimsC(W, H, NNlib.channels_in(c), N, kW, kH, NNlib.channels_out(c), sw, sh, pwl, pwh, phl, phh, dw, dh,
        NNlib.groupcount(c), NNlib.flipkernel(c) ? 1 : 0)
end

function Impl.conv_bias_act(::Type{LuxHIPDevice}, x::HIPArray{T,4}, w::HIPArray{T,4}, cdims::DenseConvDims{2}, bias, act::F) where {F,T<:HIPFloat}
    id = act_id(act)
    y = similar(x, T, (NNlib.output_size(cdims)..., NNlib.channels_out(cdims), size(x, 4)))
    d = Ref(ConvDimsC(cdims, size(x, 4)))
    ok = id !== nothing && check(ccall((:luxhip_conv_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), id, d, optr(x), optr(w), optr(bias), optr(y), C_NULL, C_NULL))
    ok || throw(HIPFallbackError("conv_bias_act with activation $(act)"))
    return y
end
function Impl.conv!(y::HIPArray{T,4}, ::Type{LuxHIPDevice}, x::HIPArray{T,4}, w::HIPArray{T,4}, cdims::DenseConvDims{2}) where {T<:HIPFloat}
    d = Ref(ConvDimsC(cdims, size(x, 4)))
    check(ccall((:luxhip_conv_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), Cint(0), d, optr(x), optr(w), C_NULL, optr(y), C_NULL, C_NULL)) || throw(HIPFallbackError("conv!"))
    return nothing
end
function Impl.∇conv_data(dy::HIPArray{T,4}, w::HIPArray{T,4}, cdims::DenseConvDims{2}) where {T<:HIPFloat}
    dx = similar(dy, T, (NNlib.input_size(cdims)..., NNlib.channels_in(cdims), size(dy, 4)))
    d = Ref(ConvDimsC(cdims, size(dy, 4)))
    check(ccall((:luxhip_conv_bwd_data, libluxhip), Cint, (Ptr{Cvoid}, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), d, optr(dy), optr(w), optr(dx))) || throw(HIPFallbackError("∇conv_data"))
    return dx
end
function Impl.∇conv_filter(x::HIPArray{T,4}, dy::HIPArray{T,4}, cdims::DenseConvDims{2}) where {T<:HIPFloat}
    dw = similar(x, T, (NNlib.kernel_size(cdims)..., NNlib.channels_in(cdims) ÷ NNlib.groupcount(cdims), NNlib.channels_out(cdims)))
    d = Ref(ConvDimsC(cdims, size(x, 4)))
    check(ccall((:luxhip_conv_bwd_filter, libluxhip), Cint, (Ptr{Cvoid}, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), d, optr(x), optr(dy), optr(dw))) || throw(HIPFallbackError("∇conv_filter"))
    return dw
end

# CRC.rrule(fused_conv) + ∇fused_conv (impl/conv.jl:204-275) as one forward and one pullback call.  The forward
# pass hands over the channel-contiguous copy of x that its kernels read (xt_keep); the pullback's filter
# gradient reads it instead of transposing x again.
function CRC.rrule(::CRC.RuleConfig{>:CRC.HasReverseMode}, ::typeof(Impl.fused_conv), ::HIPOp, act::F, w::HIPArray{T,4}, x::HIPArray{T,4},
        bias::Union{Nothing,HIPArray{T,1}}, cdims::DenseConvDims{2}) where {F,T<:HIPFloat}
    id = act_id(act)
    id === nothing && throw(HIPFallbackError("the pullback of fused_conv with activation $(act)"))
    y = similar(x, T, (NNlib.output_size(cdims)..., NNlib.channels_out(cdims), size(x, 4)))
    pre = id in (4, 5, 6, 7, 8) ? similar(y) : nothing
    xt = similar(x)
    d = Ref(ConvDimsC(cdims, size(x, 4)))
    check(ccall((:luxhip_conv_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), id, d, optr(x), optr(w), optr(bias), optr(y), optr(pre), optr(xt))) || throw(HIPFallbackError("fused_conv"))
    𝒫w, 𝒫x, 𝒫b = ProjectTo(w), ProjectTo(x), ProjectTo(bias)
    function ∇fused_conv_hip(Δ′)
        Δ = CRC.unthunk(Δ′)
        ∂w, ∂x = similar(w), similar(x)
        ∂b = bias === nothing ? nothing : similar(bias)
        dz = id == 0 ? nothing : similar(y)
        check(ccall((:luxhip_fused_conv_bwd, libluxhip), Cint,
            (Ptr{Cvoid}, Cint, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid},
                Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
            stream(), dtype_code(T), id, d, optr(Δ), optr(y), optr(pre), optr(x), optr(w), optr(dz), optr(∂w), optr(∂x), optr(∂b),
            optr(xt))) || error(last_error())
        nt = NoTangent()
        return nt, nt, nt, nt, 𝒫w(∂w), 𝒫x(∂x), bias === nothing ? nt : 𝒫b(∂b), nt
    end
    return y, ∇fused_conv_hip
end

# Three spatial dims (x (W, H, D, C, N), DenseConvDims{3}): the two-dimensional problem on the
# depth-unfolded input.  `inner2d` is the DenseConvDims{2} over (W, H, kD*C, Dout*N); the weight is
# reshaped, not copied.
function inner2d(c::DenseConvDims{3}, N::Integer)
    (W, H, D), (kW, kH, kD) = NNlib.input_size(c), NNlib.kernel_size(c)
    Dout = NNlib.output_size(c)[3]
    g = NNlib.groupcount(c)
    return DenseConvDims((W, H, kD * NNlib.channels_in(c), Dout * N), (kW, kH, kD * (NNlib.channels_in(c) ÷ g), NNlib.channels_out(c));
        stride=NNlib.stride(c)[1:2], padding=NNlib.padding(c)[1:4], dilation=NNlib.dilation(c)[1:2], groups=g,
        flipkernel=NNlib.flipkernel(c))
end
depth_args(c::DenseConvDims{3}, N::Integer) = (Int64(prod(NNlib.input_size(c)[1:2])), Int64(NNlib.input_size(c)[3]),
    Int64(NNlib.channels_in(c)), Int64(N), Int64(NNlib.kernel_size(c)[3]), Int64(NNlib.output_size(c)[3]),
    Int64(NNlib.stride(c)[3]), Int64(NNlib.padding(c)[5]), Int64(NNlib.dilation(c)[3]), Cint(NNlib.flipkernel(c)))
function depth_unfold(x::HIPArray{T,5}, c::DenseConvDims{3}) where {T<:HIPFloat}
    c2 = inner2d(c, size(x, 5))
    xu = similar(x, T, (NNlib.input_size(c2)..., NNlib.channels_in(c2), NNlib.output_size(c)[3] * size(x, 5)))
    I, D, Cin, N, kD, Dout, sD, pD, dD, flip = depth_args(c, size(x, 5))       # a ccall takes no splatted arguments
    check(ccall((:luxhip_conv_depth_unfold, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Cint, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), I, D, Cin, N, kD, Dout, sD, pD, dD, flip, optr(x), optr(xu))) || error("luxhip_conv_depth_unfold")
    return xu, c2
end
function depth_fold(dxu::HIPArray{T,4}, c::DenseConvDims{3}, N::Integer) where {T<:HIPFloat}
    dx = similar(dxu, T, (NNlib.input_size(c)..., NNlib.channels_in(c), N))
    I, D, Cin, Nn, kD, Dout, sD, pD, dD, flip = depth_args(c, N)
    check(ccall((:luxhip_conv_depth_fold, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Cint, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), I, D, Cin, Nn, kD, Dout, sD, pD, dD, flip, optr(dxu), optr(dx))) || error("luxhip_conv_depth_fold")
    return dx
end
function swap_middle(a::HIPArray{T}, inner, A, B, outer, shape) where {T<:HIPFloat}
    out = similar(a, T, shape)
    check(ccall((:luxhip_swap_middle_dims, libluxhip), Cint, (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), inner, A, B, outer, optr(a), optr(out))) || error("luxhip_swap_middle_dims")
    return out
end
function from_inner(y2::HIPArray{T,4}, c::DenseConvDims{3}, N) where {T}     # (OW, OH, Cout, Dout*N) -> (OW, OH, Dout, Cout, N)
    (ow, oh, od), co = NNlib.output_size(c), NNlib.channels_out(c)
    return swap_middle(y2, ow * oh, co, od, N, (ow, oh, od, co, N))
end
function to_inner(dy::HIPArray{T,5}, c::DenseConvDims{3}) where {T}          # the inverse
    (ow, oh, od), co, N = NNlib.output_size(c), NNlib.channels_out(c), size(dy, 5)
    return swap_middle(dy, ow * oh, od, co, N, (ow, oh, co, od * N))
end
w2d(w::HIPArray{T,5}) where {T} = reshape(w, size(w, 1), size(w, 2), size(w, 3) * size(w, 4), size(w, 5))

function Impl.conv_bias_act(::Type{LuxHIPDevice}, x::HIPArray{T,5}, w::HIPArray{T,5}, cdims::DenseConvDims{3}, bias, act::F) where {F,T<:HIPFloat}
    xu, c2 = depth_unfold(x, cdims)
    return from_inner(Impl.conv_bias_act(LuxHIPDevice, xu, w2d(w), c2, bias, act), cdims, size(x, 5))
end
function Impl.conv!(y::HIPArray{T,5}, ::Type{LuxHIPDevice}, x::HIPArray{T,5}, w::HIPArray{T,5}, cdims::DenseConvDims{3}) where {T<:HIPFloat}
    xu, c2 = depth_unfold(x, cdims)
    y2 = similar(y, T, (NNlib.output_size(c2)..., NNlib.channels_out(c2), size(xu, 4)))
    Impl.conv!(y2, LuxHIPDevice, xu, w2d(w), c2)
    copyto!(y, from_inner(y2, cdims, size(x, 5)))
    return nothing
end
Impl.∇conv_data(dy::HIPArray{T,5}, w::HIPArray{T,5}, cdims::DenseConvDims{3}) where {T<:HIPFloat} =
    depth_fold(Impl.∇conv_data(to_inner(dy, cdims), w2d(w), inner2d(cdims, size(dy, 5))), cdims, size(dy, 5))
function Impl.∇conv_filter(x::HIPArray{T,5}, dy::HIPArray{T,5}, cdims::DenseConvDims{3}) where {T<:HIPFloat}
    xu, c2 = depth_unfold(x, cdims)
    return reshape(Impl.∇conv_filter(xu, to_inner(dy, cdims), c2), NNlib.kernel_size(cdims)...,
        NNlib.channels_in(cdims) ÷ NNlib.groupcount(cdims), NNlib.channels_out(cdims))
end

function CRC.rrule(cfg::CRC.RuleConfig{>:CRC.HasReverseMode}, ::typeof(Impl.fused_conv), op::HIPOp, act::F, w::HIPArray{T,5},
        x::HIPArray{T,5}, bias::Union{Nothing,HIPArray{T,1}}, cdims::DenseConvDims{3}) where {F,T<:HIPFloat}
    xu, c2 = depth_unfold(x, cdims)
    y2, back2 = CRC.rrule(cfg, Impl.fused_conv, op, act, w2d(w), xu, bias, c2)
    N = size(x, 5)
    function ∇fused_conv3d_hip(Δ′)
        _, _, _, _, ∂w2, ∂xu, ∂b, _ = back2(to_inner(CRC.unthunk(Δ′), cdims))
        return NoTangent(), NoTangent(), NoTangent(), NoTangent(), reshape(∂w2, size(w)), depth_fold(∂xu, cdims, N), ∂b, NoTangent()
    end
    return from_inner(y2, cdims, N), ∇fused_conv3d_hip
end

# ---------------------------------------------------------------------------------------------
# batched_matmul: Impl.batched_matmul!(z, opmode, x, y)  (impl/batched_mul.jl:204-212) and the
# products of the rrule (:320-334), which arrive as NNlib.BatchedAdjoint wrappers
# ---------------------------------------------------------------------------------------------
bunwrap(a::HIPArray{T,3}) where {T} = (a, Cint(0))
bunwrap(a::Union{NNlib.BatchedAdjoint{<:Any,<:HIPArray},NNlib.BatchedTranspose{<:Any,<:HIPArray}}) = (parent(a), Cint(1))
bstride(a::HIPArray{T,3}) where {T} = size(a, 3) == 1 ? 0 : size(a, 1) * size(a, 2)      # extent 1 = shared by all products

function Impl.batched_matmul!(z::HIPArray{T,3}, ::HIPOp, x::AbstractArray{T,3}, y::AbstractArray{T,3}) where {T<:HIPFloat}
    (xp, tx), (yp, ty) = bunwrap(x), bunwrap(y)
    M, N, B = size(z)
    K = size(x, 2)
    check(ccall((:luxhip_batched_matmul, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Cint, Int64, Int64, Int64, Int64, Ptr{Cvoid}, Int64, Int64, Ptr{Cvoid}, Int64, Int64,
         Ptr{Cvoid}, Int64, Int64),
        stream(), dtype_code(T), tx, ty, M, N, K, B, optr(xp), max(1, size(xp, 1)), bstride(xp), optr(yp), max(1, size(yp, 1)),
        bstride(yp), optr(z), max(1, M), M * N)) || throw(HIPFallbackError("batched_matmul!"))
    return nothing
end

# `sum(tmp; dims=3)` of the rrule when an operand was shared among the products
function batch_sum(tmp::HIPArray{T,3}) where {T<:HIPFloat}
    out = similar(tmp, T, (size(tmp, 1), size(tmp, 2), 1))
    check(ccall((:luxhip_batch_sum, libluxhip), Cint, (Ptr{Cvoid}, Cint, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), size(tmp, 1) * size(tmp, 2), size(tmp, 3), optr(tmp), optr(out))) || throw(HIPFallbackError("sum over the batch dim"))
    return out
end

# ---------------------------------------------------------------------------------------------
# dropout: the device generator stands in for `rand!(rng, y)`  (impl/dropout.jl:171-228)
# ---------------------------------------------------------------------------------------------
mutable struct PhiloxRNG <: Random.AbstractRNG      # what LuxCore.replicate copies
    seed::UInt64
    offset::UInt64
end
Base.copy(r::PhiloxRNG) = PhiloxRNG(r.seed, r.offset)

function Random.rand!(rng::PhiloxRNG, y::HIPArray{T}) where {T<:HIPFloat}
    check(ccall((:luxhip_rand_uniform, libluxhip), Cint, (Ptr{Cvoid}, Cint, Int64, UInt64, UInt64, Ptr{Cvoid}),
        stream(), dtype_code(T), length(y), rng.seed, rng.offset, optr(y))) || error(last_error())
    rng.offset += cld(length(y), 4)
    return y
end

function Impl.generate_dropout_mask!(y::HIPArray{T}, ::HIPOp, p, invp) where {T<:HIPFloat}
    check(ccall((:luxhip_dropout_mask, libluxhip), Cint, (Ptr{Cvoid}, Cint, Int64, Cdouble, Cdouble, Ptr{Cvoid}),
        stream(), dtype_code(T), length(y), Float64(p), Float64(invp), optr(y))) || throw(HIPFallbackError("generate_dropout_mask!"))
    return nothing
end

function Impl.dropout_dot_mul(x::HIPArray{T,N}, mask::HIPArray{T,N}) where {T<:HIPFloat,N}
    y = similar(x)
    xs, ms = Int64[size(x)...], Int64[size(mask)...]
    check(ccall((:luxhip_dropout_mul, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), N, xs, ms, optr(x), optr(mask), optr(y))) || throw(HIPFallbackError("dropout_dot_mul"))
    return y
end

# full-size masks: noise, mask and product in one pass (impl/dropout.jl:3-6 with dims = :)
function Impl.dropout(rng::PhiloxRNG, x::HIPArray{T}, p::P, ::True, invp::P, ::Colon) where {T<:HIPFloat,P}
    rngₙ = copy(rng)
    y, mask = similar(x), similar(x)
    check(ccall((:luxhip_dropout_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Int64, UInt64, UInt64, Cdouble, Cdouble, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), length(x), rngₙ.seed, rngₙ.offset, Float64(p), Float64(invp), optr(x), optr(y), optr(mask))) ||
        error(last_error())
    rngₙ.offset += cld(length(x), 4)
    return y, mask, rngₙ
end
# its pullback is dropout_dot_mul(Δ, mask), as in the reference's rrule (impl/dropout.jl:222-228)

function Impl.alpha_dropout(::HIPOp, noise::HIPArray{T}, p, x::HIPArray{T}, α, A, B) where {T<:HIPFloat}
    y = similar(x)
    check(ccall((:luxhip_alpha_dropout_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Int64, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}, Cdouble, Cdouble, Cdouble, Ptr{Cvoid}),
        stream(), dtype_code(T), length(x), optr(noise), Float64(p), optr(x), Float64(α), Float64(A), Float64(B), optr(y))) ||
        throw(HIPFallbackError("alpha_dropout"))
    return y
end
function CRC.rrule(::typeof(Impl.alpha_dropout), op::HIPOp, noise::HIPArray{T}, p, x::HIPArray{T}, α, A, B) where {T<:HIPFloat}
    y = Impl.alpha_dropout(op, noise, p, x, α, A, B)
    function ∇alpha_dropout_hip(Δ′)
        Δ = CRC.unthunk(Δ′)
        ∂x = similar(x)
        check(ccall((:luxhip_alpha_dropout_bwd, libluxhip), Cint,
            (Ptr{Cvoid}, Cint, Int64, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}),
            stream(), dtype_code(T), length(x), optr(noise), Float64(p), optr(Δ), Float64(A), optr(∂x))) ||
            throw(HIPFallbackError("the pullback of alpha_dropout"))
        return (ntuple(Returns(NoTangent()), 4)..., ∂x, ntuple(Returns(NoTangent()), 3)...)
    end
    return y, ∇alpha_dropout_hip
end

# ---------------------------------------------------------------------------------------------
# scaled_dot_product_attention (impl/attention.jl:5-117): two strided batched products around the fused
# scale / mask / bias / softmax pass; grouped key/value heads are addressed with a stride of 0 along the
# repeat (no repeat_inner_gqa copy); a causal mask is passed to the products as a triangular structure.
# Covers head_dim = 1 (embedding dim first) with the token dim in position 2 or 3; other placements are
# brought there with luxhip_permute_leading3 and the gradients taken back.
# ---------------------------------------------------------------------------------------------
struct AttnLayout
    E::Int; tokens::Int; heads::Int; st::Int; sh::Int; sb::Int; batch::Int
end
function AttnLayout(a::HIPArray, token_dim::Int)
    E, d2, d3 = size(a, 1), size(a, 2), size(a, 3)
    tokens, heads = token_dim == 2 ? (d2, d3) : (d3, d2)
    st, sh = token_dim == 2 ? (E, E * d2) : (E * d2, E)
    sb = E * d2 * d3
    return AttnLayout(E, tokens, heads, st, sh, sb, sb == 0 ? 0 : length(a) ÷ sb)
end
i64x3(t) = Int64[t[1], t[2], t[3]]

# LUXHIP_BF16_WIDE: bf16 operands with the attention logits and the cotangent of the weights in fp32
const BF16_WIDE = Cint(2)
wide_type(::Type{T}) where {T} = T === Core.BFloat16 ? Float32 : T
wide_code(::Type{T}, ::Type{TW}) where {T,TW} = (T === Core.BFloat16 && TW === Float32) ? BF16_WIDE : dtype_code(T)

function bmm_strided!(C::HIPArray{TC}, tA::Bool, tB::Bool, M, N, K, bdims, A::HIPArray{T}, lda, sA, B::HIPArray{T}, ldb, sB, ldc, sC,
        structure::Integer) where {T<:HIPFloat,TC<:HIPFloat}
    check(ccall((:luxhip_batched_matmul_strided, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Cint, Int64, Int64, Int64, Ptr{Int64}, Ptr{Cvoid}, Int64, Ptr{Int64}, Ptr{Cvoid}, Int64, Ptr{Int64},
            Ptr{Cvoid}, Int64, Ptr{Int64}, Cint),
        stream(), wide_code(T, TC), Cint(tA), Cint(tB), M, N, K, i64x3(bdims), optr(A), max(1, lda), i64x3(sA), optr(B), max(1, ldb),
        i64x3(sB), optr(C), max(1, ldc), i64x3(sC), Cint(structure))) || throw(HIPFallbackError("batched_matmul"))
    return C
end

function permute_leading3(a::HIPArray{T,N}, perm::NTuple{3,Int}) where {T<:HIPFloat,N}
    out = similar(a, T, (size(a, perm[1]), size(a, perm[2]), size(a, perm[3]), size(a)[4:N]...))
    check(ccall((:luxhip_permute_leading3, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Int64, Cint, Cint, Cint, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), size(a, 1), size(a, 2), size(a, 3), prod(size(a)[4:N]; init=1), Cint(perm[1]), Cint(perm[2]),
        Cint(perm[3]), optr(a), optr(out))) || throw(HIPFallbackError("permutedims"))
    return out
end

# mask: HIPArray{UInt8} or nothing; bias: HIPArray{T} or nothing; both [S, L, H or 1, B or 1]
function side_strides(a, S, L, H, B)
    a === nothing && return 0, 0
    s3 = ndims(a) ≥ 3 ? size(a, 3) : 1
    s4 = ndims(a) ≥ 4 ? prod(size(a)[4:end]) : 1
    (size(a, 1) == S && size(a, 2) == L && s3 in (1, H) && s4 in (1, B)) ||
        throw(DimensionMismatch("mask / bias of size $(size(a)) does not broadcast to the logits $((S, L, H, B))"))
    return (s3 == H && H > 1 ? S * L : 0), (s4 == B && B > 1 ? S * L * s3 : 0)
end

function attention_device(q::HIPArray{T,N}, k::HIPArray{T,N}, v::HIPArray{T,N}, token_dim::Int, scale, mask, causal::Bool, bias,
        fdrop::F) where {T<:HIPFloat,N,F}
    lq, lk, lv = AttnLayout(q, token_dim), AttnLayout(k, token_dim), AttnLayout(v, token_dim)
    E, Ev, H, G, L, S, B = lq.E, lv.E, lq.heads, lk.heads, lq.tokens, lk.tokens, lq.batch
    r = G == 0 ? 1 : H ÷ G
    bshape = size(q)[4:N]
    scale⁻¹ = 1 / (scale === nothing ? sqrt(Float64(E)) : Float64(scale))                  # impl/attention.jl:50-51
    bdims = (r, G, B)
    mask_sh, mask_sb = side_strides(mask, S, L, H, B)
    bias_sh, bias_sb = side_strides(bias, S, L, H, B)
    sC = (S * L, S * L * r, S * L * H)
    sq = (lq.sh, lq.sh * r, lq.sb)
    tri = causal && fdrop === identity        # an arbitrary fdrop need not keep the masked weights at zero
    TW = wide_type(T)                         # bf16: logits in fp32 (see luxhip.h, attention)
    logits = similar(q, TW, (S, L, H, bshape...))
    bmm_strided!(logits, true, false, S, L, E, bdims, k, lk.st, (0, lk.sh, lk.sb), q, lq.st, sq, S, sC, causal ? 1 : 0)
    softmaxed = similar(q, T, (S, L, H, bshape...))
    check(ccall((:luxhip_attention_softmax_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Int64, Ptr{Cvoid}, Cdouble, Cint, Ptr{UInt8}, Int64, Int64, Ptr{Cvoid}, Int64, Int64,
            Ptr{Cvoid}),
        stream(), wide_code(T, TW), S, L, H, B, optr(logits), scale⁻¹, Cint(causal), mask === nothing ? Ptr{UInt8}(C_NULL) : Ptr{UInt8}(pointer(mask)),
        mask_sh, mask_sb, optr(bias), bias_sh, bias_sb, optr(softmaxed))) || throw(HIPFallbackError("softmax of the attention logits"))
    probs, fdrop_back = fdrop === identity ? (softmaxed, nothing) : CRC.rrule_via_ad(ZygoteLikeConfig(), fdrop, softmaxed)
    so = (Ev, Ev * r, Ev * H * L)
    # bf16 without an fdrop: the product is written unrounded (fp32) and kept for the pullback, whose softmax rule takes
    # its inner product from it; the array that is returned is its rounded copy
    out_wide = (fdrop === identity && TW !== T) ? similar(q, TW, (Ev, H, L, bshape...)) : nothing
    out = out_wide === nothing ? similar(q, T, (Ev, H, L, bshape...)) : out_wide
    bmm_strided!(out, false, false, Ev, L, S, bdims, v, lv.st, (0, lv.sh, lv.sb), probs, S, sC, Ev * H, so, tri ? 2 : 0)
    if out_wide !== nothing
        out = similar(q, T, (Ev, H, L, bshape...))
        check(ccall((:luxhip_convert, libluxhip), Cint, (Ptr{Cvoid}, Cint, Cint, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
            stream(), dtype_code(TW), dtype_code(T), length(out), optr(out_wide), optr(out))) || error(last_error())
    end
    saved = (; lq, lk, lv, r, bdims, sC, sq, so, scale⁻¹, tri, logits, softmaxed, probs, fdrop_back, out_wide)
    return out, probs, saved
end
# the rule configuration `fdrop`'s own pullback is taken with: whatever AD engine drives LuxLib supplies it
struct ZygoteLikeConfig <: CRC.RuleConfig{Union{CRC.HasReverseMode,CRC.NoForwardsMode}} end

function attention_canonical(f, q::HIPArray{T,N}, k, v, head_dim::Int, token_dim::Int) where {T,N}
    head_dim == 1 && return f(q, k, v, token_dim, identity)
    heads_dim = only(setdiff(1:3, (head_dim, token_dim)))
    perm = (head_dim, heads_dim, token_dim)
    inv = ntuple(d -> findfirst(==(d), perm), 3)
    return f(permute_leading3(q, perm), permute_leading3(k, perm), permute_leading3(v, perm), 3, g -> permute_leading3(g, inv))
end

function attention_checks(q::HIPArray{T,N}, k, v, head_dim, token_dim, mask, is_causal) where {T,N}
    # impl/attention.jl:16-43
    @assert N ≥ 4 "N must be at least 4"
    @assert 1 ≤ head_dim ≤ 3 && 1 ≤ token_dim ≤ 3 && head_dim ≠ token_dim "head_dim and token_dim must differ, in 1:3"
    @assert size(q, head_dim) == size(k, head_dim) "`q` and `k` must have the same number of heads."
    for i in 4:N
        (size(q, i) == size(k, i) == size(v, i)) || throw(DimensionMismatch("All dimensions (except first 3) of q, k, v must be the same."))
    end
    @assert !(mask !== nothing && is_causal isa Bool) "`mask` and `is_causal` cannot both be specified"
    return nothing
end

function Impl.scaled_dot_product_attention(q::HIPArray{T,N}, k::HIPArray{T,N}, v::HIPArray{T,N}; head_dim::Int=1, token_dim::Int=3,
        scale=nothing, mask=nothing, is_causal::Union{Bool,Nothing}=nothing, bias=nothing, fdrop::F=identity) where {T<:HIPFloat,N,F}
    attention_checks(q, k, v, head_dim, token_dim, mask, is_causal)
    return attention_canonical(q, k, v, head_dim, token_dim) do qc, kc, vc, td, _
        out, probs, _ = attention_device(qc, kc, vc, td, scale, mask, is_causal === true, bias, fdrop)
        return out, probs
    end
end

function CRC.rrule(::typeof(Impl.scaled_dot_product_attention), q::HIPArray{T,N}, k::HIPArray{T,N}, v::HIPArray{T,N}; head_dim::Int=1,
        token_dim::Int=3, scale=nothing, mask=nothing, is_causal::Union{Bool,Nothing}=nothing, bias=nothing, fdrop::F=identity) where {T<:HIPFloat,N,F}
    attention_checks(q, k, v, head_dim, token_dim, mask, is_causal)
    return attention_canonical(q, k, v, head_dim, token_dim) do qc, kc, vc, td, back_perm
        out, probs, s = attention_device(qc, kc, vc, td, scale, mask, is_causal === true, bias, fdrop)
        (; lq, lk, lv, r, bdims, sC, sq, so, tri) = s
        E, Ev, H, L, S = lq.E, lv.E, lq.heads, lq.tokens, lk.tokens
        function ∇attention_hip(Δ′)
            Δ = CRC.unthunk(Δ′)
            Δout = CRC.unthunk(Δ[1])
            Δ[2] isa CRC.AbstractZero || throw(HIPFallbackError("a cotangent for the returned attention weights"))
            dlogits = eltype(s.logits) === T ? s.logits : similar(probs)   # the logits are no longer needed
            if s.fdrop_back === nothing
                # the cotangent of the weights (v' Δout) and the softmax rule in one call: the cotangent stays in the
                # product's fp32 accumulators, its inner product with the weights comes from Δout and out
                check(ccall((:luxhip_attention_weights_pullback, libluxhip), Cint,
                    (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Ptr{Int64}, Ptr{Cvoid}, Int64, Ptr{Int64}, Ptr{Cvoid}, Ptr{Cvoid}, Int64,
                        Ptr{Int64}, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}, Int64, Ptr{Int64}, Cint),
                    stream(), s.out_wide === nothing ? dtype_code(T) : BF16_WIDE, S, L, Ev, i64x3(bdims), optr(vc), max(1, lv.st),
                    i64x3((0, lv.sh, lv.sb)), optr(Δout), optr(something(s.out_wide, out)), max(1, Ev * H), i64x3(so), optr(s.softmaxed),
                    s.scale⁻¹, optr(dlogits), max(1, S), i64x3(sC),
                    Cint(tri ? 1 : 0))) || error(last_error())
            else
                dp = similar(probs)
                bmm_strided!(dp, true, false, S, L, Ev, bdims, vc, lv.st, (0, lv.sh, lv.sb), Δout, Ev * H, so, S, sC, tri ? 1 : 0)
                dp = CRC.unthunk(s.fdrop_back(dp)[2])
                # tri, not is_causal: with an fdrop the products below run in full and read the whole cotangent
                check(ccall((:luxhip_attention_softmax_bwd, libluxhip), Cint,
                    (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Cint, Ptr{Cvoid}, Ptr{Cvoid}, Cdouble, Ptr{Cvoid}),
                    stream(), dtype_code(T), S, L, L * H * lq.batch, Cint(tri), optr(dp), optr(s.softmaxed), s.scale⁻¹, optr(dlogits))) ||
                    error(last_error())
            end
            ∂q = similar(qc)
            bmm_strided!(∂q, false, false, E, L, S, bdims, kc, lk.st, (0, lk.sh, lk.sb), dlogits, S, sC, lq.st, sq, tri ? 2 : 0)
            function kv_grad(like, lay, A, lda, sA, Bm)
                full = r > 1 ? similar(like, T, (r, size(like)...)) : similar(like)
                bmm_strided!(full, false, true, lay.E, S, L, bdims, A, lda, sA, Bm, S, sC, lay.st,
                    (r > 1 ? length(like) : 0, lay.sh, lay.sb), tri ? 3 : 0)
                r == 1 && return full
                red = similar(like)                               # pullback of repeat_inner_gqa: sum over the heads of a group
                check(ccall((:luxhip_batch_sum, libluxhip), Cint, (Ptr{Cvoid}, Cint, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
                    stream(), dtype_code(T), length(like), r, optr(full), optr(red))) || error(last_error())
                return red
            end
            ∂v = kv_grad(vc, lv, Δout, Ev * H, so, probs)
            ∂k = kv_grad(kc, lk, qc, lq.st, sq, dlogits)
            return NoTangent(), back_perm(∂q), back_perm(∂k), back_perm(∂v)
        end
        return (out, probs), ∇attention_hip
    end
end

# Host-side compositions that the Python mirror (lux.jl_amd/luxlib.py) has and this file does not repeat:
#   * layernorm parameters with gaps between the dims they vary along ((3, 1, 3) against a 4-d x): repeated
#     along the gaps first, gradients summed back (_expand_parameters); here they raise HIPFallbackError;
#   * batched_matmul with lhs_batching_dims / rhs_batching_dims anywhere and partly repeated operands: the
#     arrays' own strides go to luxhip_batched_matmul_strided (_rrule_batched_matmul_general);
#   * operands of mixed element types in fused_dense / fused_conv: luxhip_convert to the widest type first
#     (the reference's own rule, ext/CUDAExt/cublaslt.jl:46-63), gradients converted back (_promote).

end # module
