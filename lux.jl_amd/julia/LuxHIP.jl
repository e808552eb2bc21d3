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
# with the very same argument order and is what the parity tests run.
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
    gemm!(C, A, B, nothing) || invoke(Impl.matmul!, Tuple{AbstractMatrix,Traits.AbstractInternalArrayOpMode,AbstractMatrix,AbstractMatrix}, C, HIPOp(), A, B)
    return nothing
end
function Impl.matmuladd!(C::HIPArray{T,2}, ::HIPOp, A::AbstractMatrix, B::AbstractMatrix, bias::HIPArray{T,1}) where {T<:HIPFloat}
    gemm!(C, A, B, bias) || (C .= bias; Impl.matmul!(C, HIPOp(), A, B))   # reference fallback is C .= bias; mul!(C, A, B, 1, 1)
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

function Impl.fused_dense!(y::HIPArray{T,2}, opmode::HIPOp, act::F, W::HIPArray{T,2}, x::HIPArray{T,2},
        b::Union{Nothing,HIPArray{T,1}}) where {F,T<:HIPFloat}
    if !fused_dense_device!(y, nothing, act, W, x, b)            # -1: warn once, generic path (cublaslt.jl:359-402)
        @warn "libluxhip cannot handle this fused dense call; using the generic path" maxlog = 1
        Impl.matmul!(y, opmode, W, x)
        Impl.bias_activation!(y, opmode, act, y, b)
    end
    return nothing
end

# rrule with the saved pre-activation for activations that need it (precedent: the cuBLASLt AUX
# output used by the gelu rrule, impl/dense.jl:116-134) and a single fused device pullback.
function CRC.rrule(::typeof(Impl.fused_dense), opmode::HIPOp, act::F, W::HIPArray{T,2}, x::HIPArray{T,2},
        b::Union{Nothing,HIPArray{T,1}}) where {F,T<:HIPFloat}
    id = act_id(act)
    id === nothing && return CRC.rrule_via_ad(CRC.NoForwardsMode(), Impl.fused_dense, Traits.GenericBroadcastOp(), act, W, x, b)
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
    ok = id !== nothing && check(ccall((:luxhip_bias_activation_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Int64, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), id, I, C, Nb, optr(x), optr(bias), optr(y), C_NULL))
    ok || broadcast!(σ ∘ +, y, x, Impl.reshape_bias(x, bias))
    return nothing
end
Impl.activation!(y::HIPArray{T,N}, op::HIPOp, σ::F, x::HIPArray{T,N}) where {F,T<:HIPFloat,N} =
    Impl.bias_activation!(y, op, σ, x, nothing)

function Impl.∇activation(::HIPOp, Δ::HIPArray{T,N}, out::HIPArray{T,N}, act::F, x) where {F,T<:HIPFloat,N}
    id = act_id(act)
    id === nothing && return @. Δ * Utils.only_derivative(out, act, x)
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
    act_id(act) === nothing && return invoke(Impl.batchnorm, Tuple{AbstractArray,Any,Any,Any,Any,StaticBool,Any,Any,Any}, x, γ, β, rμ, rσ², training, act, m, ϵ)
    y, rμ′, rσ²′, _, _ = batchnorm_device(x, γ, β, rμ, rσ², known(training), act, m, ϵ, false)
    return y, rμ′, rσ²′
end

function CRC.rrule(::typeof(Impl.batchnorm), x::HIPArray{T,N}, γ, β, rμ, rσ², training::StaticBool, act::F, m, ϵ) where {F,T<:HIPFloat,N}
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

# groupnorm and layernorm follow the same pattern on luxhip_groupnorm_{fwd,bwd} and
# luxhip_layernorm_{fwd,bwd}: a whole-op method on Impl.groupnorm / Impl.layernorm for
# HIPArray that returns y, and an rrule that keeps the saved statistics and makes one device
# call for (∂x, ∂γ, ∂β).  (lux.jl_amd/luxlib.py: rrule_groupnorm, rrule_layernorm.)

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
    ok || return invoke(Impl.conv_bias_act, Tuple{Type,Any,Any,Any,Any,Any}, Nothing, x, w, cdims, bias, act)
    return y
end
function Impl.conv!(y::HIPArray{T,4}, ::Type{LuxHIPDevice}, x::HIPArray{T,4}, w::HIPArray{T,4}, cdims::DenseConvDims{2}) where {T<:HIPFloat}
    d = Ref(ConvDimsC(cdims, size(x, 4)))
    check(ccall((:luxhip_conv_fwd, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), Cint(0), d, optr(x), optr(w), C_NULL, optr(y), C_NULL, C_NULL)) || NNlib.conv!(y, x, w, cdims)
    return nothing
end
function Impl.∇conv_data(dy::HIPArray{T,4}, w::HIPArray{T,4}, cdims::DenseConvDims{2}) where {T<:HIPFloat}
    dx = similar(dy, T, (NNlib.input_size(cdims)..., NNlib.channels_in(cdims), size(dy, 4)))
    d = Ref(ConvDimsC(cdims, size(dy, 4)))
    check(ccall((:luxhip_conv_bwd_data, libluxhip), Cint, (Ptr{Cvoid}, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), d, optr(dy), optr(w), optr(dx))) || return NNlib.∇conv_data(dy, w, cdims)
    return dx
end
function Impl.∇conv_filter(x::HIPArray{T,4}, dy::HIPArray{T,4}, cdims::DenseConvDims{2}) where {T<:HIPFloat}
    dw = similar(x, T, (NNlib.kernel_size(cdims)..., NNlib.channels_in(cdims) ÷ NNlib.groupcount(cdims), NNlib.channels_out(cdims)))
    d = Ref(ConvDimsC(cdims, size(x, 4)))
    check(ccall((:luxhip_conv_bwd_filter, libluxhip), Cint, (Ptr{Cvoid}, Cint, Ptr{ConvDimsC}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), d, optr(x), optr(dy), optr(dw))) || return NNlib.∇conv_filter(x, dy, cdims)
    return dw
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
const DepthSig = (Ptr{Cvoid}, Cint, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Int64, Cint, Ptr{Cvoid}, Ptr{Cvoid})
function depth_unfold(x::HIPArray{T,5}, c::DenseConvDims{3}) where {T<:HIPFloat}
    c2 = inner2d(c, size(x, 5))
    xu = similar(x, T, (NNlib.input_size(c2)..., NNlib.channels_in(c2), NNlib.output_size(c)[3] * size(x, 5)))
    check(ccall((:luxhip_conv_depth_unfold, libluxhip), Cint, DepthSig, stream(), dtype_code(T), depth_args(c, size(x, 5))..., optr(x), optr(xu))) ||
        error("luxhip_conv_depth_unfold")
    return xu, c2
end
function depth_fold(dxu::HIPArray{T,4}, c::DenseConvDims{3}, N::Integer) where {T<:HIPFloat}
    dx = similar(dxu, T, (NNlib.input_size(c)..., NNlib.channels_in(c), N))
    check(ccall((:luxhip_conv_depth_fold, libluxhip), Cint, DepthSig, stream(), dtype_code(T), depth_args(c, N)..., optr(dxu), optr(dx))) ||
        error("luxhip_conv_depth_fold")
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
        bstride(yp), optr(z), max(1, M), M * N)) || NNlib.batched_mul!(z, x, y)
    return nothing
end

# `sum(tmp; dims=3)` of the rrule when an operand was shared among the products
function batch_sum(tmp::HIPArray{T,3}) where {T<:HIPFloat}
    out = similar(tmp, T, (size(tmp, 1), size(tmp, 2), 1))
    check(ccall((:luxhip_batch_sum, libluxhip), Cint, (Ptr{Cvoid}, Cint, Int64, Int64, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), size(tmp, 1) * size(tmp, 2), size(tmp, 3), optr(tmp), optr(out))) || return sum(tmp; dims=3)
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
        stream(), dtype_code(T), length(y), Float64(p), Float64(invp), optr(y))) || (y .= (y .> T(p)) .* T(invp))
    return nothing
end

function Impl.dropout_dot_mul(x::HIPArray{T,N}, mask::HIPArray{T,N}) where {T<:HIPFloat,N}
    y = similar(x)
    xs, ms = Int64[size(x)...], Int64[size(mask)...]
    check(ccall((:luxhip_dropout_mul, libluxhip), Cint,
        (Ptr{Cvoid}, Cint, Cint, Ptr{Int64}, Ptr{Int64}, Ptr{Cvoid}, Ptr{Cvoid}, Ptr{Cvoid}),
        stream(), dtype_code(T), N, xs, ms, optr(x), optr(mask), optr(y))) || return x .* mask
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
        return @. muladd(ifelse(noise > p, x, T(α)), T(A), T(B))
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
            (∂x = Δ .* (noise .> p) .* T(A))
        return (ntuple(Returns(NoTangent()), 4)..., ∂x, ntuple(Returns(NoTangent()), 3)...)
    end
    return y, ∇alpha_dropout_hip
end

# instancenorm (impl/normalization.jl:191-208) is Impl.groupnorm with G = C, followed in training
# with running statistics by luxhip_instancenorm_running_stats on the saved (C, N) statistics;
# scaled_dot_product_attention (impl/attention.jl:70-117) is two luxhip_batched_matmul_strided
# calls around luxhip_attention_softmax_fwd, its rrule four products around
# luxhip_attention_softmax_bwd.  (lux.jl_amd/luxlib.py: rrule_instancenorm,
# rrule_scaled_dot_product_attention spell out the strides.)
#
# The same file holds the host side of what the hooks above do not cover one to one:
#   * layernorm over 1:k with parameters that do not span exactly those dims (dims = Colon() with
#     (1, 1, C, 1) parameters, dims = nothing): luxhip_layernorm_fwd without γ, β, then the per-channel
#     affine transform and activation as luxhip_batchnorm_fwd in inference mode (mean 0, variance 1,
#     ε = 0) on the (I, C, N) view; the pullback runs the two in reverse (_layernorm_fwd);
#   * attention operands whose embedding dim is not the first: luxhip_permute_leading3 before, and on
#     ∂q, ∂k, ∂v after; `fdrop` between the softmax and the second product (attention_dropout);
#   * batched_matmul with lhs_batching_dims / rhs_batching_dims anywhere and partly repeated operands:
#     the arrays' own strides go to luxhip_batched_matmul_strided, no permutedims / repeat
#     (_rrule_batched_matmul_general);
#   * operands of mixed element types in fused_dense / fused_conv: luxhip_convert to the widest type
#     first (the reference's own rule, ext/CUDAExt/cublaslt.jl:46-63), gradients converted back (_promote).

end # module
