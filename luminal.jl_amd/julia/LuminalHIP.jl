# LuminalHIP.jl — Julia glue between Luminal.jl and libluminal_hip.so (MI355X / gfx950).
#
# Nothing in Luminal.jl is edited. This module adds
#   * a device type          HIPDevice <: Luminal.AbstractDevice     (src/Device.jl:9-16)
#   * a device array type    HipArray{T,N} (pointer + dims, freed by a finalizer)
#   * to_device / from_device methods                                  (src/Device.jl:82-105)
#   * execute_op / execute_op! methods for FlashAttentionOp on HipArray arguments; multiple
#     dispatch prefers them over the generic method at src/Execution.jl:565-578
#   * an execute_with_capture method that records a step into a HIP graph     (src/Device.jl:108-121)
#   * DecodeAttentionOp + decode_attention, the fused form of the cached single-token attention
#     subgraph (src/Whisper.jl:584-620) with the GQA head sharing of src/NN.jl:305-317
#   * RotaryEmbeddingOp / KVAppendOp graph nodes (apply_rotary_embeddings, src/NN.jl:253-303; _kv_scatter,
#     src/Whisper.jl:552-570) whose positions are device tensors, so one graph serves every decode position
#   * the array methods Luminal's interpreter and compiled graphs apply to whatever to_device returned
#     (length, reshape, similar, copyto!: src/Execution.jl:92-97, :253; src/Compiler.jl:82-90)
#   * compile_hip(graph): Luminal.compile (src/Compiler.jl:181-255) with the node buffers on the device,
#     returning Luminal's own CompiledGraph
#   * a host fallback for every other op of Luminal's (MatMul, Reshape, Permute, Add ... src/Execution.jl:216-250):
#     on HipArray arguments it downloads them, runs Luminal's own CPU method and uploads the result, so a model
#     graph executes on a HIPDevice with attention on the GPU and the rest where the reference computes it
#   * self_attention(sa, x, prev_seq): Luminal.NN.SelfAttention's own projections and reshapes
#     (src/NN.jl:343-361, :383-386) around the fused attention core instead of src/NN.jl:362-382
# and calls the C ABI of include/luminal_hip.h through `ccall`. There are no AMDGPU.jl kernels here.
#
# Layout: Luminal tensors are column-major (B,H,S,D) arrays (B fastest). The library takes
# row-major [B,H,S,D] (D contiguous), which is the memory order of a column-major (D,S,H,B) array,
# so upload is permutedims(x, (4,3,2,1)) and download is the inverse permutation.
module LuminalHIP

using Luminal
using InteractiveUtils: subtypes
import Luminal: AbstractDevice, Op, FlashAttentionOp, GraphTensor, add_op!, realized_dims, eval_dim, realize_view,
                to_device, from_device, execute_op, execute_op!, execute_with_capture
# Luminal exports an Op called `Function`; the Julia type is always written Base.Function here.

const libluminal_hip = get(ENV, "LUMINAL_HIP_LIB", joinpath(@__DIR__, "..", "lib", "libluminal_hip.so"))

# element type codes of include/luminal_hip.h
const LMH_F32, LMH_F16, LMH_BF16 = Int32(0), Int32(1), Int32(2)
const HEADMAP_INTERLEAVED, HEADMAP_BLOCKED = Int32(0), Int32(1)
# bf16 tensors are carried as UInt16 bit patterns (Julia has no native BFloat16 array type)
struct BF16Bits; bits::UInt16; end
function BF16Bits(x::Float32)           # round to nearest even, NaN stays NaN
    u = reinterpret(UInt32, x)
    isnan(x) && return BF16Bits(((u >> 16) | 0x00000040) % UInt16)
    return BF16Bits(((u + 0x00007fff + ((u >> 16) & 0x00000001)) >> 16) % UInt16)
end
Base.Float32(b::BF16Bits) = reinterpret(Float32, UInt32(b.bits) << 16)
dtype_code(::Type{Float32}) = LMH_F32
dtype_code(::Type{Float16}) = LMH_F16
dtype_code(::Type{BF16Bits}) = LMH_BF16

check(rc::Integer) = rc == 0 ? nothing :
    error("libluminal_hip: ", unsafe_string(ccall((:lmh_last_error, libluminal_hip), Cstring, ())), " (code $rc)")

struct HIPDevice <: AbstractDevice
    index::Int
end
HIPDevice() = HIPDevice(0)

"Health check in the style of get_device(): true when a gfx950 device answers a tiny allocation."
function functional()
    try
        ccall((:lmh_device_count, libluminal_hip), Cint, ()) > 0 || return false
        return ccall((:lmh_init, libluminal_hip), Cint, (Cint,), 0) == 0
    catch
        return false
    end
end

"Best device: HIPDevice when the library finds an MI355X, otherwise whatever Luminal picks."
get_device() = functional() ? HIPDevice(0) : Luminal.get_device()

# ------------------------------------------------------------------------------------------
# device arrays
# ------------------------------------------------------------------------------------------
mutable struct HipArray{T,N}
    ptr::Ptr{Cvoid}
    dims::NTuple{N,Int}      # logical Luminal dims, e.g. (B,H,S,D)
    parent::Any              # nothing for an owning array; the owner for a reshaped view
    function HipArray{T,N}(dims::NTuple{N,Int}) where {T,N}
        p = Ref{Ptr{Cvoid}}(C_NULL)
        check(ccall((:lmh_malloc, libluminal_hip), Cint, (Ptr{Ptr{Cvoid}}, Csize_t), p, max(prod(dims), 1) * sizeof(T)))
        a = new{T,N}(p[], dims, nothing)
        finalizer(x -> ccall((:lmh_free, libluminal_hip), Cint, (Ptr{Cvoid},), x.ptr), a)
        return a
    end
    # same memory under other dims (Base.reshape); frees nothing and keeps the owner reachable
    HipArray{T,N}(ptr::Ptr{Cvoid}, dims::NTuple{N,Int}, owner) where {T,N} = new{T,N}(ptr, dims, owner)
end
# ---- what Luminal applies to its arrays on the interpreter and compiled paths ----
# length: src/Execution.jl:95, src/Compiler.jl:86; similar: src/Execution.jl:253; size / ndims / eltype: executors
Base.size(a::HipArray) = a.dims
Base.size(a::HipArray, i::Integer) = a.dims[i]
Base.length(a::HipArray) = prod(a.dims)
Base.ndims(::HipArray{T,N}) where {T,N} = N
Base.eltype(::HipArray{T}) where {T} = T
Base.similar(a::HipArray{T,N}) where {T,N} = HipArray{T,N}(a.dims)
Base.similar(a::HipArray{T}, dims::NTuple{N,Int}) where {T,N} = HipArray{T,N}(dims)
owner(a::HipArray) = a.parent === nothing ? a : a.parent

"Freshly allocated, zero-filled device array (zeros(T, dims...) of src/Compiler.jl:227)."
function zeros_hip(::Type{T}, dims::NTuple{N,Int}) where {T,N}
    a = HipArray{T,N}(dims)
    check(ccall((:lmh_memset, libluminal_hip), Cint, (Ptr{Cvoid}, Cint, Csize_t, Ptr{Cvoid}),
                a.ptr, 0, max(prod(dims), 1) * sizeof(T), C_NULL))
    return a
end

# Host values in the element type of the device array.
to_storage(::Type{T}, x::AbstractArray) where {T} = eltype(x) === T ? x : convert_elements(T, x)
convert_elements(::Type{T}, x::AbstractArray) where {T<:Number} = T.(x)
convert_elements(::Type{BF16Bits}, x::AbstractArray{UInt16}) = BF16Bits.(x)       # already bit patterns
convert_elements(::Type{BF16Bits}, x::AbstractArray) = BF16Bits.(Float32.(x))      # values: round to bf16

# Column-major (d1 fastest) host array -> the same values with the dimension order reversed, i.e. the
# memory order of row-major [d1, ..., dN] (dN contiguous), and back.
reverse_dims(x::AbstractArray{T,N}) where {T,N} = N <= 1 ? Array(x) : Array(permutedims(x, ntuple(i -> N + 1 - i, N)))

"Host array -> device, reversing the dimension order so that D becomes the contiguous axis."
function to_device(data::AbstractArray{T,N}, ::HIPDevice) where {T,N}
    host = reverse_dims(data)
    dev = HipArray{T,N}(size(data))
    check(ccall((:lmh_memcpy_h2d, libluminal_hip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                dev.ptr, host, sizeof(host), C_NULL))
    return dev
end
to_device(data::HipArray, ::HIPDevice) = data

"Device -> host; synchronises like Array(::CuArray)."
function from_device(a::HipArray{T,N}) where {T,N}
    host = Array{T,N}(undef, reverse(a.dims))
    check(ccall((:lmh_memcpy_d2h, libluminal_hip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                host, a.ptr, sizeof(host), C_NULL))
    return reverse_dims(host)
end

# Base.reshape(data, dims...) is the first thing realize_view does to every node input (src/Execution.jl:94-97,
# :101-104; called at :639 and src/Compiler.jl:252). Equal dims (the buffer "already matches logical size") and
# dims that differ only in singleton axes are the same memory: a view that keeps the owner alive. A reshape
# that regroups axes is a different permutation of a row-major buffer than of Julia's column-major arrays, so
# it goes through the host (correct, slow, and no longer a view).
Base.reshape(a::HipArray, dims::Int...) = Base.reshape(a, dims)
function Base.reshape(a::HipArray{T}, dims::NTuple{N,Int}) where {T,N}
    prod(dims) == length(a) ||
        throw(DimensionMismatch("reshape: HipArray of size $(a.dims) has $(length(a)) elements, $(dims) needs $(prod(dims))"))
    dims == a.dims && return a
    if [d for d in dims if d != 1] == [d for d in a.dims if d != 1]
        return HipArray{T,N}(a.ptr, dims, owner(a))
    end
    cache_capturing() && error("reshape of a HipArray from $(a.dims) to $(dims) regroups axes: it goes through the host and " *
                               "cannot be part of a recorded HIP graph")
    return to_device(Base.reshape(from_device(a), dims), HIPDevice())
end
"true when `v` is `a` itself or a view of `a`'s memory (what compile_hip requires of captured step arguments)"
same_memory(v::HipArray, a::HipArray) = v.ptr == a.ptr && length(v) == length(a)
same_memory(v, a) = v === a

# copyto!(cg.results[k], v) is how a compiled graph takes its inputs (src/Compiler.jl:82-90), and how compile
# fills constants (:229-234). Like copyto! between Arrays it copies in linear (column-major) order.
function Base.copyto!(dst::HipArray{T,N}, src::AbstractArray) where {T,N}
    length(src) == length(dst) ||
        throw(DimensionMismatch("copyto!: HipArray has $(length(dst)) elements, the source $(length(src))"))
    shaped = size(src) == dst.dims ? src : Base.reshape(src, dst.dims)
    host = reverse_dims(to_storage(T, shaped))
    check(ccall((:lmh_memcpy_h2d, libluminal_hip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                dst.ptr, host, sizeof(host), C_NULL))
    return dst
end
function Base.copyto!(dst::HipArray{T}, src::HipArray{T}) where {T}
    length(src) == length(dst) ||
        throw(DimensionMismatch("copyto!: HipArray has $(length(dst)) elements, the source $(length(src))"))
    [d for d in dst.dims if d != 1] == [d for d in src.dims if d != 1] ||
        error("copyto! between HipArrays of sizes $(src.dims) and $(dst.dims) would regroup axes; reshape on the host")
    check(ccall((:lmh_memcpy_d2d, libluminal_hip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}, Csize_t, Ptr{Cvoid}),
                dst.ptr, src.ptr, length(dst) * sizeof(T), current_stream()))
    return dst
end
Base.copyto!(dst::Array, src::HipArray) = copyto!(dst, from_device(src))

# ------------------------------------------------------------------------------------------
# parameter blocks (field order and types mirror include/luminal_hip.h)
# ------------------------------------------------------------------------------------------
struct AttnParams
    out::Ptr{Cvoid}; q::Ptr{Cvoid}; k::Ptr{Cvoid}; v::Ptr{Cvoid}; kv_len::Ptr{Int32}
    B::Int32; Hq::Int32; Hkv::Int32; Sq::Int32; Sk::Int32; D::Int32
    q_stride::NTuple{3,Int64}; k_stride::NTuple{3,Int64}; v_stride::NTuple{3,Int64}; o_stride::NTuple{3,Int64}
    dtype::Int32; scale::Float32; causal::Int32; head_map::Int32; out_f32::Int32
    stream::Ptr{Cvoid}
    q_rope::Int32; q_rope_pairing::Int32; q_pos0::Ptr{Int32}; q_prev_seq::Int32; q_rope_base::Float32
end
# the trailing fields of AttnParams for "no rotary embedding of the queries"
const NO_Q_ROPE = (Int32(0), Int32(0), Ptr{Int32}(C_NULL), Int32(0), 0.0f0)

struct DecodeParams
    out::Ptr{Cvoid}; q::Ptr{Cvoid}; k_cache::Ptr{Cvoid}; v_cache::Ptr{Cvoid}; kv_len::Ptr{Int32}
    B::Int32; Hq::Int32; Hkv::Int32; Lmax::Int32; D::Int32
    q_stride::NTuple{2,Int64}; o_stride::NTuple{2,Int64}; k_stride::NTuple{3,Int64}; v_stride::NTuple{3,Int64}
    dtype::Int32; scale::Float32; head_map::Int32; out_f32::Int32; num_splits::Int32
    workspace::Ptr{Cvoid}; workspace_bytes::Csize_t
    stream::Ptr{Cvoid}
end

# The stream every executor below enqueues on: the null stream, except while execute_with_capture records.
const _stream = Ref{Ptr{Cvoid}}(C_NULL)
current_stream() = _stream[]

const Z3 = (Int64(0), Int64(0), Int64(0))   # all-zero strides = contiguous
const Z2 = (Int64(0), Int64(0))

# ------------------------------------------------------------------------------------------
# FlashAttentionOp on device arrays
# ------------------------------------------------------------------------------------------
function execute_op!(out::HipArray{TO,4}, op::FlashAttentionOp, q::HipArray{T,4}, k::HipArray{T,4}, v::HipArray{T,4};
                     head_map::Int32=HEADMAP_INTERLEAVED, kv_len::Union{Nothing,HipArray{Int32,1}}=nothing,
                     q_rope_base=nothing, q_prev_seq::Integer=0,
                     q_pos0::Union{Nothing,HipArray{Int32,1}}=nothing) where {TO,T}
    B, Hq, Sq, D = size(q)
    _, Hkv, Sk, _ = size(k)
    size(out) == size(q) || error("FlashAttentionOp: output shape $(size(out)) differs from q shape $(size(q))")
    # q_rope_base: the kernel rotates the query rows as it loads them (apply_rotary_embeddings on the queries,
    # src/NN.jl:357), row i of sequence b at position (q_pos0 === nothing ? q_prev_seq : q_pos0[b]) + i
    rope = q_rope_base === nothing ? NO_Q_ROPE :
           (Int32(1), Int32(0), q_pos0 === nothing ? Ptr{Int32}(C_NULL) : Ptr{Int32}(q_pos0.ptr), Int32(q_prev_seq), Float32(q_rope_base))
    p = Ref(AttnParams(out.ptr, q.ptr, k.ptr, v.ptr, kv_len === nothing ? Ptr{Int32}(C_NULL) : Ptr{Int32}(kv_len.ptr),
                       B, Hq, Hkv, Sq, Sk, D, Z3, Z3, Z3, Z3,
                       dtype_code(T), op.scale, Int32(op.causal), head_map, Int32(TO === Float32 && T !== Float32), current_stream(),
                       rope...))
    check(ccall((:lmh_flash_attn_fwd, libluminal_hip), Cint, (Ref{AttnParams},), p))
    return out
end

"""
    flash_attention_plan(op, q, k, v) -> String

Names the kernel (instantiation, workgroup count) that `execute_op!` would launch for these arrays; launches nothing.
"""
function flash_attention_plan(op::FlashAttentionOp, q::HipArray{T,4}, k::HipArray{T,4}, v::HipArray{T,4};
                              head_map::Int32=HEADMAP_INTERLEAVED) where {T}
    B, Hq, Sq, D = size(q)
    _, Hkv, Sk, _ = size(k)
    p = Ref(AttnParams(q.ptr, q.ptr, k.ptr, v.ptr, C_NULL, B, Hq, Hkv, Sq, Sk, D, Z3, Z3, Z3, Z3,
                       dtype_code(T), op.scale, Int32(op.causal), head_map, Int32(0), C_NULL, NO_Q_ROPE...))
    text = Vector{UInt8}(undef, 256)
    check(ccall((:lmh_flash_attn_plan, libluminal_hip), Cint, (Ref{AttnParams}, Ptr{UInt8}, Csize_t), p, text, length(text)))
    return GC.@preserve text unsafe_string(pointer(text))
end

function execute_op(op::FlashAttentionOp, q::HipArray, k::HipArray, v::HipArray)
    out = similar(q)                      # src/Execution.jl:252-255
    return execute_op!(out, op, q, k, v)
end

# ------------------------------------------------------------------------------------------
# DecodeAttentionOp: q (B,H,D); caches (B,Hkv,max_seq,D) like KVCacheState (src/Whisper.jl:519-540);
# kv_len (B,) Int32 on the device — a tensor, not a graph constant, so one compiled graph serves
# every decode position (the reference compiles one graph per position, src/Decoding.jl:98-106).
# ------------------------------------------------------------------------------------------
struct DecodeAttentionOp <: Op
    scale::Float32
    head_map::Int32
end

"""
q: (B,H,D), or (B,H,1,D) as the projections of one decode step produce it; caches (B,Hkv,max_seq,D); kv_len (B,)
Int32. The output has q's shape.
"""
function decode_attention(q::GraphTensor, k_cache::GraphTensor, v_cache::GraphTensor, kv_len::GraphTensor;
                          scale=nothing, head_map::Int32=HEADMAP_INTERLEAVED)
    q_dims = realized_dims(q.shape)
    if isnothing(scale)
        scale = 1.0f0 / sqrt(Float32(q_dims[end]))
    end
    inputs = [(q.id, 0, q.shape), (k_cache.id, 0, k_cache.shape), (v_cache.id, 0, v_cache.shape),
              (kv_len.id, 0, kv_len.shape)]
    return add_op!(q.graph_ref, DecodeAttentionOp(Float32(scale), head_map), inputs, q.shape)
end

const _workspace = Ref{Union{Nothing,HipArray{UInt8,1}}}(nothing)
function workspace(bytes::Integer)
    if bytes > 0 && (_workspace[] === nothing || length(_workspace[]) < bytes)
        _workspace[] = HipArray{UInt8,1}((Int(bytes),))
    end
    return _workspace[]
end

function execute_op!(out::HipArray{TO,3}, op::DecodeAttentionOp, q::HipArray{T,3}, kc::HipArray{T,4}, vc::HipArray{T,4},
                     kv_len::HipArray{Int32,1}; static_scratch::Bool=false) where {TO,T}
    B, Hq, D = size(q)
    _, Hkv, Lmax, _ = size(kc)
    out_f32 = Int32(TO === Float32 && T !== Float32)
    if static_scratch
        # lmh_decode_attn_static: no workspace, nothing allocated (split-KV partials in the library's static device array)
        p = Ref(DecodeParams(out.ptr, q.ptr, kc.ptr, vc.ptr, Ptr{Int32}(kv_len.ptr), B, Hq, Hkv, Lmax, D, Z2, Z2, Z3, Z3,
                             dtype_code(T), op.scale, op.head_map, out_f32, Int32(0), C_NULL, Csize_t(0), current_stream()))
        check(ccall((:lmh_decode_attn_static, libluminal_hip), Cint, (Ref{DecodeParams},), p))
        return out
    end
    splits = ccall((:lmh_decode_auto_splits, libluminal_hip), Int32, (Int32, Int32, Int32), B, Hkv, Lmax)
    need = ccall((:lmh_decode_workspace_bytes, libluminal_hip), Csize_t, (Int32, Int32, Int32, Int32, Int32, Int32),
                 B, Hq, Hkv, Lmax, D, splits)
    ws = workspace(need)
    p = Ref(DecodeParams(out.ptr, q.ptr, kc.ptr, vc.ptr, Ptr{Int32}(kv_len.ptr), B, Hq, Hkv, Lmax, D, Z2, Z2, Z3, Z3,
                         dtype_code(T), op.scale, op.head_map, out_f32, splits,
                         ws === nothing ? C_NULL : ws.ptr, need, current_stream()))
    check(ccall((:lmh_decode_attn, libluminal_hip), Cint, (Ref{DecodeParams},), p))
    return out
end

# q and out as (B,H,1,D): the same memory as (B,H,D)
function execute_op!(out::HipArray{TO,4}, op::DecodeAttentionOp, q::HipArray{T,4}, kc::HipArray{T,4}, vc::HipArray{T,4},
                     kv_len::HipArray{Int32,1}; static_scratch::Bool=false) where {TO,T}
    size(q, 3) == 1 || error("DecodeAttentionOp takes one query token per sequence; got q of size $(size(q))")
    size(out) == size(q) || error("DecodeAttentionOp: output shape $(size(out)) differs from q shape $(size(q))")
    dims3 = (size(q, 1), size(q, 2), size(q, 4))
    execute_op!(Base.reshape(out, dims3), op, Base.reshape(q, dims3), kc, vc, kv_len; static_scratch=static_scratch)
    return out
end

execute_op(op::DecodeAttentionOp, q::HipArray, kc::HipArray, vc::HipArray, kv_len::HipArray) =
    execute_op!(similar(q), op, q, kc, vc, kv_len)

# ------------------------------------------------------------------------------------------
# DecodeStepOp: one decode step of a cached attention layer as one node and two launches (lmh_decode_step): what
# decode_step! and whisper_self_attn_cached do for one layer (src/Whisper.jl:761-801, :584-620) with the rotary embedding
# of src/NN.jl:356-358. Inputs (q, k_cache, v_cache, k_new, v_new, pos); the value of the node is the attention result
# over rows 0 .. pos[b] inclusive; the caches are updated in place (row pos[b]; K rotated when rope_base is set); q is
# rotated inside the kernel and left as it was.
# ------------------------------------------------------------------------------------------
struct DecodeStepExtra
    k_new::Ptr{Cvoid}; v_new::Ptr{Cvoid}; rope::Int32; pairing::Int32; rope_base::Float32
end

struct DecodeStepOp <: Op
    scale::Float32
    head_map::Int32
    rope_base::Float32      # 0: no rotary embedding
end

"Whether lmh_decode_step takes this element type and head dim (otherwise: kv_append! + decode attention, three launches)."
decode_step_supported(::Type{T}, head_dim::Integer; rope::Bool=true) where {T} =
    (T === Float16 || T === BF16Bits) && head_dim in (64, 96, 128, 256) && (!rope || iseven(head_dim ÷ 32))

function decode_step(q::GraphTensor, k_cache::GraphTensor, v_cache::GraphTensor, k_new::GraphTensor, v_new::GraphTensor,
                     pos::GraphTensor; scale=nothing, head_map::Int32=HEADMAP_INTERLEAVED, rope_base=nothing)
    q_dims = realized_dims(q.shape)
    s = isnothing(scale) ? 1.0f0 / sqrt(Float32(q_dims[end])) : Float32(scale)
    inputs = [(t.id, 0, t.shape) for t in (q, k_cache, v_cache, k_new, v_new, pos)]
    return add_op!(q.graph_ref, DecodeStepOp(s, head_map, Float32(something(rope_base, 0.0f0))), inputs, q.shape)
end

function execute_op!(out::HipArray{TO,3}, op::DecodeStepOp, q::HipArray{T,3}, kc::HipArray{T,4}, vc::HipArray{T,4},
                     k_new::HipArray{T,4}, v_new::HipArray{T,4}, pos::HipArray{Int32,1}) where {TO,T}
    B, Hq, D = size(q)
    _, Hkv, Lmax, _ = size(kc)
    out_f32 = Int32(TO === Float32 && T !== Float32)
    splits = ccall((:lmh_decode_step_splits, libluminal_hip), Int32, (Int32, Int32, Int32), B, Hkv, Lmax)
    need = ccall((:lmh_decode_workspace_bytes, libluminal_hip), Csize_t, (Int32, Int32, Int32, Int32, Int32, Int32),
                 B, Hq, Hkv, Lmax, D, splits)
    ws = workspace(need)
    p = Ref(DecodeParams(out.ptr, q.ptr, kc.ptr, vc.ptr, Ptr{Int32}(pos.ptr), B, Hq, Hkv, Lmax, D, Z2, Z2, Z3, Z3,
                         dtype_code(T), op.scale, op.head_map, out_f32, splits,
                         ws === nothing ? C_NULL : ws.ptr, need, current_stream()))
    x = Ref(DecodeStepExtra(k_new.ptr, v_new.ptr, Int32(op.rope_base > 0), Int32(0), op.rope_base > 0 ? op.rope_base : 10000.0f0))
    check(ccall((:lmh_decode_step, libluminal_hip), Cint, (Ref{DecodeParams}, Ref{DecodeStepExtra}), p, x))
    return out
end

# q and out as (B,H,1,D): the same memory as (B,H,D)
function execute_op!(out::HipArray{TO,4}, op::DecodeStepOp, q::HipArray{T,4}, kc::HipArray{T,4}, vc::HipArray{T,4},
                     k_new::HipArray{T,4}, v_new::HipArray{T,4}, pos::HipArray{Int32,1}) where {TO,T}
    size(q, 3) == 1 || error("DecodeStepOp takes one query token per sequence; got q of size $(size(q))")
    dims3 = (size(q, 1), size(q, 2), size(q, 4))
    execute_op!(Base.reshape(out, dims3), op, Base.reshape(q, dims3), kc, vc, k_new, v_new, pos)
    return out
end

execute_op(op::DecodeStepOp, q::HipArray, kc::HipArray, vc::HipArray, k_new::HipArray, v_new::HipArray, pos::HipArray) =
    execute_op!(similar(q), op, q, kc, vc, k_new, v_new, pos)

# ------------------------------------------------------------------------------------------
# the operators in front of decode attention
# ------------------------------------------------------------------------------------------
struct RopeParams
    out::Ptr{Cvoid}; x::Ptr{Cvoid}; pos0::Ptr{Int32}; prev_seq::Int32
    B::Int32; H::Int32; S::Int32; D::Int32
    x_stride::NTuple{3,Int64}; o_stride::NTuple{3,Int64}
    dtype::Int32; base::Float32; pairing::Int32
    stream::Ptr{Cvoid}
end

"In-place rotary embedding of a (B,H,S,D) device array; same pairing as apply_rotary_embeddings (src/NN.jl:253-303)."
function rope!(x::HipArray{T,4}; prev_seq::Integer=0, base::Real=10000.0f0,
               pos0::Union{Nothing,HipArray{Int32,1}}=nothing) where {T}
    B, H, S, D = size(x)
    p = Ref(RopeParams(x.ptr, x.ptr, pos0 === nothing ? Ptr{Int32}(C_NULL) : Ptr{Int32}(pos0.ptr), prev_seq, B, H, S, D,
                       Z3, Z3, dtype_code(T), Float32(base), Int32(0), current_stream()))
    check(ccall((:lmh_rope, libluminal_hip), Cint, (Ref{RopeParams},), p))
    return x
end

struct KvAppendParams
    k_cache::Ptr{Cvoid}; v_cache::Ptr{Cvoid}; k_new::Ptr{Cvoid}; v_new::Ptr{Cvoid}; pos::Ptr{Int32}; pos_all::Int32
    B::Int32; Hkv::Int32; T::Int32; D::Int32; Lmax::Int32
    k_stride::NTuple{3,Int64}; v_stride::NTuple{3,Int64}
    dtype::Int32; rope_k::Int32; pairing::Int32; base::Float32
    stream::Ptr{Cvoid}
    q_rope::Ptr{Cvoid}; Hq::Int32
end

"""
cache[b,h,pos[b]+t,:] = new[b,h,t,:] in place (the reference rebuilds the cache with _kv_scatter,
src/Whisper.jl:552-570). With `q` (B,Hq,T,D) the same launch rotates this step's queries in place at the same
positions (apply_rotary_embeddings on the queries, src/NN.jl:356).
"""
function kv_append!(kc::HipArray{T,4}, vc::HipArray{T,4}, k_new::HipArray{T,4}, v_new::HipArray{T,4},
                    pos::HipArray{Int32,1}; rope_k::Bool=false, base::Real=10000.0f0,
                    q::Union{Nothing,HipArray{T,4}}=nothing) where {T}
    B, Hkv, Lmax, D = size(kc)
    p = Ref(KvAppendParams(kc.ptr, vc.ptr, k_new.ptr, v_new.ptr, Ptr{Int32}(pos.ptr), 0, B, Hkv, size(k_new, 3), D, Lmax,
                           Z3, Z3, dtype_code(T), Int32(rope_k), Int32(0), Float32(base), current_stream(),
                           q === nothing ? C_NULL : q.ptr, q === nothing ? Int32(0) : Int32(size(q, 2))))
    check(ccall((:lmh_kv_append, libluminal_hip), Cint, (Ref{KvAppendParams},), p))
    return kc, vc
end

# ------------------------------------------------------------------------------------------
# The same two operators as graph nodes, so that a decode step is a Luminal graph whose positions are
# tensors: one graph (interpreted or compiled) then serves every position, where the reference bakes
# step_pos into the slices of one graph per position (src/Whisper.jl:673-675, src/Decoding.jl:98-106).
# ------------------------------------------------------------------------------------------
"apply_rotary_embeddings(input, prev_seq; base) (src/NN.jl:253-303) as one node; inputs (x,) or (x, pos0)."
struct RotaryEmbeddingOp <: Op
    prev_seq::Int32
    base::Float32
end

"""
x: (B,H,S,D). Row s of sequence b is rotated by position prev_seq + s, or pos0[b] + s when the Int32 (B,)
tensor pos0 is given. Output shape = x's.
"""
function rotary_embedding(x::GraphTensor; prev_seq::Integer=0, base::Real=10000.0f0,
                          pos0::Union{Nothing,GraphTensor}=nothing)
    inputs = [(x.id, 0, x.shape)]
    pos0 === nothing || push!(inputs, (pos0.id, 0, pos0.shape))
    return add_op!(x.graph_ref, RotaryEmbeddingOp(Int32(prev_seq), Float32(base)), inputs, x.shape)
end

function execute_op!(out::HipArray{T,4}, op::RotaryEmbeddingOp, x::HipArray{T,4},
                     pos0::Union{Nothing,HipArray{Int32,1}}=nothing) where {T}
    size(out) == size(x) || error("RotaryEmbeddingOp: output shape $(size(out)) differs from input shape $(size(x))")
    B, H, S, D = size(x)
    p = Ref(RopeParams(out.ptr, x.ptr, pos0 === nothing ? Ptr{Int32}(C_NULL) : Ptr{Int32}(pos0.ptr), op.prev_seq,
                       B, H, S, D, Z3, Z3, dtype_code(T), op.base, Int32(0), current_stream()))
    check(ccall((:lmh_rope, libluminal_hip), Cint, (Ref{RopeParams},), p))
    return out
end
execute_op(op::RotaryEmbeddingOp, x::HipArray, pos0::HipArray...) = execute_op!(similar(x), op, x, pos0...)

"""
In-place cache update as a node; inputs (k_cache, v_cache, k_new, v_new, pos) plus, with rope_q, this step's
queries. The node's value IS its k_cache input (the same buffer, rows pos[b] .. pos[b]+T-1 overwritten, K rotated
on the way in when rope_k); v_cache and the queries are updated in place as well, so later nodes that read them
through their own ids see the new contents — nodes run in graph order (src/Execution.jl:630, src/Compiler.jl:92-96).
"""
struct KVAppendOp <: Op
    rope_k::Bool
    rope_q::Bool
    base::Float32
end

function kv_cache_append(k_cache::GraphTensor, v_cache::GraphTensor, k_new::GraphTensor, v_new::GraphTensor,
                         pos::GraphTensor; rope_k::Bool=false, base::Real=10000.0f0,
                         q::Union{Nothing,GraphTensor}=nothing)
    inputs = [(k_cache.id, 0, k_cache.shape), (v_cache.id, 0, v_cache.shape), (k_new.id, 0, k_new.shape),
              (v_new.id, 0, v_new.shape), (pos.id, 0, pos.shape)]
    q === nothing || push!(inputs, (q.id, 0, q.shape))
    return add_op!(k_cache.graph_ref, KVAppendOp(rope_k, q !== nothing, Float32(base)), inputs, k_cache.shape)
end

function execute_op!(out::HipArray{T,4}, op::KVAppendOp, kc::HipArray{T,4}, vc::HipArray{T,4}, k_new::HipArray{T,4},
                     v_new::HipArray{T,4}, pos::HipArray{Int32,1}, q::Union{Nothing,HipArray{T,4}}=nothing) where {T}
    same_memory(out, kc) || error("KVAppendOp works in place: its output buffer must be its k_cache input")
    (q !== nothing) == op.rope_q || error("KVAppendOp: rope_q is $(op.rope_q) but the node has $(q === nothing ? 5 : 6) inputs")
    kv_append!(kc, vc, k_new, v_new, pos; rope_k=op.rope_k, base=op.base, q=q)
    return out
end
execute_op(op::KVAppendOp, kc::HipArray, rest::HipArray...) = execute_op!(kc, op, kc, rest...)

# ------------------------------------------------------------------------------------------
# What the attention layers do between their projections, as fused calls on device arrays.
# SelfAttention (src/NN.jl:352-382) = rotary embedding of Q and K, repeat_kv, scaled causal softmax
# attention; the fused op reads the Hkv key/value heads directly in the head order repeat_kv produces
# (src/NN.jl:305-317). Whisper's layers (src/Whisper.jl:263-272, :310-312) are the same call without
# rotary embedding, cross attention with causal=false.
# ------------------------------------------------------------------------------------------
# head dims for which the matrix-core attention kernels rotate the queries in registers
const FUSED_ROPE_HEAD_DIMS = (64, 96, 128)

function self_attention_core!(out::HipArray, q::HipArray{T,4}, k::HipArray{T,4}, v::HipArray{T,4}; causal::Bool=true,
                              prev_seq::Integer=0, rope_base=nothing, scale=nothing,
                              head_map::Int32=HEADMAP_INTERLEAVED) where {T}
    s = isnothing(scale) ? 1.0f0 / sqrt(Float32(size(q, 4))) : Float32(scale)
    rope_base === nothing && return execute_op!(out, FlashAttentionOp(s, causal), q, k, v; head_map=head_map)
    rope!(k; prev_seq=prev_seq, base=rope_base)
    if size(q, 4) in FUSED_ROPE_HEAD_DIMS   # q is rotated inside the attention kernel: no launch (and no write) of its own
        return execute_op!(out, FlashAttentionOp(s, causal), q, k, v; head_map=head_map, q_rope_base=rope_base, q_prev_seq=prev_seq)
    end
    rope!(q; prev_seq=prev_seq, base=rope_base)
    return execute_op!(out, FlashAttentionOp(s, causal), q, k, v; head_map=head_map)
end

"""
The prompt pass of a cached attention layer in two launches (the reference runs SelfAttention on the prompt,
src/NN.jl:352-382, and fills its caches by slice + concat, src/Whisper.jl:552-570): the prompt's K/V rows go into the
caches at rows pos[b] .. (K rotated on the way in), then attention reads the caches' first kv_len[b] rows and rotates
the queries as it loads them. The causal mask aligns query row i with cache row i: the prompt starts its cache
(pos[b] = 0, kv_len[b] = T).
"""
function prompt_self_attention_core!(out::HipArray, q::HipArray{T,4}, k_new::HipArray{T,4}, v_new::HipArray{T,4},
                                     kc::HipArray{T,4}, vc::HipArray{T,4}, pos::HipArray{Int32,1}, kv_len::HipArray{Int32,1};
                                     rope_base=nothing, scale=nothing, head_map::Int32=HEADMAP_INTERLEAVED) where {T}
    kv_append!(kc, vc, k_new, v_new, pos; rope_k=(rope_base !== nothing), base=something(rope_base, 10000.0f0))
    s = isnothing(scale) ? 1.0f0 / sqrt(Float32(size(q, 4))) : Float32(scale)
    fused = rope_base !== nothing && size(q, 4) in FUSED_ROPE_HEAD_DIMS
    rope_base !== nothing && !fused && rope!(q; base=rope_base, pos0=pos)
    return execute_op!(out, FlashAttentionOp(s, true), q, kc, vc; head_map=head_map, kv_len=kv_len,
                       q_rope_base=(fused ? rope_base : nothing), q_pos0=(fused ? pos : nothing))
end

"""
One decode step of a cached attention layer (src/Whisper.jl:584-620): q (B,Hq,1,D) and k_new, v_new
(B,Hkv,1,D) are this step's projections, `pos` (B,) the cache row each sequence writes, `kv_len` = pos .+ 1
the rows it then attends over. Both are device arrays, so nothing is recompiled per position
(the reference builds one graph per position, src/Decoding.jl:98-106).
"""
function cached_self_attention_core!(out::HipArray{TO,3}, q::HipArray{T,4}, k_new::HipArray{T,4}, v_new::HipArray{T,4},
                                     kc::HipArray{T,4}, vc::HipArray{T,4}, pos::HipArray{Int32,1},
                                     kv_len::HipArray{Int32,1}; rope_base=nothing, scale=nothing,
                                     head_map::Int32=HEADMAP_INTERLEAVED, fused::Bool=false) where {TO,T}
    size(q, 3) == 1 || error("cached attention takes one query token per sequence")
    if fused && decode_step_supported(T, size(q, 4); rope=(rope_base !== nothing))
        # two launches instead of three: the split kernel rotates q as it loads it, the merge launch adds and stores the new row
        s = isnothing(scale) ? 1.0f0 / sqrt(Float32(size(q, 4))) : Float32(scale)
        q3 = HipArray{T,3}(q.ptr, (size(q, 1), size(q, 2), size(q, 4)), q)
        return execute_op!(out, DecodeStepOp(s, head_map, Float32(something(rope_base, 0.0f0))), q3, kc, vc, k_new, v_new, pos)
    end
    # one launch: the new rows go into the caches (K rotated on the way in) and q is rotated in place
    kv_append!(kc, vc, k_new, v_new, pos; rope_k=(rope_base !== nothing), base=something(rope_base, 10000.0f0),
               q=(rope_base !== nothing ? q : nothing))
    s = isnothing(scale) ? 1.0f0 / sqrt(Float32(size(q, 4))) : Float32(scale)
    q3 = HipArray{T,3}(q.ptr, (size(q, 1), size(q, 2), size(q, 4)), q)   # same memory, (B,Hq,D); keeps q alive
    return execute_op!(out, DecodeAttentionOp(s, head_map), q3, kc, vc, kv_len)
end

# ------------------------------------------------------------------------------------------
# Device-resident decode cache: the self-attention half of KVCacheState (src/Whisper.jl:519-540; one (K, V) pair of
# (B, Hkv, max_seq, D) per layer, zero-filled) with the step of decode_step! (src/Whisper.jl:761-801) that concerns it.
# The reference keeps the caches on the host, feeds them to the step graph as inputs and replaces them by the graph's
# new-cache outputs every step (:775-797); here they stay on the device, a step writes its rows in place, and every
# sequence carries its own length (the reference has one step_pos for the batch).
# ------------------------------------------------------------------------------------------
mutable struct HipKVCache{T}
    max_seq::Int
    self_cache::Vector{Tuple{HipArray{T,4},HipArray{T,4}}}   # per layer, as in KVCacheState
    kv_len_host::Vector{Int32}                               # rows in use, per sequence (the same in every layer)
    pos::HipArray{Int32,1}                                   # device copy of kv_len_host before a step ...
    kv_len::HipArray{Int32,1}                                # ... and after it
end

"HipKVCache{T}(batch, n_layers, n_kv_heads, head_dim; max_seq): zeroed caches for a new decode session (KVCacheState(...), src/Whisper.jl:527-540)."
function HipKVCache{T}(batch::Int, n_layers::Int, n_kv_heads::Int, head_dim::Int; max_seq::Int) where {T}
    caches = [(zeros_hip(T, (batch, n_kv_heads, max_seq, head_dim)), zeros_hip(T, (batch, n_kv_heads, max_seq, head_dim)))
              for _ in 1:n_layers]
    return HipKVCache{T}(max_seq, caches, zeros(Int32, batch), zeros_hip(Int32, (batch,)), zeros_hip(Int32, (batch,)))
end

"The reference's single position (KVCacheState.step_pos): the longest sequence's length."
step_pos(c::HipKVCache) = Int(maximum(c.kv_len_host))

"""
begin_step!(cache, n_new): uploads the rows the next `n_new` tokens of every sequence will occupy (pos = the lengths so
far, kv_len = pos .+ n_new) and returns (pos, kv_len). Call it once per step, before the layers; `advance!` afterwards.
"""
function begin_step!(c::HipKVCache, n_new::Integer=1)
    step_pos(c) + n_new <= c.max_seq || error("KV cache is full (max_seq = $(c.max_seq))")
    copyto!(c.pos, c.kv_len_host)
    copyto!(c.kv_len, c.kv_len_host .+ Int32(n_new))
    return c.pos, c.kv_len
end

"advance!(cache, n_new): the step is done in every layer (cache.step_pos += 1, src/Whisper.jl:799)."
function advance!(c::HipKVCache, n_new::Integer=1)
    c.kv_len_host .+= Int32(n_new)
    return c
end

"""
One layer of a decode step (whisper_self_attn_cached, src/Whisper.jl:584-620): this step's q (B,Hq,1,D) and k_new, v_new
(B,Hkv,1,D) against layer `layer`'s caches, between begin_step! and advance!. With `rope_base` the new K rows and q are
rotated at their positions (src/NN.jl:356-358). Returns out (B,Hq,D).
"""
function decode_layer!(out::HipArray{TO,3}, c::HipKVCache{T}, layer::Integer, q::HipArray{T,4}, k_new::HipArray{T,4},
                       v_new::HipArray{T,4}; rope_base=nothing, scale=nothing, head_map::Int32=HEADMAP_INTERLEAVED,
                       fused::Bool=true) where {TO,T}
    kc, vc = c.self_cache[layer]
    return cached_self_attention_core!(out, q, k_new, v_new, kc, vc, c.pos, c.kv_len; rope_base=rope_base, scale=scale,
                                       head_map=head_map, fused=fused)
end

"The prompt pass of layer `layer` (T tokens per sequence into empty caches), between begin_step!(cache, T) and advance!(cache, T)."
function prompt_layer!(out::HipArray, c::HipKVCache{T}, layer::Integer, q::HipArray{T,4}, k_new::HipArray{T,4},
                       v_new::HipArray{T,4}; rope_base=nothing, scale=nothing, head_map::Int32=HEADMAP_INTERLEAVED) where {T}
    kc, vc = c.self_cache[layer]
    return prompt_self_attention_core!(out, q, k_new, v_new, kc, vc, c.pos, c.kv_len; rope_base=rope_base, scale=scale,
                                       head_map=head_map)
end

# The same two cores as graph builders (GraphTensor in, GraphTensor out), for model code that builds a Luminal graph.
function self_attention_core(q::GraphTensor, k::GraphTensor, v::GraphTensor; causal::Bool=true, prev_seq::Integer=0,
                             rope_base=nothing, scale=nothing)
    # FlashAttentionOp reads the Hkv key/value heads in the order repeat_kv produces (src/NN.jl:305-317)
    rope_base === nothing && return Luminal.flash_attention(q, k, v; scale=scale, causal=causal)
    k = rotary_embedding(k; prev_seq=prev_seq, base=rope_base)
    D = Int(eval_dim(realized_dims(q.shape)[end]))
    if D in FUSED_ROPE_HEAD_DIMS
        return rope_flash_attention(q, k, v; scale=scale, causal=causal, prev_seq=prev_seq, base=rope_base)
    end
    q = rotary_embedding(q; prev_seq=prev_seq, base=rope_base)
    return Luminal.flash_attention(q, k, v; scale=scale, causal=causal)
end

"""
FlashAttentionOp whose queries are rotated inside the kernel: the reference's op carries (scale, causal) only
(src/Ops.jl:104-107), so the fused form is a node type of the glue. Inputs (q, k, v) like FlashAttentionOp.
"""
struct RopeFlashAttentionOp <: Op
    scale::Float32
    causal::Bool
    prev_seq::Int32
    base::Float32
end

function rope_flash_attention(q::GraphTensor, k::GraphTensor, v::GraphTensor; scale=nothing, causal::Bool=false,
                              prev_seq::Integer=0, base::Real=10000.0f0)
    if isnothing(scale)
        scale = 1.0f0 / sqrt(Float32(eval_dim(realized_dims(q.shape)[end])))   # src/HighLevelOps.jl:378-381
    end
    inputs = [(q.id, 0, q.shape), (k.id, 0, k.shape), (v.id, 0, v.shape)]
    return add_op!(q.graph_ref, RopeFlashAttentionOp(Float32(scale), causal, Int32(prev_seq), Float32(base)), inputs, q.shape)
end

function execute_op!(out::HipArray{TO,4}, op::RopeFlashAttentionOp, q::HipArray{T,4}, k::HipArray{T,4}, v::HipArray{T,4}) where {TO,T}
    return execute_op!(out, FlashAttentionOp(op.scale, op.causal), q, k, v; q_rope_base=op.base, q_prev_seq=op.prev_seq)
end
execute_op(op::RopeFlashAttentionOp, q::HipArray, k::HipArray, v::HipArray) = execute_op!(similar(q), op, q, k, v)

"Returns (out, k_cache): `out` has q's shape (B,Hq,1,D); `k_cache` is the append node (the updated cache)."
function cached_self_attention_core(q::GraphTensor, k_new::GraphTensor, v_new::GraphTensor, k_cache::GraphTensor,
                                    v_cache::GraphTensor, pos::GraphTensor, kv_len::GraphTensor;
                                    rope_base=nothing, scale=nothing, head_map::Int32=HEADMAP_INTERLEAVED)
    kc = kv_cache_append(k_cache, v_cache, k_new, v_new, pos; rope_k=(rope_base !== nothing),
                         base=something(rope_base, 10000.0f0), q=(rope_base !== nothing ? q : nothing))
    # q and v_cache were updated in place by the append node, which precedes this one in graph order
    out = decode_attention(q, kc, v_cache, kv_len; scale=scale, head_map=head_map)
    return out, kc
end

# ------------------------------------------------------------------------------------------
# Host fallback: the ops around attention in a model graph (projections, reshapes, permutes, elementwise:
# src/Execution.jl:216-250) have no kernel in libluminal_hip.so. When one of them meets a HipArray — which is what
# the interpreter hands it on a HIPDevice (src/Execution.jl:630-656) — the arguments are downloaded, Luminal's own
# CPU method runs (the call below dispatches to it: the arguments are Arrays by then), and the result is uploaded.
# Slow and correct: a model runs end to end with attention on the GPU. Luminal's methods take untyped arguments, so
# the fallback methods are generated per op type and per pattern of HipArray positions (one untyped method per op
# type would be ambiguous with Luminal's own).
# ------------------------------------------------------------------------------------------
host_value(x::HipArray{BF16Bits}) = Float32.(from_device(x))
host_value(x::HipArray) = from_device(x)
host_value(x) = x
function host_fallback(op::Op, args...)
    cache_capturing() && error("$(typeof(op)) runs through the host and cannot be recorded into a HIP graph")
    res = execute_op(op, map(host_value, args)...)
    return res isa AbstractArray ? to_device(Array(res), HIPDevice()) : res
end
cache_capturing() = _stream[] != C_NULL

const FIXED_FALLBACK_ARITIES = 1:3
const DeviceOp = Union{FlashAttentionOp,RopeFlashAttentionOp,DecodeAttentionOp,DecodeStepOp,RotaryEmbeddingOp,KVAppendOp}
is_device_op_type(T) = T <: DeviceOp
for T in subtypes(Op)
    (is_device_op_type(T) || parentmodule(T) === @__MODULE__) && continue
    for n in FIXED_FALLBACK_ARITIES, pattern in 1:(2^n - 1)       # every non-empty set of HipArray positions
        sig = [(pattern >> (k - 1)) & 1 == 1 ? :($(Symbol(:a, k))::HipArray) : Symbol(:a, k) for k in 1:n]
        names = [Symbol(:a, k) for k in 1:n]
        @eval execute_op(op::$T, $(sig...)) = host_fallback(op, $(names...))
    end
    # ops with a variable number of inputs (FusedElementwiseOp, Function): a HipArray anywhere among four or more
    @eval execute_op(op::$T, a1, a2, a3, a4, rest...) =
        any(x -> x isa HipArray, (a1, a2, a3, a4, rest...)) ? host_fallback(op, a1, a2, a3, a4, rest...) :
        invoke(execute_op, Tuple{$T,Vararg{Any}}, op, a1, a2, a3, a4, rest...)
end

"""
    self_attention(sa::Luminal.NN.SelfAttention, x, prev_seq; rope_base=10000f0)

The reference layer (src/NN.jl:343-387) with its own nodes kept — the four projections, the split of `hidden` into
heads (a column-major Reshape: the head index is the fast one), the permutes — and everything between them (rotary
embedding of Q and K, repeat_kv, scaled causal softmax attention, src/NN.jl:356-382) replaced by
self_attention_core: the fused op reads the Hkv key/value heads directly and rotates the queries inside the kernel.
"""
"""
WhisperSelfAttention / WhisperCrossAttention (src/Whisper.jl:253-272, :295-316) around one flash attention node: the
layer's own projections (any struct with q_proj, k_proj, v_proj, o_proj, as both reference layers are), its
column-major split into `n_heads` heads and its permutes are kept; matmul, mask, softmax and matmul between them
become `flash_attention`. The reference scales q and k by D^-0.25 each (:256, :305-307): the kernel scales the product
by D^-0.5. Self attention: `whisper_attention(sa, x; n_heads, mask=true)`; cross attention:
`whisper_attention(ca, queries_t; n_heads, keys_from=enc, values_from=enc)`.
"""
function whisper_attention(layer, x::GraphTensor; n_heads::Int, mask::Bool=false, keys_from::GraphTensor=x,
                           values_from::GraphTensor=x)
    batch, seq, hidden = realized_dims(x.shape)
    head_dim = hidden ÷ n_heads
    function heads(proj, t)
        b, s, _ = realized_dims(t.shape)
        return Luminal.permute(Luminal.reshape(proj(t), [b, s, n_heads, head_dim]), [1, 3, 2, 4])
    end
    out = Luminal.flash_attention(heads(layer.q_proj, x), heads(layer.k_proj, keys_from), heads(layer.v_proj, values_from);
                                  causal=mask)
    out = Luminal.reshape(Luminal.permute(out, [1, 3, 2, 4]), [batch, seq, hidden])
    return layer.o_proj(out)
end

function self_attention(sa::Luminal.NN.SelfAttention, x::GraphTensor, prev_seq::Int; rope_base=10000.0f0)
    batch, seq, hidden = realized_dims(x.shape)
    heads(proj, n) = Luminal.permute(Luminal.reshape(proj(x), [batch, seq, n, sa.head_dim]), [1, 3, 2, 4])
    queries, keys, values = heads(sa.q_proj, sa.n_heads), heads(sa.k_proj, sa.n_kv_heads), heads(sa.v_proj, sa.n_kv_heads)
    out = self_attention_core(queries, keys, values; causal=true, prev_seq=prev_seq, rope_base=rope_base)
    out = Luminal.reshape(Luminal.permute(out, [1, 3, 2, 4]), [batch, seq, hidden])
    return sa.o_proj(out)
end

# ------------------------------------------------------------------------------------------
# compile_hip(graph): Luminal.compile (src/Compiler.jl:181-255) for graphs of the operators above, with the
# node buffers on the device. Luminal.compile itself cannot serve: it allocates host `zeros` for every
# non-CUDA device (:224-228) and its step closures capture those host arrays at compile time (:250-255), so
# nothing done to cg.results afterwards reaches them. The result is Luminal's own CompiledGraph, so calling
# it is the reference's code (src/Compiler.jl:81-100): length and copyto! on the node buffers, then
# execute_with_capture(device, run_graph, cache) — all of which have HipArray / HIPDevice methods above.
#   eltypes: node id => element type for input nodes (default Float32; inputs consumed as positions or
#            lengths default to Int32) and, optionally, for op nodes (default: the type of their first
#            input; Float32 on a half-precision attention node asks for the fp32 result).
# ------------------------------------------------------------------------------------------
is_input_node(op) = op isa Luminal.Function && op.name == "InputTensor"

function compile_hip(graph::Luminal.Graph; eltypes::AbstractDict=Dict{Int,DataType}())
    functional() || error("compile_hip: no gfx950 device answers libluminal_hip.so")
    n = length(graph.nodes)
    int_inputs = Set{Int}()                      # nodes read as Int32 positions / lengths
    for node in graph.nodes
        op = node.op
        op isa DecodeAttentionOp && push!(int_inputs, node.inputs[4][1])
        op isa KVAppendOp && push!(int_inputs, node.inputs[5][1])
        op isa RotaryEmbeddingOp && length(node.inputs) >= 2 && push!(int_inputs, node.inputs[2][1])
    end
    # 1. allocate results (src/Compiler.jl:218-235)
    eltype_of = Vector{DataType}(undef, n)
    results = Vector{Any}(undef, n)
    for (node_id, node) in enumerate(graph.nodes)
        op = node.op
        dims = Tuple(Int.(eval_dim.(realized_dims(graph.shapes[node_id]))))
        if is_input_node(op)
            eltype_of[node_id] = get(eltypes, node_id, node_id in int_inputs ? Int32 : Float32)
            results[node_id] = zeros_hip(eltype_of[node_id], dims)
        elseif op isa KVAppendOp                 # in place: the node's value is its k_cache input
            eltype_of[node_id] = eltype_of[node.inputs[1][1]]
            results[node_id] = results[node.inputs[1][1]]
        elseif op isa DeviceOp
            eltype_of[node_id] = get(eltypes, node_id, eltype_of[node.inputs[1][1]])
            results[node_id] = zeros_hip(eltype_of[node_id], dims)
        else                                     # served by the host fallback: a Float32 buffer the step uploads into
            eltype_of[node_id] = Float32
            results[node_id] = zeros_hip(Float32, dims)
        end
    end
    # 2. one in-place step per op; arguments are views of the persistent buffers, captured once (:250-255)
    steps = Base.Function[]
    n_host = 0
    for (node_id, node) in enumerate(graph.nodes)
        op = node.op
        is_input_node(op) && continue
        step_args = [realize_view(results[id], st) for (id, _, st) in node.inputs]
        for (k, (id, _, _)) in enumerate(node.inputs)
            same_memory(step_args[k], results[id]) ||
                error("compile_hip: input $k of node $node_id is a reshape that regroups axes; not supported on device buffers")
        end
        target_buf = results[node_id]
        if op isa DeviceOp
            push!(steps, (results, device) -> execute_op!(target_buf, op, step_args...))
        else                                     # download, Luminal's CPU method, upload into the node's buffer
            n_host += 1
            push!(steps, (results, device) -> copyto!(target_buf, Array(execute_op(op, map(host_value, step_args)...))))
        end
    end
    cache = Dict{Symbol,Any}()
    n_host > 0 && (cache[:hip_host_steps] = n_host)
    return Luminal.CompiledGraph(steps, results, cache)
end

"From the next call on, run the compiled steps as one recorded HIP graph (see execute_with_capture below)."
function enable_capture!(cg::Luminal.CompiledGraph)
    get(cg.cache, :hip_host_steps, 0) == 0 ||
        error("enable_capture!: $(cg.cache[:hip_host_steps]) steps of this graph run through the host; only graphs of device ops can be recorded")
    cg.cache[:hip_capture] = true
    return cg
end

# ------------------------------------------------------------------------------------------
# execute_with_capture(device, f, cache) (src/Device.jl:108-121; called by the compiled step closure,
# src/Compiler.jl:98). The reference stubs its CUDA method out because transient workspaces freed after
# the recording invalidated it. Here every buffer a step touches outlives the recording (the caches and
# results belong to the compiled graph, the split-KV workspace to this module and it only grows before
# the recording: the first call runs eagerly), and positions / lengths are device tensors, so one
# recording serves every decode position. Every call runs f's work exactly once. Off unless the cache holds
# :hip_capture => true (enable_capture!(cg) for a compiled graph).
# `f` must enqueue only through the executors of this module and must not upload or download.
# ------------------------------------------------------------------------------------------
function execute_with_capture(::HIPDevice, f, cache::Dict)
    # Opt-in (enable_capture!): on this runtime a recording of three kernel launches replays no faster than the
    # launches themselves, so the default is the plain loop, like the reference's stub.
    get(cache, :hip_capture, false) || return f()
    if !haskey(cache, :hip_exec)
        if !get(cache, :hip_warm, false)
            cache[:hip_warm] = true
            return f()                       # first use: allocations and set-up stay outside the recording
        end
        check(ccall((:lmh_sync, libluminal_hip), Cint, (Ptr{Cvoid},), C_NULL))
        sref = Ref{Ptr{Cvoid}}(C_NULL)
        check(ccall((:lmh_stream_create, libluminal_hip), Cint, (Ref{Ptr{Cvoid}},), sref))
        gref = Ref{Ptr{Cvoid}}(C_NULL)
        check(ccall((:lmh_graph_capture_begin, libluminal_hip), Cint, (Ptr{Cvoid},), sref[]))
        _stream[] = sref[]
        try
            f()
        catch
            _stream[] = C_NULL
            ccall((:lmh_graph_capture_end, libluminal_hip), Cint, (Ptr{Cvoid}, Ref{Ptr{Cvoid}}), sref[], gref)
            gref[] == C_NULL || ccall((:lmh_graph_destroy, libluminal_hip), Cint, (Ptr{Cvoid},), gref[])
            ccall((:lmh_stream_destroy, libluminal_hip), Cint, (Ptr{Cvoid},), sref[])
            rethrow()
        end
        _stream[] = C_NULL
        rc = ccall((:lmh_graph_capture_end, libluminal_hip), Cint, (Ptr{Cvoid}, Ref{Ptr{Cvoid}}), sref[], gref)
        if rc != 0
            ccall((:lmh_stream_destroy, libluminal_hip), Cint, (Ptr{Cvoid},), sref[])
            check(rc)
        end
        cache[:hip_exec] = gref[]
        cache[:hip_stream] = sref[]
        cache[:hip_workspace] = _workspace[]   # keeps the recorded scratch alive if the module's one is replaced by a larger one
    end
    # the recording's stream is blocking: work enqueued on the null stream before this call is waited for
    check(ccall((:lmh_graph_launch, libluminal_hip), Cint, (Ptr{Cvoid}, Ptr{Cvoid}), cache[:hip_exec], cache[:hip_stream]))
    return nothing
end

"Drop the recording execute_with_capture keeps in `cache` (the buffers it works on are untouched)."
function release_capture!(cache::Dict)
    if haskey(cache, :hip_exec)
        check(ccall((:lmh_sync, libluminal_hip), Cint, (Ptr{Cvoid},), cache[:hip_stream]))
        check(ccall((:lmh_graph_destroy, libluminal_hip), Cint, (Ptr{Cvoid},), pop!(cache, :hip_exec)))
        check(ccall((:lmh_stream_destroy, libluminal_hip), Cint, (Ptr{Cvoid},), pop!(cache, :hip_stream)))
    end
    delete!(cache, :hip_warm)
    delete!(cache, :hip_workspace)
    delete!(cache, :hip_capture)
    return nothing
end

export HIPDevice, HipArray, BF16Bits, release_capture!, enable_capture!, compile_hip, DecodeAttentionOp, decode_attention,
       RotaryEmbeddingOp, rotary_embedding, KVAppendOp, kv_cache_append, get_device, functional, rope!, kv_append!,
       self_attention_core!, cached_self_attention_core!, self_attention_core, cached_self_attention_core, flash_attention_plan,
       RopeFlashAttentionOp, rope_flash_attention, prompt_self_attention_core!, self_attention, host_fallback,
       HipKVCache, step_pos, begin_step!, advance!, decode_layer!, prompt_layer!, DecodeStepOp, decode_step, decode_step_supported,
       whisper_attention

end # module
