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
# and calls the C ABI of include/luminal_hip.h through `ccall`. There are no AMDGPU.jl kernels here.
#
# Layout: Luminal tensors are column-major (B,H,S,D) arrays (B fastest). The library takes
# row-major [B,H,S,D] (D contiguous), which is the memory order of a column-major (D,S,H,B) array,
# so upload is permutedims(x, (4,3,2,1)) and download is the inverse permutation.
module LuminalHIP

using Luminal
import Luminal: AbstractDevice, Op, FlashAttentionOp, GraphTensor, add_op!, realized_dims,
                to_device, from_device, execute_op, execute_op!, execute_with_capture

const libluminal_hip = get(ENV, "LUMINAL_HIP_LIB", joinpath(@__DIR__, "..", "lib", "libluminal_hip.so"))

# element type codes of include/luminal_hip.h
const LMH_F32, LMH_F16, LMH_BF16 = Int32(0), Int32(1), Int32(2)
const HEADMAP_INTERLEAVED, HEADMAP_BLOCKED = Int32(0), Int32(1)
# bf16 tensors are carried as UInt16 bit patterns (Julia has no native BFloat16 array type)
struct BF16Bits; bits::UInt16; end
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
Base.size(a::HipArray) = a.dims
Base.size(a::HipArray, i::Integer) = a.dims[i]
Base.length(a::HipArray) = prod(a.dims)
Base.eltype(::HipArray{T}) where {T} = T
Base.similar(a::HipArray{T,N}) where {T,N} = HipArray{T,N}(a.dims)

"Host array -> device, reversing the dimension order so that D becomes the contiguous axis."
function to_device(data::AbstractArray{T,N}, ::HIPDevice) where {T,N}
    host = Array(permutedims(data, ntuple(i -> N + 1 - i, N)))
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
    return permutedims(host, ntuple(i -> N + 1 - i, N))
end

# ------------------------------------------------------------------------------------------
# parameter blocks (field order and types mirror include/luminal_hip.h)
# ------------------------------------------------------------------------------------------
struct AttnParams
    out::Ptr{Cvoid}; q::Ptr{Cvoid}; k::Ptr{Cvoid}; v::Ptr{Cvoid}; kv_len::Ptr{Int32}
    B::Int32; Hq::Int32; Hkv::Int32; Sq::Int32; Sk::Int32; D::Int32
    q_stride::NTuple{3,Int64}; k_stride::NTuple{3,Int64}; v_stride::NTuple{3,Int64}; o_stride::NTuple{3,Int64}
    dtype::Int32; scale::Float32; causal::Int32; head_map::Int32; out_f32::Int32
    stream::Ptr{Cvoid}
end

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
                     head_map::Int32=HEADMAP_INTERLEAVED) where {TO,T}
    B, Hq, Sq, D = size(q)
    _, Hkv, Sk, _ = size(k)
    size(out) == size(q) || error("FlashAttentionOp: output shape $(size(out)) differs from q shape $(size(q))")
    p = Ref(AttnParams(out.ptr, q.ptr, k.ptr, v.ptr, C_NULL, B, Hq, Hkv, Sq, Sk, D, Z3, Z3, Z3, Z3,
                       dtype_code(T), op.scale, Int32(op.causal), head_map, Int32(TO === Float32 && T !== Float32), current_stream()))
    check(ccall((:lmh_flash_attn_fwd, libluminal_hip), Cint, (Ref{AttnParams},), p))
    return out
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

execute_op(op::DecodeAttentionOp, q::HipArray, kc::HipArray, vc::HipArray, kv_len::HipArray) =
    execute_op!(similar(q), op, q, kc, vc, kv_len)

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
# What the attention layers do between their projections, as fused calls on device arrays.
# SelfAttention (src/NN.jl:352-382) = rotary embedding of Q and K, repeat_kv, scaled causal softmax
# attention; the fused op reads the Hkv key/value heads directly in the head order repeat_kv produces
# (src/NN.jl:305-317). Whisper's layers (src/Whisper.jl:263-272, :310-312) are the same call without
# rotary embedding, cross attention with causal=false.
# ------------------------------------------------------------------------------------------
function self_attention_core!(out::HipArray, q::HipArray{T,4}, k::HipArray{T,4}, v::HipArray{T,4}; causal::Bool=true,
                              prev_seq::Integer=0, rope_base=nothing, scale=nothing,
                              head_map::Int32=HEADMAP_INTERLEAVED) where {T}
    if rope_base !== nothing
        rope!(q; prev_seq=prev_seq, base=rope_base)
        rope!(k; prev_seq=prev_seq, base=rope_base)
    end
    s = isnothing(scale) ? 1.0f0 / sqrt(Float32(size(q, 4))) : Float32(scale)
    return execute_op!(out, FlashAttentionOp(s, causal), q, k, v; head_map=head_map)
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
                                     head_map::Int32=HEADMAP_INTERLEAVED) where {TO,T}
    size(q, 3) == 1 || error("cached attention takes one query token per sequence")
    # one launch: the new rows go into the caches (K rotated on the way in) and q is rotated in place
    kv_append!(kc, vc, k_new, v_new, pos; rope_k=(rope_base !== nothing), base=something(rope_base, 10000.0f0),
               q=(rope_base !== nothing ? q : nothing))
    s = isnothing(scale) ? 1.0f0 / sqrt(Float32(size(q, 4))) : Float32(scale)
    q3 = HipArray{T,3}(q.ptr, (size(q, 1), size(q, 2), size(q, 4)), q)   # same memory, (B,Hq,D); keeps q alive
    return execute_op!(out, DecodeAttentionOp(s, head_map), q3, kc, vc, kv_len)
end

# ------------------------------------------------------------------------------------------
# execute_with_capture(device, f, cache) (src/Device.jl:108-121; called by the compiled step closure,
# src/Compiler.jl:98). The reference stubs its CUDA method out because transient workspaces freed after
# the recording invalidated it. Here every buffer a step touches outlives the recording (the caches and
# results belong to the compiled graph, the split-KV workspace to this module and it only grows before
# the recording: the first call runs eagerly), and positions / lengths are device tensors, so one
# recording serves every decode position. Every call runs f's work exactly once.
# `f` must enqueue only through the executors of this module and must not upload or download.
# ------------------------------------------------------------------------------------------
function execute_with_capture(::HIPDevice, f, cache::Dict)
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
    return nothing
end

export HIPDevice, HipArray, release_capture!, DecodeAttentionOp, decode_attention, get_device, functional, rope!, kv_append!,
       self_attention_core!, cached_self_attention_core!

end # module
