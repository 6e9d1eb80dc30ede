"""Host-side mirror of the slice of Luminal.jl's API that the attention hot path goes through.

The reference's host is Julia; its toolchain is not available where this backend is built and
tested, so the same interface is mirrored here in Python over the same C ABI the Julia glue
(julia/LuminalHIP.jl) calls. Names, argument meaning and error behaviour follow the reference:

  Graph, GraphTensor, tensor, add_op             reference src/Graph.jl:4-82
  FlashAttentionOp(scale, causal)                reference src/Ops.jl:104-107
  flash_attention(q, k, v; scale, causal)        reference src/HighLevelOps.jl:377-388
  execute_op / execute_op_inplace                reference src/Execution.jl:252-255, :565-578
  execute(graph, ids, inputs, device)            reference src/Execution.jl:620-670
  compile(graph) -> CompiledGraph(inputs, dev)   reference src/Compiler.jl:75-100, :181-255
  HIPDevice, get_device, to_device, from_device  reference src/Device.jl:9-16, :31-74, :82-105

Additions the reference has only as un-fused subgraphs:
  DecodeAttentionOp / decode_attention           reference src/Whisper.jl:584-620, :628-645
  GQA (Hkv < Hq) inside the fused ops            reference src/NN.jl:305-317, :362-366

Around the attention path, a model graph also holds the nodes of the layer that calls it (projections, reshapes,
permutes: reference src/NN.jl:343-361, :383-386). Those have no kernel here; they run through a host fallback
(HostOp: download the inputs, the reference's CPU semantics in numpy, upload the result), so that a whole
attention layer executes on a HIPDevice with attention itself on the GPU:
  MatMul, Permute, Reshape, Add, Expand          reference src/Execution.jl:216-250, src/HighLevelOps.jl:173-266
  Linear, SelfAttention                          reference src/NN.jl:11-38, :319-387

Arrays here are row-major [B, H, S, D] (numpy order), which is the layout the C ABI takes. There
is no CPU execution path for the attention ops: running one on host arrays raises.
"""
import ctypes
import math

import numpy as np

from . import binding
from .binding import HEADMAP_BLOCKED, HEADMAP_INTERLEAVED, LuminalHipError  # noqa: F401


# ---------------------------------------------------------------------------------------------
# element types
# ---------------------------------------------------------------------------------------------
def f32_to_bf16_bits(x):
    """fp32 array -> uint16 bf16 bit patterns, round-to-nearest-even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(bits):
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def encode(x, dtype):
    """fp32 numpy array -> the byte representation of `dtype` ('f32' | 'f16' | 'bf16')."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "f32":
        return x
    if dtype == "f16":
        return x.astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(x)
    raise ValueError("unknown dtype %r" % (dtype,))


def decode(raw, dtype):
    if dtype == "f32":
        return np.asarray(raw, dtype=np.float32)
    if dtype == "f16":
        return np.asarray(raw).view(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(np.asarray(raw).view(np.uint16))
    raise ValueError("unknown dtype %r" % (dtype,))


_NP_STORAGE = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16, "i32": np.int32}


# ---------------------------------------------------------------------------------------------
# devices and arrays
# ---------------------------------------------------------------------------------------------
class AbstractDevice:
    pass


class CPUDevice(AbstractDevice):
    def __repr__(self):
        return "CPUDevice()"


class HIPDevice(AbstractDevice):
    """An MI355X reached through libluminal_hip.so (not through AMDGPU.jl-style array packages)."""

    def __init__(self, index=0):
        self.index = index

    def __repr__(self):
        return "HIPDevice(%d)" % self.index


_initialised = set()


def get_device():
    """Best available device; same try-then-fall-through shape as the reference's get_device()
    (health check = lmh_init's tiny allocation). Falls through to CPUDevice, on which the attention
    ops refuse to run."""
    try:
        if binding.device_count() > 0:
            binding.init(0)
            _initialised.add(0)
            return HIPDevice(0)
    except (LuminalHipError, RuntimeError, OSError):
        pass
    return CPUDevice()


def _ensure_init(device):
    if device.index not in _initialised:
        binding.init(device.index)
        _initialised.add(device.index)


class HipArray:
    """Device buffer + shape + element type; frees its memory when collected (the Julia glue's
    HipArray does it in a finalizer)."""

    def __init__(self, shape, dtype="f32", device=None):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.device = device or HIPDevice(0)
        _ensure_init(self.device)
        itemsize = 4 if dtype == "i32" else binding.DTYPE_BYTES[dtype]
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * itemsize
        self.ptr = binding.malloc(max(self.nbytes, 1))

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def copy_from_host(self, arr):
        """arr: fp32 values (converted to this array's dtype) or already-encoded storage."""
        if self.dtype == "i32":
            raw = np.ascontiguousarray(arr, dtype=np.int32)
        elif np.asarray(arr).dtype == _NP_STORAGE[self.dtype] and self.dtype != "f32":
            raw = np.ascontiguousarray(arr)
        else:
            raw = encode(arr, self.dtype)
        if raw.size != self.size:
            raise ValueError("Input length mismatch: expected %d, got %d" % (self.size, raw.size))
        binding.memcpy_h2d(self.ptr, raw.ctypes.data, self.nbytes)
        return self

    def to_host_raw(self):
        raw = np.empty(self.shape, dtype=_NP_STORAGE[self.dtype])
        binding.memcpy_d2h(raw.ctypes.data, self.ptr, self.nbytes)
        return raw

    def to_host(self):
        raw = self.to_host_raw()
        return raw if self.dtype == "i32" else decode(raw, self.dtype).reshape(self.shape)

    def fill_bytes(self, value):
        binding.memset(self.ptr, value, self.nbytes)
        return self

    def view(self, shape):
        """Same memory under another shape of equal size (Base.reshape); the view keeps this array alive and
        frees nothing."""
        shape = tuple(int(x) for x in shape)
        if int(np.prod(shape, dtype=np.int64)) != self.size:
            raise ValueError("reshape: %s has %d elements, %s needs %d" % (self.shape, self.size, shape,
                                                                          int(np.prod(shape, dtype=np.int64))))
        v = HipArray.__new__(HipArray)
        v.shape, v.dtype, v.device, v.nbytes, v.ptr = shape, self.dtype, self.device, self.nbytes, self.ptr
        v._base = self
        return v

    def free(self):
        if getattr(self, "_base", None) is not None:
            self.ptr = 0
            return
        if getattr(self, "ptr", 0):
            binding.free(self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def to_device(data, device, dtype="f32"):
    """Move data to `device`; dicts are mapped value-wise (reference src/Device.jl:82-96)."""
    if isinstance(data, dict):
        return {k: to_device(v, device, dtype) for k, v in data.items()}
    if isinstance(device, HIPDevice):
        if isinstance(data, HipArray):
            return data
        if isinstance(data, np.ndarray):
            if data.dtype == np.int32:
                return HipArray(data.shape, "i32", device).copy_from_host(data)
            return HipArray(data.shape, dtype, device).copy_from_host(data)
    return data


def from_device(data):
    """Move data back to the host (reference src/Device.jl:103-105)."""
    if isinstance(data, HipArray):
        return data.to_host()
    return data


# ---------------------------------------------------------------------------------------------
# graph IR (only what the attention path touches)
# ---------------------------------------------------------------------------------------------
class Op:
    pass


class InputTensor(Op):
    name = "InputTensor"


class FlashAttentionOp(Op):
    """Fused flash attention node (reference src/Ops.jl:104-107), plus the GQA head map. Inputs (q, k, v), then
    optionally kv_len (int32[B], `has_kv_len`) and q_pos0 (int32[B], `has_q_pos0`). With `q_rope_base` the kernel
    rotates the query rows as it loads them (apply_rotary_embeddings on the queries, reference src/NN.jl:357, without
    a launch of its own): row i of sequence b at position (q_pos0 ? q_pos0[b] : q_prev_seq) + i."""

    def __init__(self, scale, causal, head_map=HEADMAP_INTERLEAVED, out_dtype=None, has_kv_len=False,
                 q_rope_base=None, q_prev_seq=0, q_rope_interleaved=False, has_q_pos0=False):
        self.scale = float(np.float32(scale))
        self.causal = bool(causal)
        self.head_map = head_map
        self.out_dtype = out_dtype  # None = q's element type; "f32" = full-precision result
        self.has_kv_len = bool(has_kv_len)
        self.q_rope_base = None if q_rope_base is None else float(q_rope_base)
        self.q_prev_seq = int(q_prev_seq)
        self.q_rope_interleaved = bool(q_rope_interleaved)
        self.has_q_pos0 = bool(has_q_pos0)
        if self.has_q_pos0 and self.q_rope_base is None:
            raise ValueError("q_pos0 is the position input of the rotary embedding: give q_rope_base as well")


class DecodeAttentionOp(Op):
    """Single-token attention over a KV cache; inputs (q, k_cache, v_cache, kv_len)."""

    def __init__(self, scale, head_map=HEADMAP_INTERLEAVED, num_splits=0, out_dtype=None):
        self.scale = float(np.float32(scale))
        self.head_map = head_map
        self.num_splits = num_splits
        self.out_dtype = out_dtype


class DecodeStepOp(Op):
    """One decode step of a cached attention layer as ONE node and two launches (lmh_decode_step): inputs
    (q (B,Hq,D), k_cache, v_cache, k_new (B,Hkv,1,D), v_new, pos int32[B]); output 0 is the attention result over rows
    0 .. pos[b] inclusive, outputs 1 and 2 are the caches themselves with row pos[b] written (K rotated when rope_base
    is set; q is rotated inside the kernel and left as it was). What decode_step! and whisper_self_attn_cached do for
    one layer (reference src/Whisper.jl:761-801, :584-620) with the rotary embedding of src/NN.jl:356-358."""

    def __init__(self, scale, head_map=HEADMAP_INTERLEAVED, num_splits=0, out_dtype=None, rope_base=None, interleaved=False):
        self.scale = float(np.float32(scale))
        self.head_map = head_map
        self.num_splits = num_splits
        self.out_dtype = out_dtype
        self.rope_base = None if rope_base is None else float(rope_base)
        self.interleaved = bool(interleaved)


def decode_step_supported(dtype, head_dim, rope=True, interleaved=False):
    """Whether lmh_decode_step takes this element type and head dim (otherwise: append + attend, three launches)."""
    if dtype not in ("f16", "bf16") or head_dim not in (64, 96, 128, 256):
        return False
    return (not rope) or interleaved or (head_dim // 32) % 2 == 0


class RotaryEmbeddingOp(Op):
    """apply_rotary_embeddings(input, prev_seq; base) (reference src/NN.jl:253-303) as one node; inputs (x,) or
    (x, pos0) with pos0 an int32[B] tensor of per-sequence start positions."""

    def __init__(self, prev_seq=0, base=10000.0, interleaved=False):
        self.prev_seq = int(prev_seq)
        self.base = float(base)
        self.interleaved = bool(interleaved)


class KVAppendOp(Op):
    """In-place cache update (the reference rebuilds the cache with _kv_scatter, src/Whisper.jl:552-570); inputs
    (k_cache, v_cache, k_new, v_new, pos); outputs 0 and 1 are the two caches themselves (same buffers).
    With rope_q a sixth input, this step's queries (B,Hq,T,D), is rotated in place by the same launch and is
    output 2 (the rotary embedding of the queries, reference src/NN.jl:356, without a launch of its own)."""

    def __init__(self, rope_k=False, base=10000.0, interleaved=False, rope_q=False):
        self.rope_k = bool(rope_k)
        self.base = float(base)
        self.interleaved = bool(interleaved)
        self.rope_q = bool(rope_q)


class HostOp(Op):
    """A node of the reference's graph that has no kernel in libluminal_hip.so. On a HIPDevice it runs through the host:
    inputs are downloaded, `compute` applies the reference's CPU semantics in fp32 numpy (reference
    src/Execution.jl:216-250), the result is uploaded in `out_dtype`. The logical meaning is the reference's; where
    that depends on Julia's column-major element order (Reshape) the numpy form says so."""
    out_dtype = "f32"

    def compute(self, *arrays):
        raise NotImplementedError


class MatMulOp(HostOp):
    """MatMul (reference src/Execution.jl:12-90 batch_matmul): (..., M, K) x (K, N) or x (..., K, N)."""

    def compute(self, a, b):
        if a.shape[-1] != b.shape[-2]:
            raise ValueError("Matmul dimension mismatch: A is %s, B is %s" % (a.shape, b.shape))
        return np.matmul(a, b)


class PermuteOp(HostOp):
    """Permute(dims) = permutedims (reference src/Execution.jl:229); dims are 0-based here."""

    def __init__(self, dims):
        self.dims = tuple(int(d) for d in dims)

    def compute(self, a):
        return np.transpose(a, self.dims)


class ReshapeOp(HostOp):
    """Reshape(shape) = Base.reshape on a column-major array (reference src/Execution.jl:228): the elements keep
    their column-major order, which in numpy is order='F'. Splitting hidden into (heads, head_dim) this way makes the
    head index the fast one: hidden index = head + n_heads * d (reference src/NN.jl:347)."""

    def __init__(self, shape):
        self.shape = tuple(int(d) for d in shape)

    def compute(self, a):
        return np.reshape(a, self.shape, order="F")


class AddOp(HostOp):
    """Add with the lower-rank operand given leading singleton axes (reference src/Execution.jl:207-216)."""

    def compute(self, a, b):
        return a + b


class ExpandOp(HostOp):
    """Expand(dim, size): a new axis at `dim` (0-based), repeated `size` times (reference src/Execution.jl:238-248)."""

    def __init__(self, dim, size):
        self.dim, self.size = int(dim), int(size)

    def compute(self, a):
        return np.repeat(np.expand_dims(a, self.dim), self.size, axis=self.dim)


class Node:
    def __init__(self, op, inputs):
        self.op = op
        self.inputs = inputs  # list of (node_id, output_index, shape)


class GraphTensor:
    def __init__(self, id, shape, graph_ref, index=0):
        self.id = id
        self.index = index  # which output of node `id` (reference src/Graph.jl input triples carry the same index)
        self.shape = tuple(shape)
        self.graph_ref = graph_ref


class Graph:
    def __init__(self):
        self.nodes = []
        self.shapes = []
        self.dtypes = []
        self.tensors = {}


def add_op(graph, op, inputs, output_shape, dtype="f32"):
    graph.nodes.append(Node(op, inputs))
    graph.shapes.append(tuple(output_shape))
    graph.dtypes.append(dtype)
    return GraphTensor(len(graph.nodes) - 1, output_shape, graph)


def tensor(graph, shape, dtype="f32"):
    """Define a new input tensor on the graph (reference src/Graph.jl:56-61)."""
    if isinstance(shape, np.ndarray):
        shape = shape.shape
    return add_op(graph, InputTensor(), [], tuple(shape), dtype)


def _host_node(op, inputs, shape, dtype):
    op.out_dtype = dtype
    g = inputs[0].graph_ref
    return add_op(g, op, [(t.id, t.index, t.shape) for t in inputs], shape, dtype)


def matmul(a, b, dtype="f32"):
    """(..., M, K) * (..., K, N) -> (..., M, N) (reference src/HighLevelOps.jl:252-266)."""
    if len(a.shape) < 2 or len(b.shape) < 2:
        raise ValueError("Matmul inputs must be at least 2D")
    return _host_node(MatMulOp(), [a, b], tuple(a.shape[:-1]) + (b.shape[-1],), dtype)


def permute(a, dims, dtype=None):
    """reference src/HighLevelOps.jl:183-192; dims 0-based."""
    return _host_node(PermuteOp(dims), [a], tuple(a.shape[d] for d in dims), dtype or a.graph_ref.dtypes[a.id])


def reshape(a, new_shape, dtype=None):
    """reference src/HighLevelOps.jl:173-181: column-major element order, see ReshapeOp."""
    if int(np.prod(new_shape, dtype=np.int64)) != int(np.prod(a.shape, dtype=np.int64)):
        raise ValueError("reshape: %s does not hold the elements of %s" % (tuple(new_shape), a.shape))
    return _host_node(ReshapeOp(new_shape), [a], tuple(new_shape), dtype or a.graph_ref.dtypes[a.id])


def add(a, b):
    shape = np.broadcast_shapes(a.shape, b.shape)
    return _host_node(AddOp(), [a, b], tuple(shape), "f32")


def expand(a, dim, size):
    """reference src/HighLevelOps.jl:194-200; dim 0-based."""
    shape = list(a.shape)
    shape.insert(dim, size)
    return _host_node(ExpandOp(dim, size), [a], tuple(shape), a.graph_ref.dtypes[a.id])


class Linear:
    """y = x W^T + b with W (out_features, in_features) (reference src/NN.jl:11-38)."""

    def __init__(self, in_features, out_features, graph, bias=True):
        self.weight = tensor(graph, (out_features, in_features))
        self.bias = tensor(graph, (out_features,)) if bias else None

    def __call__(self, x):
        out = matmul(x, permute(self.weight, (1, 0)))
        if self.bias is not None:
            b = self.bias
            for size in reversed(out.shape[:-1]):  # (the reference expands over the batch axis only; same values)
                b = expand(b, 0, size)
            out = add(out, b)
        return out


class SelfAttention:
    """SelfAttention (reference src/NN.jl:319-387) with the layer's own nodes kept — projections, the split of hidden
    into heads (a column-major reshape, so the head index is the fast one), the permutes — and everything between them
    (rotary embedding of Q and K, repeat_kv, scaled causal softmax attention, src/NN.jl:356-382) replaced by
    self_attention_core: GQA without copies of K/V, the queries rotated inside the attention kernel. `attn_dtype` is
    the element type attention runs in (the reference is fp32 only); the projections stay fp32 on the host."""

    def __init__(self, hidden, n_heads, n_kv_heads, graph, attn_dtype="f32"):
        if hidden % n_heads or n_heads % n_kv_heads:
            raise ValueError("hidden must be a multiple of n_heads, n_heads of n_kv_heads")
        self.n_heads, self.n_kv_heads, self.head_dim = n_heads, n_kv_heads, hidden // n_heads
        self.attn_dtype = attn_dtype
        self.q_proj = Linear(hidden, hidden, graph, bias=False)
        self.k_proj = Linear(hidden, n_kv_heads * self.head_dim, graph, bias=False)
        self.v_proj = Linear(hidden, n_kv_heads * self.head_dim, graph, bias=False)
        self.o_proj = Linear(hidden, hidden, graph, bias=False)

    def __call__(self, x, prev_seq=0, rope_base=10000.0):
        batch, seq, hidden = x.shape
        dt = self.attn_dtype

        def heads(proj, n):  # (B, S, n*D) -> (B, n, S, D), uploaded in the element type attention reads
            return permute(reshape(proj(x), (batch, seq, n, self.head_dim)), (0, 2, 1, 3), dtype=dt)

        queries, keys, values = heads(self.q_proj, self.n_heads), heads(self.k_proj, self.n_kv_heads), heads(self.v_proj, self.n_kv_heads)
        out = self_attention_core(queries, keys, values, causal=True, prev_seq=prev_seq, rope_base=rope_base,
                                  out_dtype="f32")
        out = reshape(permute(out, (0, 2, 1, 3)), (batch, seq, hidden))
        return self.o_proj(out)


class WhisperAttention:
    """WhisperSelfAttention and WhisperCrossAttention (reference src/Whisper.jl:238-272, :278-316) with the layer's own
    nodes kept — projections (q, v and the output with a bias, k without: :247-251, :288-292), the column-major split of
    hidden into heads, the permutes — and the matmul / mask / softmax / matmul between them replaced by one flash
    attention node. The reference scales q and k by D^-0.25 each (:256, :305-307); here the product is scaled by
    D^-0.5 inside the kernel. Self attention: layer(x, mask=True); cross attention: layer(x, mask=False, keys_from=enc,
    values_from=enc) (queries from the decoder, keys and values from the encoder output)."""

    def __init__(self, hidden, n_heads, graph, attn_dtype="f32"):
        if hidden % n_heads:
            raise ValueError("hidden must be a multiple of n_heads")
        self.n_heads, self.head_dim, self.attn_dtype = n_heads, hidden // n_heads, attn_dtype
        self.q_proj = Linear(hidden, hidden, graph, bias=True)
        self.k_proj = Linear(hidden, hidden, graph, bias=False)
        self.v_proj = Linear(hidden, hidden, graph, bias=True)
        self.o_proj = Linear(hidden, hidden, graph, bias=True)

    def __call__(self, x, mask=False, keys_from=None, values_from=None):
        batch, seq, hidden = x.shape
        k_in = x if keys_from is None else keys_from
        v_in = x if values_from is None else values_from

        def heads(proj, t):  # (B, S, H*D) -> (B, H, S, D), uploaded in the element type attention reads
            return permute(reshape(proj(t), (t.shape[0], t.shape[1], self.n_heads, self.head_dim)), (0, 2, 1, 3),
                           dtype=self.attn_dtype)

        out = flash_attention(heads(self.q_proj, x), heads(self.k_proj, k_in), heads(self.v_proj, v_in), causal=bool(mask),
                              out_dtype="f32")
        out = reshape(permute(out, (0, 2, 1, 3)), (batch, seq, hidden))
        return self.o_proj(out)


def flash_attention(q, k, v, scale=None, causal=False, head_map=HEADMAP_INTERLEAVED, out_dtype=None, kv_len=None,
                    q_rope_base=None, q_prev_seq=0, q_pos0=None, q_rope_interleaved=False):
    """q, k, v: (Batch, Head, Seq, HeadDim). Output has q's shape; scale defaults to 1/sqrt(D)
    computed in fp32 (reference src/HighLevelOps.jl:377-388). kv_len (int32[B] tensor) limits sequence b to its
    first kv_len[b] keys; q_rope_base asks for the rotary embedding of the queries inside the kernel, at positions
    q_prev_seq + i or q_pos0[b] + i (q_pos0 an int32[B] tensor)."""
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(q.shape[-1]))
    inputs = [(q.id, q.index, q.shape), (k.id, k.index, k.shape), (v.id, v.index, v.shape)]
    if kv_len is not None:
        inputs.append((kv_len.id, kv_len.index, kv_len.shape))
    if q_pos0 is not None:
        inputs.append((q_pos0.id, q_pos0.index, q_pos0.shape))
    op = FlashAttentionOp(np.float32(scale), causal, head_map, out_dtype, has_kv_len=kv_len is not None,
                          q_rope_base=q_rope_base, q_prev_seq=q_prev_seq, q_rope_interleaved=q_rope_interleaved,
                          has_q_pos0=q_pos0 is not None)
    return add_op(q.graph_ref, op, inputs, q.shape, out_dtype or q.graph_ref.dtypes[q.id])


def decode_attention(q, k_cache, v_cache, kv_len, scale=None, head_map=HEADMAP_INTERLEAVED, num_splits=0,
                     out_dtype=None):
    """q: (Batch, Head, HeadDim); caches: (Batch, KVHead, MaxSeq, HeadDim); kv_len: (Batch,) int32."""
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(q.shape[-1]))
    inputs = [(q.id, q.index, q.shape), (k_cache.id, k_cache.index, k_cache.shape),
              (v_cache.id, v_cache.index, v_cache.shape), (kv_len.id, kv_len.index, kv_len.shape)]
    return add_op(q.graph_ref, DecodeAttentionOp(np.float32(scale), head_map, num_splits, out_dtype), inputs, q.shape,
                  out_dtype or q.graph_ref.dtypes[q.id])


def decode_step(q, k_cache, v_cache, k_new, v_new, pos, scale=None, head_map=HEADMAP_INTERLEAVED, num_splits=0,
                out_dtype=None, rope_base=None, interleaved=False):
    """Graph form of lmh_decode_step: q (B,Hq,D); returns (out, k_cache, v_cache)."""
    g = q.graph_ref
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(q.shape[-1]))
    inputs = [(t.id, t.index, t.shape) for t in (q, k_cache, v_cache, k_new, v_new, pos)]
    out = add_op(g, DecodeStepOp(np.float32(scale), head_map, num_splits, out_dtype, rope_base, interleaved), inputs, q.shape,
                 out_dtype or g.dtypes[q.id])
    return out, GraphTensor(out.id, k_cache.shape, g, index=1), GraphTensor(out.id, v_cache.shape, g, index=2)


def rotary_embedding(x, prev_seq=0, base=10000.0, pos0=None, interleaved=False):
    """Graph form of apply_rotary_embeddings (reference src/NN.jl:253-303): x (B,H,S,D); row s of sequence b is
    rotated by position prev_seq + s, or pos0[b] + s when the int32[B] tensor pos0 is given."""
    g = x.graph_ref
    inputs = [(x.id, x.index, x.shape)]
    if pos0 is not None:
        inputs.append((pos0.id, pos0.index, pos0.shape))
    return add_op(g, RotaryEmbeddingOp(prev_seq, base, interleaved), inputs, x.shape, g.dtypes[x.id])


def kv_cache_append(k_cache, v_cache, k_new, v_new, pos, rope_k=False, base=10000.0, interleaved=False, q=None):
    """Graph form of the cache update: returns the (k, v) cache tensors after rows pos[b] .. pos[b]+T-1 of sequence
    b were overwritten by k_new / v_new (K optionally rotated by its position on the way in). With `q`, this
    step's queries (B,Hq,T,D), the same node rotates them in place at the same positions and a third tensor, the
    rotated queries (q's own buffer: the unrotated values are gone), is returned as well."""
    g = k_cache.graph_ref
    tensors = (k_cache, v_cache, k_new, v_new, pos) + (() if q is None else (q,))
    inputs = [(t.id, t.index, t.shape) for t in tensors]
    k_out = add_op(g, KVAppendOp(rope_k, base, interleaved, rope_q=q is not None), inputs, k_cache.shape,
                   g.dtypes[k_cache.id])
    v_out = GraphTensor(k_out.id, v_cache.shape, g, index=1)
    if q is None:
        return k_out, v_out
    return k_out, v_out, GraphTensor(k_out.id, q.shape, g, index=2)


def self_attention_core(q, k, v, causal=True, prev_seq=0, rope_base=None, scale=None, head_map=HEADMAP_INTERLEAVED,
                        out_dtype=None):
    """What SelfAttention does between its projections (reference src/NN.jl:352-382: rotary embedding of Q and K,
    repeat_kv, scaled causal softmax attention), emitted as fused nodes: two rotary nodes and one flash attention
    node that reads the Hkv key/value heads directly (`head_map` INTERLEAVED is the head order repeat_kv produces,
    src/NN.jl:305-317) instead of materialising G copies. rope_base=None skips the rotary embedding (Whisper's
    attention layers, reference src/Whisper.jl:263-272 and :310-312, with causal=False for cross attention)."""
    if rope_base is None:
        return flash_attention(q, k, v, scale=scale, causal=causal, head_map=head_map, out_dtype=out_dtype)
    k = rotary_embedding(k, prev_seq, rope_base)
    if q.shape[-1] not in FUSED_ROPE_HEAD_DIMS:  # the vector-ALU kernel would serve the fused form: keep the rotary node
        q = rotary_embedding(q, prev_seq, rope_base)
        return flash_attention(q, k, v, scale=scale, causal=causal, head_map=head_map, out_dtype=out_dtype)
    # the queries are rotated inside the attention kernel: no node (and no launch) of their own
    return flash_attention(q, k, v, scale=scale, causal=causal, head_map=head_map, out_dtype=out_dtype,
                           q_rope_base=rope_base, q_prev_seq=prev_seq)


# head dims for which the matrix-core attention kernels rotate the queries in registers
FUSED_ROPE_HEAD_DIMS = (64, 96, 128)


def prompt_self_attention_core(q, k_new, v_new, k_cache, v_cache, pos, kv_len, rope_base=None, scale=None,
                               head_map=HEADMAP_INTERLEAVED, out_dtype=None):
    """The prompt pass of a cached attention layer as two fused nodes (the reference runs SelfAttention on the prompt,
    src/NN.jl:352-382, and fills its caches by slice + concat, src/Whisper.jl:552-570): q (B,Hq,T,D) and k_new, v_new
    (B,Hkv,T,D) are the prompt's projections; the append node writes rows pos[b] .. pos[b]+T-1 of the caches with K
    rotated on the way in, the attention node reads the caches' first kv_len[b] rows and rotates the queries as it
    loads them. The causal mask aligns query row i with cache row i, so the prompt must start its cache: pos[b] = 0
    and kv_len[b] = T (later chunks of a prompt are out of scope). Returns (out (B,Hq,T,D), k_cache, v_cache)."""
    if rope_base is not None:
        k_cache, v_cache = kv_cache_append(k_cache, v_cache, k_new, v_new, pos, rope_k=True, base=rope_base)
    else:
        k_cache, v_cache = kv_cache_append(k_cache, v_cache, k_new, v_new, pos)
    fused = rope_base is not None and q.shape[-1] in FUSED_ROPE_HEAD_DIMS
    if rope_base is not None and not fused:
        q = rotary_embedding(q, 0, rope_base, pos0=pos)
    out = flash_attention(q, k_cache, v_cache, scale=scale, causal=True, head_map=head_map, out_dtype=out_dtype,
                          kv_len=kv_len, q_rope_base=rope_base if fused else None, q_pos0=pos if fused else None)
    return out, k_cache, v_cache


def cached_self_attention_core(q, k_new, v_new, k_cache, v_cache, pos, kv_len, rope_base=None, scale=None,
                               head_map=HEADMAP_INTERLEAVED, num_splits=0, out_dtype=None, fused=False):
    """One decode step of a cached attention layer (reference src/Whisper.jl:584-620) as two fused nodes:
    q (B,Hq,1,D), k_new / v_new (B,Hkv,1,D) are this step's projections, pos int32[B] the row each sequence
    writes, kv_len = pos + 1 the rows it then attends over. Positions are tensors, so one compiled graph serves
    every step (the reference compiles one graph per position, src/Decoding.jl:98-106). Returns (out (B,Hq,D),
    k_cache, v_cache)."""
    g = q.graph_ref
    if fused and len(q.shape) == 4 and q.shape[2] == 1 and decode_step_supported(g.dtypes[q.id], q.shape[-1], rope_base is not None):
        # one node, two launches: the split kernel rotates q as it loads it, the merge launch adds and stores the new row
        # (`kv_len` is not needed: the step attends rows 0 .. pos[b])
        q3 = GraphTensor(q.id, (q.shape[0], q.shape[1], q.shape[3]), g, q.index)
        return decode_step(q3, k_cache, v_cache, k_new, v_new, pos, scale=scale, head_map=head_map, num_splits=num_splits,
                           out_dtype=out_dtype, rope_base=rope_base)
    if rope_base is not None:  # one launch: rotate q in place, write the new rows with K rotated on the way in
        k_cache, v_cache, q = kv_cache_append(k_cache, v_cache, k_new, v_new, pos, rope_k=True, base=rope_base, q=q)
    else:
        k_cache, v_cache = kv_cache_append(k_cache, v_cache, k_new, v_new, pos)
    B, Hq, one, D = q.shape
    if one != 1:
        raise ValueError("cached attention takes one query token per sequence; got q %s" % (q.shape,))
    q3 = GraphTensor(q.id, (B, Hq, D), g, q.index)  # (B,Hq,1,D) and (B,Hq,D) are the same buffer
    out = decode_attention(q3, k_cache, v_cache, kv_len, scale=scale, head_map=head_map, num_splits=num_splits,
                           out_dtype=out_dtype)
    return out, k_cache, v_cache


# ---------------------------------------------------------------------------------------------
# execution
# ---------------------------------------------------------------------------------------------
def _require_hip(*arrays):
    for a in arrays:
        if not isinstance(a, HipArray):
            raise TypeError("attention ops run on HipArray inputs only; this backend has no CPU path "
                            "(got %s)" % type(a).__name__)


class _Workspaces:
    """Decode split-KV scratch, grown on demand and reused (caller-owned from the library's view)."""

    def __init__(self):
        self.buf = None

    def get(self, nbytes, device):
        if nbytes == 0:
            return 0, 0
        if self.buf is None or self.buf.nbytes < nbytes:
            if self.buf is not None:
                binding.sync()
                self.buf.free()
            self.buf = HipArray(((nbytes + 3) // 4,), "f32", device)
        return self.buf.ptr, self.buf.nbytes


_workspaces = _Workspaces()


def flash_attention_plan(q_shape, kv_shape, dtype, causal=False, scale=None, out_dtype=None):
    """Name of the kernel (instantiation and workgroup count) a flash-attention launch of these shapes would run,
    for contiguous 16-byte aligned tensors. Launches nothing and needs no GPU."""
    p = binding.AttnParams()
    p.out = p.q = p.k = p.v = 4096  # never dereferenced: the plan query stops in front of the launch
    p.B, p.Hq, p.Sq, p.D = q_shape
    p.Hkv, p.Sk = kv_shape[1], kv_shape[2]
    p.dtype = binding.DTYPE_CODES[dtype]
    p.scale = default_scale(q_shape[-1]) if scale is None else scale
    p.causal = int(causal)
    p.out_f32 = int((out_dtype or dtype) == "f32")
    return binding.flash_attn_plan(p)


def _host_fallback(op, inputs):
    """The reference's CPU semantics for a node without a kernel: download, compute in fp32 numpy, hand back the host
    result (the caller uploads it)."""
    host = [x.to_host() if isinstance(x, HipArray) else np.asarray(x, dtype=np.float32) for x in inputs]
    return np.ascontiguousarray(op.compute(*host), dtype=np.float32)


def _prepare_decode_step(op, out, inputs, workspaces=None):
    """Validates a DecodeStepOp call and fills its parameter blocks once; returns launch(stream). A compiled graph keeps
    the launcher (its buffers never move), so a step costs one ctypes call on the host."""
    if len(inputs) != 6:
        raise ValueError("DecodeStepOp takes (q, k_cache, v_cache, k_new, v_new, pos)")
    q, kc, vc, k_new, v_new, pos = inputs
    res = out[0] if isinstance(out, tuple) else out
    if isinstance(out, tuple) and not (out[1] is kc and out[2] is vc):
        raise ValueError("DecodeStepOp updates the caches in place: outputs 1 and 2 are its cache inputs")
    _require_hip(res, q, kc, vc, k_new, v_new, pos)
    if len(q.shape) != 3 or len(kc.shape) != 4 or kc.shape != vc.shape or res.shape != q.shape:
        raise ValueError("decode step expects q and out (B,H,D) and caches (B,Hkv,Lmax,D); got %s %s %s %s" %
                         (q.shape, res.shape, kc.shape, vc.shape))
    B, Hkv, Lmax, D = kc.shape
    if k_new.shape != v_new.shape or k_new.shape not in ((B, Hkv, 1, D), (B, Hkv, D)) or pos.shape != (B,) or pos.dtype != "i32":
        raise ValueError("decode step: new rows %s / %s for caches %s, pos %s" % (k_new.shape, v_new.shape, kc.shape, pos.shape))
    if not (q.dtype == kc.dtype == vc.dtype == k_new.dtype == v_new.dtype) or res.dtype not in (q.dtype, "f32"):
        raise ValueError("q, the caches and the new rows must share one element type; out has that type or f32")
    p = binding.DecodeParams()
    p.out, p.q, p.k_cache, p.v_cache, p.kv_len = res.ptr, q.ptr, kc.ptr, vc.ptr, pos.ptr
    p.B, p.Hq, p.D = q.shape
    p.Hkv, p.Lmax = Hkv, Lmax
    p.dtype = binding.DTYPE_CODES[q.dtype]
    p.scale, p.head_map = op.scale, op.head_map
    p.out_f32 = int(res.dtype == "f32")
    p.num_splits = op.num_splits or binding.decode_step_splits(p.B, p.Hkv, p.Lmax)
    need = binding.decode_workspace_bytes(p.B, p.Hq, p.Hkv, p.Lmax, p.D, p.num_splits)
    x = binding.DecodeStepExtra()
    x.k_new, x.v_new = k_new.ptr, v_new.ptr
    x.rope = int(op.rope_base is not None)
    x.pairing = binding.ROPE_INTERLEAVED if op.interleaved else binding.ROPE_HALF_SPLIT
    x.rope_base = op.rope_base if op.rope_base is not None else 10000.0
    pool, result = (workspaces or _workspaces), (res, kc, vc)

    def launch(stream=None):
        p.workspace, p.workspace_bytes = pool.get(need, q.device)
        p.stream = stream
        binding.decode_step(p, x)
        return result

    return launch


def execute_op_inplace(out, op, *inputs, stream=None, workspaces=None):
    """execute_op!(out, op, inputs...) (reference src/Execution.jl:565-578) for the attention ops. `workspaces`
    is where decode attention takes its split-KV scratch from (default: one buffer shared by all eager calls)."""
    if isinstance(op, HostOp):
        if stream is not None:
            raise RuntimeError("%s runs through the host and cannot be part of a recorded HIP graph" % type(op).__name__)
        _require_hip(out)
        res = _host_fallback(op, inputs)
        if res.shape != out.shape:
            raise ValueError("%s: result shape %s differs from the node's %s" % (type(op).__name__, res.shape, out.shape))
        binding.sync()  # the inputs were produced by kernels on the null stream; the download above waited for them
        return out.copy_from_host(res)
    if isinstance(op, FlashAttentionOp):
        q, k, v = inputs[:3]
        rest = list(inputs[3:])
        if not (op.has_kv_len or op.has_q_pos0) and len(rest) == 1:  # eager callers pass kv_len as a fourth array
            kv_len, q_pos0 = rest[0], None
        else:
            if len(rest) != int(op.has_kv_len) + int(op.has_q_pos0):
                raise ValueError("FlashAttentionOp takes (q, k, v%s%s); got %d inputs" %
                                 (", kv_len" if op.has_kv_len else "", ", q_pos0" if op.has_q_pos0 else "", len(inputs)))
            kv_len = rest.pop(0) if op.has_kv_len else None
            q_pos0 = rest.pop(0) if op.has_q_pos0 else None
        _require_hip(out, q, k, v)
        if len(q.shape) != 4 or len(k.shape) != 4 or k.shape != v.shape:
            raise ValueError("flash attention expects q (B,H,S,D) and k, v (B,Hkv,Sk,D); got %s %s %s" %
                             (q.shape, k.shape, v.shape))
        if out.shape != q.shape:
            raise ValueError("output shape %s differs from q shape %s" % (out.shape, q.shape))
        if not (q.dtype == k.dtype == v.dtype) or out.dtype not in (q.dtype, "f32"):
            raise ValueError("q, k, v must share one element type; out has that type or f32")
        if k.shape[0] != q.shape[0] or k.shape[3] != q.shape[3]:
            raise ValueError("k/v batch or head dim differ from q's")
        p = binding.AttnParams()
        p.out, p.q, p.k, p.v = out.ptr, q.ptr, k.ptr, v.ptr
        p.kv_len = kv_len.ptr if kv_len is not None else None
        p.B, p.Hq, p.Sq, p.D = q.shape
        p.Hkv, p.Sk = k.shape[1], k.shape[2]
        p.dtype = binding.DTYPE_CODES[q.dtype]
        p.scale, p.causal, p.head_map = op.scale, int(op.causal), op.head_map
        p.out_f32 = int(out.dtype == "f32")
        p.stream = stream
        if op.q_rope_base is not None:
            p.q_rope = 1
            p.q_rope_pairing = binding.ROPE_INTERLEAVED if op.q_rope_interleaved else binding.ROPE_HALF_SPLIT
            p.q_pos0 = q_pos0.ptr if q_pos0 is not None else None
            p.q_prev_seq = op.q_prev_seq
            p.q_rope_base = op.q_rope_base
        binding.flash_attn_fwd(p)
        return out
    if isinstance(op, DecodeAttentionOp):
        q, kc, vc = inputs[:3]
        kv_len = inputs[3] if len(inputs) > 3 else None
        _require_hip(out, q, kc, vc)
        if len(q.shape) != 3 or len(kc.shape) != 4 or kc.shape != vc.shape:
            raise ValueError("decode attention expects q (B,H,D) and caches (B,Hkv,Lmax,D); got %s %s %s" %
                             (q.shape, kc.shape, vc.shape))
        if out.shape != q.shape:
            raise ValueError("output shape %s differs from q shape %s" % (out.shape, q.shape))
        if not (q.dtype == kc.dtype == vc.dtype) or out.dtype not in (q.dtype, "f32"):
            raise ValueError("q and the caches must share one element type; out has that type or f32")
        p = binding.DecodeParams()
        p.out, p.q, p.k_cache, p.v_cache = out.ptr, q.ptr, kc.ptr, vc.ptr
        p.kv_len = kv_len.ptr if kv_len is not None else None
        p.B, p.Hq, p.D = q.shape
        p.Hkv, p.Lmax = kc.shape[1], kc.shape[2]
        p.dtype = binding.DTYPE_CODES[q.dtype]
        p.scale, p.head_map = op.scale, op.head_map
        p.out_f32 = int(out.dtype == "f32")
        p.num_splits = op.num_splits or binding.decode_auto_splits(p.B, p.Hkv, p.Lmax)
        need = binding.decode_workspace_bytes(p.B, p.Hq, p.Hkv, p.Lmax, p.D, p.num_splits)
        p.workspace, p.workspace_bytes = (workspaces or _workspaces).get(need, q.device)
        p.stream = stream
        binding.decode_attn(p)
        return out
    if isinstance(op, DecodeStepOp):
        return _prepare_decode_step(op, out, inputs, workspaces)(stream)
    if isinstance(op, RotaryEmbeddingOp):
        x = inputs[0]
        pos0 = inputs[1] if len(inputs) > 1 else None
        return apply_rotary_embeddings(x, op.prev_seq, op.base, pos0=pos0, out=out, interleaved=op.interleaved,
                                       stream=stream)
    if isinstance(op, KVAppendOp):
        if len(inputs) != (6 if op.rope_q else 5):
            raise ValueError("KVAppendOp takes (k_cache, v_cache, k_new, v_new, pos%s)" % (", q" if op.rope_q else ""))
        kc, vc, k_new, v_new, pos = inputs[:5]
        q = inputs[5] if op.rope_q else None
        if out is not None and not (isinstance(out, tuple) and out[0] is kc and out[1] is vc and
                                    (q is None or out[2] is q)):
            raise ValueError("KVAppendOp works in place: its outputs are its cache (and query) inputs")
        kv_append(kc, vc, k_new, v_new, pos, rope_k=op.rope_k, base=op.base, interleaved=op.interleaved, q=q,
                  stream=stream)
        return (kc, vc) if q is None else (kc, vc, q)
    raise TypeError("no HIP kernel for op %s" % type(op).__name__)


def execute_op(op, *inputs):
    """Allocating form: out = similar(q); execute_op!(out, ...) (reference src/Execution.jl:252-255)."""
    if isinstance(op, HostOp):
        dev = next((x.device for x in inputs if isinstance(x, HipArray)), None)
        if dev is None:
            raise TypeError("%s: no input is on a HIP device" % type(op).__name__)
        res = _host_fallback(op, inputs)
        return HipArray(res.shape, op.out_dtype, dev).copy_from_host(res)
    q = inputs[0]
    _require_hip(q)
    if isinstance(op, KVAppendOp):
        return execute_op_inplace(None, op, *inputs)
    if isinstance(op, DecodeStepOp):
        res = HipArray(q.shape, op.out_dtype or q.dtype, q.device)
        return execute_op_inplace((res, inputs[1], inputs[2]), op, *inputs)
    out = HipArray(q.shape, getattr(op, "out_dtype", None) or q.dtype, q.device)
    return execute_op_inplace(out, op, *inputs)


def _pick(results, ref):
    """Value of input triple (node_id, output_index, shape): multi-output nodes store a tuple."""
    r = results[ref[0]]
    r = r[ref[1]] if isinstance(r, tuple) else r
    if isinstance(r, HipArray) and tuple(ref[2]) != r.shape:
        r = r.view(ref[2])
    return r


def execute(graph, output_ids, initial_inputs, device=None, dtype=None):
    """Interpreter (reference src/Execution.jl:620-670): upload inputs, run nodes in order, download
    the requested outputs. `output_ids` may be one id or a list."""
    device = device or get_device()
    single = isinstance(output_ids, int)
    ids = [output_ids] if single else list(output_ids)
    results = {}
    for k, v in initial_inputs.items():
        results[k] = to_device(v, device, dtype or graph.dtypes[k])
    for (node_id, out_idx), data in graph.tensors.items():
        if node_id not in results and out_idx == 0:
            results[node_id] = to_device(data, device, graph.dtypes[node_id])
    for node_id, node in enumerate(graph.nodes):
        if node_id in results:
            continue
        if isinstance(node.op, InputTensor):
            raise KeyError("no value given for input tensor %d" % node_id)
        results[node_id] = execute_op(node.op, *[_pick(results, ref) for ref in node.inputs])
    final = {i: from_device(results[i][0] if isinstance(results[i], tuple) else results[i]) for i in ids}
    return final[ids[0]] if single else final


def execute_with_capture(device, f, cache):
    """execute_with_capture(device, f, cache) (reference src/Device.jl:108-121, called from the compiled step
    closure, src/Compiler.jl:98): run `f` on `device`; where the device supports it, record what `f` enqueues
    into a graph kept in `cache` and replay it on later calls. The reference stubs this out for CUDA (its
    recording was invalidated by transient workspaces that were freed); here `f(stream)` must enqueue only on
    the stream it is given and only on buffers that outlive the recording. Every call runs `f`'s work exactly
    once: the first call runs it eagerly (the library's first-use set-up stays outside the recording), the second
    records and replays, later ones replay. Measured on an MI355X a recording of a decode step's three kernels
    replays no faster than the three launches (57 vs 52 us at B=16, L=4096), so this is there for parity with the
    reference's interface and for hosts whose per-op dispatch is slow, not as a speed-up."""
    if not isinstance(device, HIPDevice):
        return f(None)
    if "hip_exec" not in cache:
        if not cache.get("hip_warm"):
            cache["hip_warm"] = True
            return f(None)
        binding.sync()
        stream = binding.stream_create()
        try:
            binding.graph_capture_begin(stream)
            try:
                f(stream)
            except Exception:
                try:  # leave the stream usable; a recording that still instantiated is dropped
                    binding.graph_destroy(binding.graph_capture_end(stream))
                except binding.LuminalHipError:
                    pass
                raise
            cache["hip_exec"] = binding.graph_capture_end(stream)
        except Exception:
            binding.stream_destroy(stream)
            raise
        cache["hip_stream"] = stream
    # work enqueued on the null stream before this call is waited for: the capture stream was created blocking
    binding.graph_launch(cache["hip_exec"], cache["hip_stream"])
    return None


def release_capture(cache):
    """Drop the recording execute_with_capture keeps in `cache` (its buffers are untouched)."""
    if "hip_exec" in cache:
        binding.sync(cache["hip_stream"])
        binding.graph_destroy(cache.pop("hip_exec"))
        binding.stream_destroy(cache.pop("hip_stream"))
    cache.pop("hip_warm", None)


class CompiledGraph:
    """Pre-allocated node buffers + a step list (reference src/Compiler.jl:75-100). Calling it copies the
    inputs into their buffers, runs the steps in place and returns the buffer list; nothing is
    allocated per call. After capture() the steps go through execute_with_capture: one HIP graph launch."""

    def __init__(self, steps, results, workspaces=None, device=None, host_steps=0):
        self.host_steps = host_steps  # nodes served by the host fallback
        self.steps = steps
        self.results = results
        self.workspaces = workspaces  # decode scratch owned by this graph: its address never changes
        self.device = device
        self.cache = {}
        self.use_capture = False

    def _run(self, stream):
        for step in self.steps:
            step(stream)

    def __call__(self, inputs, device=None):
        for k, v in inputs.items():
            if k >= len(self.results) or self.results[k] is None:
                raise KeyError("Input node %d not found in compiled graph results." % k)
            if isinstance(v, HipArray):
                if v.nbytes != self.results[k].nbytes:
                    raise ValueError("Input length mismatch for node %d" % k)
                binding.memcpy_d2d(self.results[k].ptr, v.ptr, v.nbytes)
            else:
                self.results[k].copy_from_host(v)
        if self.use_capture:
            execute_with_capture(self.device, self._run, self.cache)
        else:
            self._run(None)
            self.cache["hip_warm"] = True
        return self.results

    def capture(self):
        """From the next call on, run the step list as one recorded HIP graph. Buffer addresses are fixed and
        per-step values (positions, lengths) are device tensors, so one recording is valid for every call."""
        if self.host_steps:
            raise RuntimeError("this graph has %d nodes that run through the host (projections, reshapes): only graphs "
                               "of device ops can be recorded" % self.host_steps)
        self.use_capture = True
        return self

    def release(self):
        """Back to step-by-step execution; drops the recording and its stream (the buffers stay)."""
        self.use_capture = False
        release_capture(self.cache)


def compile(graph, device=None):
    """compile(graph) (reference src/Compiler.jl:181-255) for graphs of attention ops: one persistent
    device buffer per node, one in-place step per op. Unlike the reference, which allocates host
    arrays for every non-CUDA device (src/Compiler.jl:224-228), buffers live on the HIP device."""
    device = device or get_device()
    if not isinstance(device, HIPDevice):
        raise RuntimeError("compile: no HIP device available and this backend has no CPU path")
    results = []
    for node_id, node in enumerate(graph.nodes):
        if isinstance(node.op, KVAppendOp):  # in place: the node's outputs are its cache (and query) inputs
            refs = [node.inputs[0], node.inputs[1]] + ([node.inputs[5]] if node.op.rope_q else [])
            results.append(tuple(_pick(results, r) for r in refs))
            continue
        if isinstance(node.op, DecodeStepOp):  # output 0 is a buffer of its own, outputs 1 and 2 are the cache inputs
            results.append((HipArray(graph.shapes[node_id], graph.dtypes[node_id], device).fill_bytes(0),
                            _pick(results, node.inputs[1]), _pick(results, node.inputs[2])))
            continue
        results.append(HipArray(graph.shapes[node_id], graph.dtypes[node_id], device).fill_bytes(0))
    steps = []
    workspaces = _Workspaces()
    for node_id, node in enumerate(graph.nodes):
        if isinstance(node.op, InputTensor):
            continue
        args = [_pick(results, ref) for ref in node.inputs]
        if isinstance(node.op, DecodeStepOp):
            steps.append(_prepare_decode_step(node.op, results[node_id], args, workspaces))
            continue
        steps.append(lambda stream, out=results[node_id], op=node.op, args=args:
                     execute_op_inplace(out, op, *args, stream=stream, workspaces=workspaces))
    host_steps = sum(isinstance(node.op, HostOp) for node in graph.nodes)
    return CompiledGraph(steps, results, workspaces, device, host_steps)


# ---------------------------------------------------------------------------------------------
# the operators directly in front of decode attention
# ---------------------------------------------------------------------------------------------
def apply_rotary_embeddings(x, prev_seq=0, base=10000.0, pos0=None, out=None, interleaved=False, stream=None):
    """Rotary embedding of a (B,H,S,D) HipArray with the reference's pairing (j, j + D/2)
    (apply_rotary_embeddings(input, prev_seq; base), reference src/NN.jl:253-303). `pos0` (HipArray
    int32[B]) gives per-sequence start positions instead of the scalar prev_seq; `out` may be x."""
    _require_hip(x)
    if len(x.shape) != 4:
        raise ValueError("rotary embedding expects (B,H,S,D); got %s" % (x.shape,))
    out = out if out is not None else HipArray(x.shape, x.dtype, x.device)
    if out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError("rotary embedding: out must match x in shape and element type")
    p = binding.RopeParams()
    p.out, p.x = out.ptr, x.ptr
    p.pos0 = pos0.ptr if pos0 is not None else None
    p.prev_seq = int(prev_seq)
    p.B, p.H, p.S, p.D = x.shape
    p.dtype = binding.DTYPE_CODES[x.dtype]
    p.base = float(base)
    p.pairing = binding.ROPE_INTERLEAVED if interleaved else binding.ROPE_HALF_SPLIT
    p.stream = stream
    binding.rope(p)
    return out


def kv_append(k_cache, v_cache, k_new, v_new, pos, rope_k=False, base=10000.0, interleaved=False, q=None,
              stream=None):
    """In-place cache update cache[b,h,pos[b]+t,:] = new[b,h,t,:] (the reference rebuilds the whole cache
    with _kv_scatter, reference src/Whisper.jl:552-570). `pos` is a HipArray int32[B] or an int. `q`
    (B,Hq,T,D), if given, is rotated in place at the same positions by the same launch."""
    _require_hip(k_cache, v_cache, k_new, v_new)
    if k_cache.shape != v_cache.shape or k_new.shape != v_new.shape or len(k_cache.shape) != 4:
        raise ValueError("kv_append expects caches (B,Hkv,Lmax,D) and new rows (B,Hkv,T,D)")
    B, Hkv, Lmax, D = k_cache.shape
    if k_new.shape[:2] != (B, Hkv) or k_new.shape[3] != D:
        raise ValueError("kv_append: new rows %s do not match the cache %s" % (k_new.shape, k_cache.shape))
    if not (k_cache.dtype == v_cache.dtype == k_new.dtype == v_new.dtype):
        raise ValueError("kv_append: caches and new rows must share one element type")
    p = binding.KvAppendParams()
    p.k_cache, p.v_cache, p.k_new, p.v_new = k_cache.ptr, v_cache.ptr, k_new.ptr, v_new.ptr
    if isinstance(pos, HipArray):
        p.pos = pos.ptr
    else:
        p.pos, p.pos_all = None, int(pos)
    p.B, p.Hkv, p.T, p.D, p.Lmax = B, Hkv, k_new.shape[2], D, Lmax
    p.dtype = binding.DTYPE_CODES[k_cache.dtype]
    p.rope_k = int(bool(rope_k))
    p.pairing = binding.ROPE_INTERLEAVED if interleaved else binding.ROPE_HALF_SPLIT
    p.base = float(base)
    p.stream = stream
    if q is not None:
        _require_hip(q)
        if len(q.shape) != 4 or q.shape[0] != B or q.shape[2:] != (k_new.shape[2], D) or q.dtype != k_cache.dtype:
            raise ValueError("kv_append: q %s (%s) does not match new rows %s (%s)" %
                             (q.shape, q.dtype, k_new.shape, k_cache.dtype))
        p.q_rope, p.Hq = q.ptr, q.shape[1]
    binding.kv_append(p)


class KVCacheState:
    """Device-resident decode cache: the mirror of KVCacheState (reference src/Whisper.jl:519-540) with
    per-sequence lengths. `append` writes the new rows in place and advances kv_len; `attend` is the
    fused cached attention (reference src/Whisper.jl:584-620) over rows 0 .. kv_len[b]-1."""

    def __init__(self, batch, n_kv_heads, head_dim, max_seq, dtype="f32", device=None):
        self.device = device or get_device()
        self.max_seq = max_seq
        self.k = HipArray((batch, n_kv_heads, max_seq, head_dim), dtype, self.device).fill_bytes(0)
        self.v = HipArray((batch, n_kv_heads, max_seq, head_dim), dtype, self.device).fill_bytes(0)
        self.kv_len_host = np.zeros(batch, np.int32)
        self.kv_len = HipArray((batch,), "i32", self.device).copy_from_host(self.kv_len_host)

    @property
    def step_pos(self):
        return int(self.kv_len_host.max())

    def append(self, k_new, v_new, rope_k=False, base=10000.0):
        T = k_new.shape[2]
        if int(self.kv_len_host.max()) + T > self.max_seq:
            raise ValueError("KV cache is full (max_seq=%d)" % self.max_seq)
        kv_append(self.k, self.v, k_new, v_new, self.kv_len, rope_k=rope_k, base=base)
        self.kv_len_host += T
        self.kv_len.copy_from_host(self.kv_len_host)

    def attend(self, q, scale=None, head_map=HEADMAP_INTERLEAVED, out_dtype=None):
        op = DecodeAttentionOp(default_scale(q.shape[-1]) if scale is None else scale, head_map, 0, out_dtype)
        return execute_op(op, q, self.k, self.v, self.kv_len)


def default_scale(D):
    return float(np.float32(1.0) / np.sqrt(np.float32(D)))


__all__ = [
    "AbstractDevice", "CPUDevice", "HIPDevice", "HipArray", "get_device", "to_device", "from_device", "Graph",
    "GraphTensor", "tensor", "add_op", "FlashAttentionOp", "DecodeAttentionOp", "flash_attention", "decode_attention",
    "RotaryEmbeddingOp", "KVAppendOp", "DecodeStepOp", "decode_step", "decode_step_supported", "rotary_embedding", "kv_cache_append", "self_attention_core",
    "cached_self_attention_core", "prompt_self_attention_core", "FUSED_ROPE_HEAD_DIMS", "HostOp", "MatMulOp", "PermuteOp", "ReshapeOp", "AddOp", "ExpandOp", "matmul", "permute",
    "reshape", "add", "expand", "Linear", "SelfAttention", "WhisperAttention", "execute_op", "execute_op_inplace", "execute", "compile", "CompiledGraph", "execute_with_capture", "release_capture", "HEADMAP_INTERLEAVED",
    "HEADMAP_BLOCKED", "LuminalHipError", "apply_rotary_embeddings", "kv_append", "KVCacheState", "encode", "decode", "f32_to_bf16_bits", "bf16_bits_to_f32", "default_scale",
    "flash_attention_plan",
]
