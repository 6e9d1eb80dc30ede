"""CPU oracle for the attention hot path — TEST INFRASTRUCTURE ONLY.

Nothing under luminal.jl_amd/ imports this package. It is loaded by tests/, by
__graft_entry__.smoke() and by bench.py's cpu_baseline leg, always as the checker.

  * liboracle.so (attn_oracle.c): C restatement of the reference's flash_attn_cpu
    (reference src/Execution.jl:453-479) generalised to cross attention, GQA and per-sequence
    KV lengths, plus an independent float64 naive attention and the seeded input generator.
  * numpy twins here: naive_attention_np (float64, independent of the C code) and the literal
    column-major replay of the reference's repeat_kv (reference src/NN.jl:305-317).

The reference is Julia and no Julia toolchain exists in the build image, so there is no
oracle/_ref build; the C restatement is pinned by closed forms, invariants and golden vectors
(see tests/test_oracle.py).
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")

HEADMAP_INTERLEAVED = 0
HEADMAP_BLOCKED = 1

_lib = None


def build():
    """Compile attn_oracle.c with gcc (always recompiles)."""
    subprocess.run(["make", "-C", HERE, "-B", "-s"], check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        f32p = ctypes.POINTER(ctypes.c_float)
        i32p = ctypes.POINTER(ctypes.c_int32)
        f64p = ctypes.POINTER(ctypes.c_double)
        L.lmo_flash_attn.restype = ctypes.c_int
        L.lmo_flash_attn.argtypes = [f32p, f32p, f32p, f32p, i32p] + [ctypes.c_int] * 6 + [
            ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.lmo_decode_attn.restype = ctypes.c_int
        L.lmo_decode_attn.argtypes = [f32p, f32p, f32p, f32p, i32p] + [ctypes.c_int] * 5 + [
            ctypes.c_float, ctypes.c_int, ctypes.c_int]
        L.lmo_attn_naive_f64.restype = ctypes.c_int
        L.lmo_attn_naive_f64.argtypes = [f64p, f32p, f32p, f32p, i32p] + [ctypes.c_int] * 6 + [
            ctypes.c_double, ctypes.c_int, ctypes.c_int]
        L.lmo_gen_normal.restype = None
        L.lmo_gen_normal.argtypes = [f32p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_float]
        L.lmo_gen_uniform_int.restype = None
        L.lmo_gen_uniform_int.argtypes = [i32p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int32, ctypes.c_int32]
        L.lmo_round_bf16.restype = None
        L.lmo_round_bf16.argtypes = [f32p, ctypes.c_uint64]
        L.lmo_round_f16.restype = None
        L.lmo_round_f16.argtypes = [f32p, ctypes.c_uint64]
        L.lmo_max_threads.restype = ctypes.c_int
        L.lmo_rope.restype = ctypes.c_int
        L.lmo_rope.argtypes = [f32p, f32p, i32p, ctypes.c_int] + [ctypes.c_int] * 4 + [ctypes.c_float, ctypes.c_int]
        L.lmo_kv_append.restype = ctypes.c_int
        L.lmo_kv_append.argtypes = [f32p, f32p, i32p] + [ctypes.c_int] * 5
        _lib = L
    return _lib


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _i32_or_null(a):
    if a is None:
        return None, None
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


def max_threads():
    return int(lib().lmo_max_threads())


def gen_normal(shape, seed, mul=1.0):
    """Seeded N(0,1)*mul fp32 array (SplitMix64 -> Box-Muller), identical in C and in gen_normal_np."""
    out = np.empty(shape, dtype=np.float32)
    lib().lmo_gen_normal(out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), out.size, seed, mul)
    return out


def gen_uniform_int(n, seed, lo, hi):
    out = np.empty(n, dtype=np.int32)
    lib().lmo_gen_uniform_int(out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), n, seed, lo, hi)
    return out


def round_to(x, dtype):
    """Round an fp32 array to the precision of 'f32' | 'f16' | 'bf16' (result stays fp32)."""
    x = np.array(x, dtype=np.float32, order="C", copy=True)
    p = x.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
    if dtype == "bf16":
        lib().lmo_round_bf16(p, x.size)
    elif dtype == "f16":
        lib().lmo_round_f16(p, x.size)
    elif dtype != "f32":
        raise ValueError(dtype)
    return x


def flash_attn(q, k, v, scale=None, causal=False, head_map=HEADMAP_INTERLEAVED, kv_len=None, nthreads=1):
    """Restated flash_attn_cpu. q [B,Hq,Sq,D], k/v [B,Hkv,Sk,D] -> [B,Hq,Sq,D] fp32."""
    q, qp = _f32(q)
    k, kp = _f32(k)
    v, vp = _f32(v)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    assert k.shape == v.shape and k.shape[0] == B and k.shape[3] == D
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(D))  # reference src/HighLevelOps.jl:380-382
    kv, kvp = _i32_or_null(kv_len)
    out = np.empty_like(q)
    rc = lib().lmo_flash_attn(out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), qp, kp, vp, kvp, B, Hq, Hkv, Sq,
                              Sk, D, float(scale), int(bool(causal)), head_map, nthreads)
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return out


def decode_attn(q, k_cache, v_cache, kv_len=None, scale=None, head_map=HEADMAP_INTERLEAVED, nthreads=1):
    """q [B,Hq,D], caches [B,Hkv,Lmax,D] -> [B,Hq,D] fp32, through the oracle's own decode entry lmo_decode_attn
    (the cached attention of reference src/Whisper.jl:610-616: one query row over the first kv_len[b] cache rows)."""
    q, qp = _f32(q)
    k, kp = _f32(k_cache)
    v, vp = _f32(v_cache)
    B, Hq, D = q.shape
    _, Hkv, Lmax, _ = k.shape
    assert k.shape == v.shape and k.shape[0] == B and k.shape[3] == D
    if scale is None:
        scale = np.float32(1.0) / np.sqrt(np.float32(D))
    kv, kvp = _i32_or_null(kv_len)
    out = np.empty_like(q)
    rc = lib().lmo_decode_attn(out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), qp, kp, vp, kvp, B, Hq, Hkv, Lmax, D,
                               float(scale), head_map, nthreads)
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return out


def naive_attention_f64(q, k, v, scale=None, causal=False, head_map=HEADMAP_INTERLEAVED, kv_len=None):
    """C float64 naive softmax attention (second oracle)."""
    q, qp = _f32(q)
    k, kp = _f32(k)
    v, vp = _f32(v)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    if scale is None:
        scale = 1.0 / np.sqrt(float(D))
    kv, kvp = _i32_or_null(kv_len)
    out = np.empty(q.shape, dtype=np.float64)
    rc = lib().lmo_attn_naive_f64(out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)), qp, kp, vp, kvp, B, Hq, Hkv,
                                  Sq, Sk, D, float(scale), int(bool(causal)), head_map)
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return out


def rope(x, prev_seq=0, base=10000.0, pos0=None, interleaved=False):
    """Restated apply_rotary_embeddings on row-major [B,H,S,D] (fp32)."""
    x, xp = _f32(x)
    B, H, S, D = x.shape
    out = np.empty_like(x)
    p0, p0p = _i32_or_null(pos0)
    rc = lib().lmo_rope(out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), xp, p0p, int(prev_seq), B, H, S, D,
                        float(base), int(bool(interleaved)))
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return out


def kv_append(cache, new_rows, pos):
    """cache [B,H,Lmax,D] with new_rows [B,H,T,D] written at rows pos[b]..pos[b]+T-1 (returns a copy)."""
    cache = np.array(cache, dtype=np.float32, order="C", copy=True)
    new_rows, nrp = _f32(new_rows)
    B, H, Lmax, D = cache.shape
    T = new_rows.shape[2]
    pos, posp = _i32_or_null(pos)
    rc = lib().lmo_kv_append(cache.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), nrp, posp, B, H, T, D, Lmax)
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return cache


# ---------------------------------------------------------------------------------------------
# numpy twins (independent of the C code)
# ---------------------------------------------------------------------------------------------
def rope_column_major_replay(x, prev_seq=0, base=10000.0):
    """Literal replay of the reference's apply_rotary_embeddings graph (reference src/NN.jl:253-303):
    every reshape is done in column-major element order, as Base.reshape does on Julia arrays
    (reference src/Execution.jl:228), in float64."""
    x = np.asarray(x, dtype=np.float64)
    B, H, S, D = x.shape
    half = D // 2
    freqs = np.arange(half, dtype=np.float64) * 2.0 / D
    inv_freqs = 1.0 / np.exp2(freqs * np.log2(base))
    pos = np.arange(S, dtype=np.float64) + prev_seq
    emb = pos[:, None] @ inv_freqs[None, :]                               # (S, half)
    split = np.asfortranarray(x).reshape((B, H, S, half, 2), order="F")  # :274
    x0 = split[..., 0]                                                    # slice_along(split, 5, 0, 1)
    x1 = split[..., 1]
    sin_e, cos_e = np.sin(emb)[None, None], np.cos(emb)[None, None]
    x0_out = x0 * cos_e - x1 * sin_e
    x1_out = x0 * sin_e + x1 * cos_e
    res = np.asfortranarray(np.stack([x0_out, x1_out], axis=4))           # concat along dim 5
    return np.ascontiguousarray(res.reshape((B, H, S, D), order="F"))


def kv_scatter_replay(past, new_slot, step_pos):
    """Literal replay of _kv_scatter (reference src/Whisper.jl:552-570): slices of `past` around
    step_pos concatenated with the one-row new_slot along the sequence axis."""
    max_seq = past.shape[2]
    suffix_len = max_seq - step_pos - 1
    if step_pos == 0:
        return np.concatenate([new_slot, past[:, :, 1:max_seq]], axis=2)
    if suffix_len == 0:
        return np.concatenate([past[:, :, 0:step_pos], new_slot], axis=2)
    return np.concatenate([past[:, :, 0:step_pos], new_slot, past[:, :, step_pos + 1:max_seq]], axis=2)

def repeat_kv_column_major(x, groups):
    """Literal replay of the reference's repeat_kv on a column-major array.

    reference src/NN.jl:305-317: expand(keys, 3, groups) then reshape to (B, Hkv*groups, S, D);
    Expand executes as reshape-with-inserted-1 + repeat(outer) (src/Execution.jl:238-248) and
    Reshape as Base.reshape (src/Execution.jl:228), both in column-major element order.
    x: logical (B, Hkv, S, D) -> logical (B, Hkv*groups, S, D).
    """
    B, Hkv, S, D = x.shape
    xf = np.asfortranarray(x)
    expanded = np.asfortranarray(np.repeat(xf.reshape((B, Hkv, 1, S, D), order="F"), groups, axis=2))
    return np.ascontiguousarray(expanded.reshape((B, Hkv * groups, S, D), order="F"))


def naive_attention_np(q, k, v, scale=None, causal=False, head_map=HEADMAP_INTERLEAVED, kv_len=None):
    """float64 numpy softmax(scale * Q K^T + mask) V, the manual attention of the reference's tests
    (reference tests/test_flash_attention_verification.jl:30-35, :60-70; src/NN.jl:369-382)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    G = Hq // Hkv
    if scale is None:
        scale = 1.0 / np.sqrt(float(D))
    if G > 1:
        if head_map == HEADMAP_INTERLEAVED:
            k = repeat_kv_column_major(k, G)
            v = repeat_kv_column_major(v, G)
        else:
            k = np.repeat(k, G, axis=1)
            v = np.repeat(v, G, axis=1)
    s = np.einsum("bhid,bhjd->bhij", q, k) * scale
    mask = np.zeros((B, 1, Sq, Sk), dtype=bool)
    if causal:
        mask |= (np.arange(Sk)[None, :] > np.arange(Sq)[:, None])[None, None]
    if kv_len is not None:
        mask |= (np.arange(Sk)[None, :] >= np.asarray(kv_len)[:, None])[:, None, None, :]
    s = np.where(mask, -np.inf, s)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p = p / p.sum(axis=-1, keepdims=True)
    return np.einsum("bhij,bhjd->bhid", p, v)


_MASK64 = (1 << 64) - 1


def _splitmix64_at_np(seed, index):
    with np.errstate(over="ignore"):
        z = (np.uint64(seed) + (index.astype(np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15))
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def gen_normal_np(shape, seed, mul=1.0):
    """numpy twin of lmo_gen_normal (same bits up to libm's last-ulp differences in log/cos/sin)."""
    n = int(np.prod(shape))
    pairs = np.arange((n + 1) // 2, dtype=np.uint64)
    a = _splitmix64_at_np(seed, 2 * pairs)
    b = _splitmix64_at_np(seed, 2 * pairs + np.uint64(1))
    u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = (b >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * len(pairs), dtype=np.float32)
    out[0::2] = (r * np.cos(2 * np.pi * u2)).astype(np.float32) * np.float32(mul)
    out[1::2] = (r * np.sin(2 * np.pi * u2)).astype(np.float32) * np.float32(mul)
    return out[:n].reshape(shape)
