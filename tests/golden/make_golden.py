"""Writes tests/golden/attention_cases.npz: small attention problems with float64 expected outputs.

Inputs are stored as bf16 bit patterns (uint16) of values that fp32, fp16 and bf16 all represent
exactly; expected outputs as fp32 roundings of the float64 result.

Self-contained on purpose: inputs come from numpy's PCG64 (not from the oracle's generator) and the
expected outputs from the ~20 lines of numpy below (not from oracle/), so the fixtures pin the
oracle and the HIP kernels from outside. The reference ships no attention fixtures of its own
(its tests draw unseeded random inputs: reference tests/test_flash_attention_verification.jl:15-17),
so these are synthetic inputs of the shapes its tests and models use.

GQA cases replay the reference's repeat_kv literally: Expand(dim 3) then Reshape on column-major
arrays (reference src/NN.jl:305-317, src/Execution.jl:238-248, :228).

Run: python tests/golden/make_golden.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def repeat_kv_julia(x, groups):
    B, Hkv, S, D = x.shape
    xf = np.asfortranarray(x)
    e = np.asfortranarray(np.repeat(xf.reshape((B, Hkv, 1, S, D), order="F"), groups, axis=2))
    return np.ascontiguousarray(e.reshape((B, Hkv * groups, S, D), order="F"))


def attention64(q, k, v, scale, causal, kv_len=None):
    q, k, v = (np.asarray(a, dtype=np.float64) for a in (q, k, v))
    G = q.shape[1] // k.shape[1]
    if G > 1:
        k, v = repeat_kv_julia(k, G), repeat_kv_julia(v, G)
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    out = np.zeros_like(q)
    for b in range(B):
        n = Sk if kv_len is None else int(kv_len[b])
        for h in range(H):
            for i in range(Sq):
                hi = min(n, i + 1) if causal else n
                s = (k[b, h, :hi] @ q[b, h, i]) * scale
                w = np.exp(s - s.max())
                out[b, h, i] = (w / w.sum()) @ v[b, h, :hi]
    return out


def bf16_exact(x):
    """Round to values that bf16, fp16 and fp32 all represent exactly (8-bit significand, magnitudes
    below fp16's normal range flushed to zero), so one fixture serves every element type."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32)
    u = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    f = u.view(np.float32).copy()
    f[np.abs(f) < 2.0 ** -14] = 0.0
    return f


def main():
    rng = np.random.Generator(np.random.PCG64(20240607))
    cases = {}

    def add(name, B, Hq, Hkv, Sq, Sk, D, causal, kv_len=None, scale=None):
        q = bf16_exact(rng.standard_normal((B, Hq, Sq, D)))
        k = bf16_exact(rng.standard_normal((B, Hkv, Sk, D)))
        v = bf16_exact(rng.standard_normal((B, Hkv, Sk, D)))
        if scale is None:
            scale = float(np.float32(1.0) / np.sqrt(np.float32(D)))
        # stored as bf16 bit patterns (exact), half the bytes of fp32
        for key, arr in (("q", q), ("k", k), ("v", v)):
            cases[name + "." + key] = (arr.view(np.uint32) >> np.uint32(16)).astype(np.uint16)
        cases[name + ".meta"] = np.array([int(causal), scale], dtype=np.float64)
        if kv_len is not None:
            cases[name + ".kv_len"] = np.asarray(kv_len, dtype=np.int32)
        cases[name + ".out"] = attention64(q, k, v, scale, causal, kv_len).astype(np.float32)

    # the shape of the reference's own attention tests (B=H=1, S=8, D=16)
    add("ref_shape_noncausal", 1, 1, 1, 8, 8, 16, False)
    add("ref_shape_causal", 1, 1, 1, 8, 8, 16, True)
    add("mha_causal_d64", 1, 2, 2, 20, 20, 64, True)
    add("cross_d64", 1, 2, 2, 5, 19, 64, False)                  # Sq != Sk, no mask
    add("gqa_causal_d32", 1, 4, 2, 9, 9, 32, True)             # G = 2, interleaved head map
    add("gqa_cross_d128", 1, 8, 2, 3, 11, 128, False)          # G = 4
    add("decode_gqa_d128", 3, 8, 2, 1, 12, 128, False, kv_len=[12, 7, 1])
    add("scaled_d96", 1, 1, 1, 34, 34, 96, True, scale=0.37)
    np.savez_compressed(os.path.join(HERE, "attention_cases.npz"), **cases)
    print("wrote", len(cases), "arrays")


if __name__ == "__main__":
    main()
