"""A literal float64 replay of the reference's SelfAttention layer (reference src/NN.jl:319-387), shared by the CPU and
GPU tests of the layer: the arrays are indexed like the reference's Julia arrays and every reshape is column-major
(order='F'), as Base.reshape is."""
import numpy as np


def reference_layer_f64(x, wq, wk, wv, wo, n_heads, n_kv_heads, prev_seq, base=10000.0):
    """The reference's SelfAttention, node by node, on arrays indexed like its Julia arrays; every reshape is
    column-major (order='F'), as Base.reshape is."""
    x, wq, wk, wv, wo = (np.asarray(a, np.float64) for a in (x, wq, wk, wv, wo))
    B, S, hidden = x.shape
    D = hidden // n_heads

    def heads(w, n):  # src/NN.jl:346-353
        return np.transpose(np.reshape(x @ w.T, (B, S, n, D), order="F"), (0, 2, 1, 3))

    def rope(t):  # src/NN.jl:253-303
        b, h, s, d = t.shape
        half = d // 2
        freqs = np.arange(half) * 2.0 / d
        inv = 1.0 / np.exp2(freqs * np.log2(base))
        emb = (np.arange(s) + prev_seq)[:, None] * inv[None, :]
        split = np.reshape(t, (b, h, s, half, 2), order="F")
        x0, x1 = split[..., 0], split[..., 1]
        x0o, x1o = x0 * np.cos(emb) - x1 * np.sin(emb), x0 * np.sin(emb) + x1 * np.cos(emb)
        return np.reshape(np.stack([x0o, x1o], axis=4), (b, h, s, d), order="F")

    def repeat_kv(t, groups):  # src/NN.jl:305-317
        b, kvh, s, d = t.shape
        return np.reshape(np.repeat(t[:, :, None], groups, axis=2), (b, kvh * groups, s, d), order="F")

    q, k, v = rope(heads(wq, n_heads)), rope(heads(wk, n_kv_heads)), heads(wv, n_kv_heads)
    g = n_heads // n_kv_heads
    k, v = repeat_kv(k, g), repeat_kv(v, g)
    w = q @ np.transpose(k, (0, 1, 3, 2)) / np.sqrt(D)
    if S > 1:
        w = w + np.triu(np.ones((S, S)), 1) * -1e9
    w = np.exp(w - w.max(-1, keepdims=True))
    p = w / w.sum(-1, keepdims=True)
    out = np.reshape(np.transpose(p @ v, (0, 2, 1, 3)), (B, S, hidden), order="F")
    return out @ wo.T


def reference_whisper_attention_f64(x, wq, bq, wk, wv, bv, wo, bo, n_heads, mask, enc=None):
    """WhisperSelfAttention (reference src/Whisper.jl:253-272) or, with `enc` (the encoder output the keys and values are
    projected from), WhisperCrossAttention (:295-316), node by node in float64: q and k scaled by D^-0.25 each, additive
    -1e9 strict upper mask for self attention with mask, column-major reshapes."""
    x, wq, bq, wk, wv, bv, wo, bo = (np.asarray(a, np.float64) for a in (x, wq, bq, wk, wv, bv, wo, bo))
    src = x if enc is None else np.asarray(enc, np.float64)
    B, S, hidden = x.shape
    Sk = src.shape[1]
    D = hidden // n_heads
    scale = float(D) ** -0.25

    def heads(t, s_len):
        return np.transpose(np.reshape(t, (B, s_len, n_heads, D), order="F"), (0, 2, 1, 3))

    q = heads((x @ wq.T + bq) * scale, S)
    k = heads((src @ wk.T) * scale, Sk)
    v = heads(src @ wv.T + bv, Sk)
    w = q @ np.transpose(k, (0, 1, 3, 2))
    if mask:
        w = w + np.triu(np.ones((S, Sk)), 1) * -1e9
    w = np.exp(w - w.max(-1, keepdims=True))
    p = w / w.sum(-1, keepdims=True)
    out = np.reshape(np.transpose(p @ v, (0, 2, 1, 3)), (B, S, hidden), order="F")
    return out @ wo.T + bo
