"""A whole attention layer of a model graph on a HIPDevice: SelfAttention (reference src/NN.jl:319-387) with its
projections, reshapes and permutes served by the host fallback and everything between them by the fused GPU ops.
Checked against a literal float64 replay of the reference layer (column-major reshapes, apply_rotary_embeddings,
repeat_kv, additive -1e9 mask, softmax), which pins the head split, the rotary pairing and the GQA head order at once,
and against the oracle's attention between float64 projections."""
import numpy as np
import pytest

from conftest import rel_err
from layer_reference import reference_layer_f64

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("attn_dtype,n_heads,n_kv_heads,hidden,seq", [
    ("f32", 8, 2, 512, 96),     # head dim 64, GQA
    ("f16", 4, 4, 384, 200),    # head dim 96, MHA
    ("bf16", 8, 4, 1024, 130),  # head dim 128
    ("f32", 4, 2, 160, 40),     # head dim 40: the rotary nodes stay separate
])
def test_llama_shaped_attention_layer_runs_with_attention_on_the_gpu(lm, hip, oracle, attn_dtype, n_heads, n_kv_heads, hidden, seq):
    B, prev_seq = 2, 5
    D = hidden // n_heads
    x = oracle.gen_normal((B, seq, hidden), 15000)
    ws = [oracle.gen_normal(shape, 15001 + i, 1.0 / np.sqrt(hidden)) for i, shape in
          enumerate([(hidden, hidden), (n_kv_heads * D, hidden), (n_kv_heads * D, hidden), (hidden, hidden)])]
    g = lm.Graph()
    tx = lm.tensor(g, x.shape)
    layer = lm.SelfAttention(hidden, n_heads, n_kv_heads, g, attn_dtype=attn_dtype)
    out = layer(tx, prev_seq)
    kinds = [type(n.op).__name__ for n in g.nodes]
    assert kinds.count("FlashAttentionOp") == 1 and kinds.count("MatMulOp") == 4
    assert kinds.count("RotaryEmbeddingOp") == (1 if D in lm.FUSED_ROPE_HEAD_DIMS else 2)
    feeds = {tx.id: x, layer.q_proj.weight.id: ws[0], layer.k_proj.weight.id: ws[1], layer.v_proj.weight.id: ws[2],
             layer.o_proj.weight.id: ws[3]}
    got = lm.execute(g, out.id, feeds, hip)
    want = reference_layer_f64(x, *ws, n_heads, n_kv_heads, prev_seq)
    tol = {"f32": 3e-5, "f16": 3e-3, "bf16": 8e-3}[attn_dtype]  # bf16: q, k, v are rounded to 8 bits before attention
    assert rel_err(got, want) <= tol
    # the same through the compiled form: persistent node buffers, one step per node
    cg = lm.compile(g, hip)
    res = cg(feeds)
    np.testing.assert_array_equal(res[out.id].to_host(), got)
    with pytest.raises(RuntimeError, match="host"):
        cg.capture()


def test_attention_between_float64_projections_equals_the_oracle(lm, hip, oracle):
    """The middle of the layer against the oracle: q, k, v computed on the host in float64 with the layer's head split,
    the oracle's rope and attention (INTERLEAVED head map = repeat_kv's order), o_proj in float64."""
    B, S, hidden, n_heads, n_kv_heads, prev_seq = 1, 64, 256, 4, 2, 0
    D = hidden // n_heads
    x = oracle.gen_normal((B, S, hidden), 15100)
    ws = [oracle.gen_normal(shape, 15101 + i, 1.0 / np.sqrt(hidden)) for i, shape in
          enumerate([(hidden, hidden), (n_kv_heads * D, hidden), (n_kv_heads * D, hidden), (hidden, hidden)])]
    g = lm.Graph()
    tx = lm.tensor(g, x.shape)
    layer = lm.SelfAttention(hidden, n_heads, n_kv_heads, g)
    out = layer(tx, prev_seq)
    got = lm.execute(g, out.id, {tx.id: x, layer.q_proj.weight.id: ws[0], layer.k_proj.weight.id: ws[1],
                                 layer.v_proj.weight.id: ws[2], layer.o_proj.weight.id: ws[3]}, hip)
    x64 = x.astype(np.float64)

    def heads(w, n):
        return np.transpose(np.reshape(x64 @ w.astype(np.float64).T, (B, S, n, D), order="F"), (0, 2, 1, 3)).astype(np.float32)

    q, k, v = heads(ws[0], n_heads), heads(ws[1], n_kv_heads), heads(ws[2], n_kv_heads)
    att = oracle.flash_attn(oracle.rope(q), oracle.rope(k), v, causal=True, head_map=0)
    want = np.reshape(np.transpose(att.astype(np.float64), (0, 2, 1, 3)), (B, S, hidden), order="F") @ ws[3].astype(np.float64).T
    assert rel_err(got, want) <= 3e-5


@pytest.mark.parametrize("attn_dtype,cross", [("f32", False), ("f16", False), ("f16", True), ("bf16", True)])
def test_whisper_attention_layers_run_with_attention_on_the_gpu(lm, hip, oracle, attn_dtype, cross):
    """WhisperSelfAttention (masked) and WhisperCrossAttention (reference src/Whisper.jl:238-316) built by the mirror —
    biased projections on the host, one flash attention node on the GPU — against a float64 replay of the reference
    layers; Whisper-tiny's width (6 heads of 64)."""
    from layer_reference import reference_whisper_attention_f64
    B, S, Senc, hidden, n_heads = 2, 70, 150, 384, 6
    x = oracle.gen_normal((B, S, hidden), 15200)
    enc = oracle.gen_normal((B, Senc, hidden), 15201) if cross else None
    ws = [oracle.gen_normal((hidden, hidden), 15210 + i, 1.0 / np.sqrt(hidden)) for i in range(4)]
    bs = [oracle.gen_normal((hidden,), 15220 + i, 0.1) for i in range(3)]
    g = lm.Graph()
    tx = lm.tensor(g, x.shape)
    tenc = lm.tensor(g, enc.shape) if cross else None
    layer = lm.WhisperAttention(hidden, n_heads, g, attn_dtype=attn_dtype)
    out = layer(tx, mask=not cross, keys_from=tenc, values_from=tenc)
    assert sum(isinstance(n.op, lm.FlashAttentionOp) for n in g.nodes) == 1
    feed = {tx.id: x, layer.q_proj.weight.id: ws[0], layer.q_proj.bias.id: bs[0], layer.k_proj.weight.id: ws[1],
            layer.v_proj.weight.id: ws[2], layer.v_proj.bias.id: bs[1], layer.o_proj.weight.id: ws[3], layer.o_proj.bias.id: bs[2]}
    if cross:
        feed[tenc.id] = enc
    got = lm.execute(g, out.id, feed, hip)
    want = reference_whisper_attention_f64(x, ws[0], bs[0], ws[1], ws[2], bs[1], ws[3], bs[2], n_heads, mask=not cross, enc=enc)
    tol = {"f32": 2e-5, "f16": 3e-3, "bf16": 1.5e-2}[attn_dtype]  # half precision: q, k, v are rounded before attention
    assert rel_err(got, want) <= tol
    cg = lm.compile(g, hip)
    res = cg(feed)
    assert rel_err(res[out.id].to_host(), want) <= tol
