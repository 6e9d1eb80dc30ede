"""Host-side mirror of the reference's operator API (no GPU needed): graph building follows
flash_attention in reference src/HighLevelOps.jl:377-388, and attention ops refuse host arrays
(there is no CPU path behind this backend)."""
import numpy as np
import pytest


def test_flash_attention_builder_matches_reference(lm):
    g = lm.Graph()
    q = lm.tensor(g, (1, 8, 128, 64))
    k = lm.tensor(g, (1, 8, 128, 64))
    v = lm.tensor(g, (1, 8, 128, 64))
    out = lm.flash_attention(q, k, v, causal=True)
    node = g.nodes[out.id]
    assert isinstance(node.op, lm.FlashAttentionOp)
    assert node.op.causal is True
    assert node.op.scale == float(np.float32(1.0) / np.sqrt(np.float32(64)))  # scale = 1f0/sqrt(Float32(D))
    assert [i[0] for i in node.inputs] == [q.id, k.id, v.id]
    assert out.shape == q.shape  # "Output has same shape as Q"
    out2 = lm.flash_attention(q, k, v, scale=0.3)
    assert g.nodes[out2.id].op.causal is False
    assert g.nodes[out2.id].op.scale == float(np.float32(0.3))
    assert g.nodes[out2.id].op.head_map == lm.HEADMAP_INTERLEAVED  # the reference's repeat_kv order


def test_output_shape_follows_q_for_cross_and_gqa(lm):
    g = lm.Graph()
    q = lm.tensor(g, (4, 20, 448, 64), "f16")
    k = lm.tensor(g, (4, 20, 1500, 64), "f16")
    v = lm.tensor(g, (4, 20, 1500, 64), "f16")
    out = lm.flash_attention(q, k, v)
    assert out.shape == (4, 20, 448, 64) and g.dtypes[out.id] == "f16"
    qd = lm.tensor(g, (16, 32, 128), "bf16")
    kc = lm.tensor(g, (16, 8, 4096, 128), "bf16")
    vc = lm.tensor(g, (16, 8, 4096, 128), "bf16")
    ln = lm.tensor(g, (16,), "i32")
    d = lm.decode_attention(qd, kc, vc, ln)
    assert d.shape == (16, 32, 128)
    assert isinstance(g.nodes[d.id].op, lm.DecodeAttentionOp)
    assert abs(g.nodes[d.id].op.scale - 128 ** -0.5) < 1e-7


def test_bf16_encoding_round_trip(lm, oracle):
    x = oracle.gen_normal((4096,), 77)
    bits = lm.f32_to_bf16_bits(x)
    back = lm.bf16_bits_to_f32(bits)
    np.testing.assert_array_equal(back, oracle.round_to(x, "bf16"))
    np.testing.assert_array_equal(lm.decode(lm.encode(x, "f16"), "f16"), oracle.round_to(x, "f16"))
    # ties round to even
    tie = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], dtype=np.float32)
    np.testing.assert_array_equal(lm.bf16_bits_to_f32(lm.f32_to_bf16_bits(tie)),
                                  np.array([1.0, 1.0 + 2.0 ** -6], dtype=np.float32))


def test_attention_ops_refuse_host_arrays(lm):
    op = lm.FlashAttentionOp(0.125, True)
    a = np.zeros((1, 1, 8, 16), np.float32)
    with pytest.raises(TypeError, match="no CPU path"):
        lm.host.execute_op(op, a, a, a)
    with pytest.raises(TypeError, match="no CPU path"):
        lm.host.execute_op_inplace(a, op, a, a, a)


def test_execute_needs_values_for_inputs(lm):
    g = lm.Graph()
    q = lm.tensor(g, (1, 1, 8, 16))
    out = lm.flash_attention(q, q, q)
    with pytest.raises(KeyError):
        lm.execute(g, out.id, {}, lm.CPUDevice())
