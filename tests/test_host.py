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


def test_cached_attention_core_emits_two_fused_nodes(lm):
    # in-place append that also rotates q (K rotated on the way in), then fused cached attention; positions are tensors
    B, Hq, Hkv, D, Lmax = 2, 8, 2, 64, 32
    g = lm.Graph()
    q, kn, vn = lm.tensor(g, (B, Hq, 1, D)), lm.tensor(g, (B, Hkv, 1, D)), lm.tensor(g, (B, Hkv, 1, D))
    kc, vc = lm.tensor(g, (B, Hkv, Lmax, D)), lm.tensor(g, (B, Hkv, Lmax, D))
    pos, kv_len = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
    n_inputs = len(g.nodes)
    out, kc2, vc2 = lm.cached_self_attention_core(q, kn, vn, kc, vc, pos, kv_len, rope_base=10000.0)
    ops = [type(n.op).__name__ for n in g.nodes[n_inputs:]]
    assert ops == ["KVAppendOp", "DecodeAttentionOp"]
    app, att = g.nodes[n_inputs:]
    assert app.op.rope_k is True and app.op.rope_q is True
    assert [i[0] for i in app.inputs] == [kc.id, vc.id, kn.id, vn.id, pos.id, q.id]
    # attention reads outputs 2 (the rotated q, as (B, Hq, D)), 0 and 1 (the caches after the update) of the append node
    assert [(i[0], i[1]) for i in att.inputs] == [(n_inputs, 2), (kc2.id, 0), (vc2.id, 1), (kv_len.id, 0)]
    assert att.inputs[0][2] == (B, Hq, D) and out.shape == (B, Hq, D)
    assert kc2.id == vc2.id == n_inputs and (kc2.index, vc2.index) == (0, 1)
    with pytest.raises(ValueError):
        lm.cached_self_attention_core(lm.tensor(g, (B, Hq, 2, D)), kn, vn, kc, vc, pos, kv_len)
    # without a rotary embedding the append node takes no q
    g2 = lm.Graph()
    q, kn, vn = lm.tensor(g2, (B, Hq, 1, D)), lm.tensor(g2, (B, Hkv, 1, D)), lm.tensor(g2, (B, Hkv, 1, D))
    kc, vc = lm.tensor(g2, (B, Hkv, Lmax, D)), lm.tensor(g2, (B, Hkv, Lmax, D))
    pos, kv_len = lm.tensor(g2, (B,), "i32"), lm.tensor(g2, (B,), "i32")
    n_inputs = len(g2.nodes)
    lm.cached_self_attention_core(q, kn, vn, kc, vc, pos, kv_len)
    app, att = g2.nodes[n_inputs:]
    assert app.op.rope_q is False and len(app.inputs) == 5 and att.inputs[0][0] == q.id


def test_self_attention_core_without_rope_is_one_flash_node(lm):
    # Whisper's layers: no rotary embedding; cross attention is the same node with causal=False
    g = lm.Graph()
    q, k, v = lm.tensor(g, (4, 20, 448, 64), "f16"), lm.tensor(g, (4, 20, 1500, 64), "f16"), lm.tensor(g, (4, 20, 1500, 64), "f16")
    n = len(g.nodes)
    out = lm.self_attention_core(q, k, v, causal=False)
    assert len(g.nodes) == n + 1 and isinstance(g.nodes[out.id].op, lm.FlashAttentionOp)
    assert g.nodes[out.id].op.causal is False and out.shape == q.shape
    out2 = lm.self_attention_core(q, k, v, causal=True, prev_seq=3, rope_base=10000.0)
    # head dim 64: K gets a rotary node, the queries are rotated inside the attention kernel
    kinds = [type(x.op).__name__ for x in g.nodes[n + 1:]]
    assert kinds == ["RotaryEmbeddingOp", "FlashAttentionOp"]
    assert g.nodes[n + 1].op.prev_seq == 3 and g.nodes[n + 1].inputs[0][0] == k.id
    att = g.nodes[out2.id].op
    assert att.causal is True and att.q_rope_base == 10000.0 and att.q_prev_seq == 3 and not att.has_q_pos0
    # a head dim the kernels do not rotate in registers keeps both rotary nodes
    g3 = lm.Graph()
    q3, k3, v3 = (lm.tensor(g3, (1, 4, 32, 80), "f16") for _ in range(3))
    out3 = lm.self_attention_core(q3, k3, v3, rope_base=10000.0)
    kinds = [type(x.op).__name__ for x in g3.nodes[3:]]
    assert kinds == ["RotaryEmbeddingOp", "RotaryEmbeddingOp", "FlashAttentionOp"] and g3.nodes[out3.id].op.q_rope_base is None


def test_prompt_core_is_append_plus_attention_over_the_cache(lm):
    g = lm.Graph()
    B, Hq, Hkv, T, D, Lmax = 2, 8, 2, 16, 128, 64
    q, kn, vn = lm.tensor(g, (B, Hq, T, D), "bf16"), lm.tensor(g, (B, Hkv, T, D), "bf16"), lm.tensor(g, (B, Hkv, T, D), "bf16")
    kc, vc = lm.tensor(g, (B, Hkv, Lmax, D), "bf16"), lm.tensor(g, (B, Hkv, Lmax, D), "bf16")
    pos, kv_len = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
    n = len(g.nodes)
    out, kc2, vc2 = lm.prompt_self_attention_core(q, kn, vn, kc, vc, pos, kv_len, rope_base=10000.0)
    app, att = g.nodes[n:]
    assert isinstance(app.op, lm.KVAppendOp) and app.op.rope_k and not app.op.rope_q
    assert isinstance(att.op, lm.FlashAttentionOp) and att.op.causal and att.op.has_kv_len and att.op.has_q_pos0
    assert [r[0] for r in att.inputs] == [q.id, kc2.id, kc2.id, kv_len.id, pos.id] and att.inputs[2][1] == 1
    assert out.shape == q.shape
    with pytest.raises(ValueError):
        lm.FlashAttentionOp(0.1, True, has_q_pos0=True)  # positions without a rotary base


def test_execute_with_capture_without_a_hip_device_just_runs(lm):
    # reference src/Device.jl:121: execute_with_capture(::AbstractDevice, f, cache) = f()
    calls, cache = [], {}
    assert lm.execute_with_capture(lm.CPUDevice(), lambda stream: calls.append(stream) or 7, cache) == 7
    assert calls == [None] and cache == {}
    lm.release_capture(cache)  # nothing recorded: a no-op
    assert cache == {}


def test_package_input_generator_is_the_oracles_generator(lm, oracle):
    # bench.py draws its inputs from the package's own generator; the tests draw theirs from the oracle's C one.
    # Same specification, so the same seeds give the same configurations (libm and numpy may differ in the last
    # bit of a float64 log / cos / sin, which survives the rounding to float32 only rarely).
    for shape, seed, mul in [((3, 5, 7), 2000, 0.5), ((1001,), 3000, 1.0), ((2, 64), 4002, 1.0)]:
        a, b = lm.synth.normal(shape, seed, mul), oracle.gen_normal(shape, seed, mul)
        assert a.shape == b.shape and a.dtype == b.dtype
        ulp = np.abs(a.view(np.int32).astype(np.int64) - b.view(np.int32).astype(np.int64))
        assert ulp.max() <= 1 and (ulp != 0).mean() < 1e-3
    np.testing.assert_array_equal(lm.synth.uniform_int(64, 5000, 8192, 32768), oracle.gen_uniform_int(64, 5000, 8192, 32768))
    big = lm.synth.normal((1 << 16,), 7, chunk_pairs=1000)  # chunking does not change the stream
    np.testing.assert_array_equal(big, lm.synth.normal((1 << 16,), 7))
    assert abs(float(big.mean())) < 0.02 and abs(float(big.std()) - 1.0) < 0.02


def test_kernel_plan_of_the_benchmark_configurations(lm):
    """Which kernel a launch reaches is decided on the host from shapes alone (the plan query launches nothing and
    needs no GPU; without one the launchers assume 256 compute units)."""
    plan = lm.flash_attention_plan
    # C1: the reference's own fp32 example, far too small to fill the chip -> fp32 matrix cores, keys split four ways
    assert plan((1, 8, 128, 64), (1, 8, 128, 64), "f32", True).startswith("prefill_f32_kernel<D=64, causal, key groups=4>")
    # C2: 32 heads x 16 tiles of 256 rows = 256 pairs (tile p with tile 15 - p), one workgroup per CU, one round
    assert plan((1, 32, 4096, 96), (1, 32, 4096, 96), "f16", True) == \
        "prefill_mfma_pair_kernel<f16, D=96, causal> query tiles=16, workgroups=256"
    # the same in bf16 (V rewritten as fp16 through registers: no room for two row blocks), or with the chip not exactly
    # full: 512 workgroups of 256 rows, one per CU at a time, 128-key tiles
    assert plan((1, 32, 4096, 96), (1, 32, 4096, 96), "bf16", True).startswith(
        "prefill_mfma_kernel<bf16, D=96, causal, key groups=1, waves=8, waves per SIMD=2> workgroups=512")
    # ... in bf16 however many rounds there are (fp16 goes to two workgroups per CU from three rounds on)
    assert "waves=8, waves per SIMD=2> workgroups=2048, V as fp16" in plan((4, 32, 4096, 96), (4, 32, 4096, 96), "bf16", True)
    # bf16 hands V to the matrix cores as fp16 from about 512 keys per query row on (1024 at the D = 96 tiling), and only in
    # the launches of one key group
    assert plan((1, 32, 4096, 96), (1, 32, 4096, 96), "bf16", True).endswith("V as fp16")
    assert plan((16, 32, 1024, 128), (16, 32, 1024, 128), "bf16", True).endswith("V as fp16")
    assert not plan((16, 32, 1024, 96), (16, 32, 1024, 96), "bf16", True).endswith("V as fp16")
    assert not plan((16, 32, 512, 128), (16, 32, 512, 128), "bf16", True).endswith("V as fp16")
    assert plan((16, 32, 512, 128), (16, 32, 512, 128), "bf16", False).endswith("V as fp16")
    assert "key groups=2" in plan((1, 8, 1024, 64), (1, 8, 1024, 64), "bf16", True)
    assert not plan((1, 8, 1024, 64), (1, 8, 1024, 64), "bf16", True).endswith("V as fp16")
    assert "waves=8, waves per SIMD=4> workgroups=2048" in plan((4, 32, 4096, 96), (4, 32, 4096, 96), "f16", True)
    assert plan((1, 40, 4096, 96), (1, 40, 4096, 96), "f16", True).startswith(
        "prefill_mfma_kernel<f16, D=96, causal, key groups=1, waves=8, waves per SIMD=2> workgroups=640")
    # C3: 80 heads x 14 row blocks on 256 CUs -> three workgroups per head of five row blocks; two of the five are split
    # between two waves and three between four (16 waves, every SIMD walks 5/4 of a block's keys)
    assert plan((4, 20, 448, 64), (4, 20, 1500, 64), "f16", False) == \
        "prefill_mfma_wide_kernel<f16, D=64> workgroups per head=3, waves=16, workgroups=240, two and four key groups"
    # seven row blocks per workgroup likewise (7/4 against 2 with two key groups each); two or three row blocks: equal groups
    assert plan((4, 20, 672, 64), (4, 20, 1500, 64), "f16", False).endswith("waves=16, workgroups=240, two and four key groups")
    assert plan((2, 20, 448, 64), (2, 20, 1500, 64), "f16", False).endswith("workgroups per head=6, waves=12, workgroups=240")
    # the same heads against few keys, or causal: 64-row workgroups whose wave pairs split the keys
    assert "key groups=2, waves=4" in plan((4, 20, 448, 64), (4, 20, 512, 64), "f16", False)
    assert "key groups=2, waves=4" in plan((4, 20, 448, 64), (4, 20, 1500, 64), "f16", True)
    # 64 heads: two 64-row workgroups per CU already balance
    assert "prefill_mfma_kernel<f16, D=64, full, key groups=2" in plan((4, 16, 448, 64), (4, 16, 1500, 64), "f16", False)
    # head dims the matrix-core kernels do not tile, unaligned scale
    assert plan((2, 4, 100, 136), (2, 4, 100, 136), "bf16", False).startswith("prefill_valu_kernel<bf16, head dim 136 padded to 192>")
    assert plan((2, 4, 100, 64), (2, 4, 100, 64), "f16", False, scale=-1.0).startswith("prefill_valu_kernel<f16")
    with pytest.raises(lm.LuminalHipError):
        plan((2, 4, 100, 264), (2, 4, 100, 264), "f16", False)


def test_host_ops_follow_the_reference_semantics(lm):
    # Reshape is Base.reshape on a column-major array (reference src/Execution.jl:228): splitting 6 into (2, 3) makes the
    # first new axis the fast one
    a = np.arange(12, dtype=np.float32).reshape(2, 6)
    r = lm.ReshapeOp((2, 2, 3)).compute(a)
    assert r[0, 1, 0] == a[0, 1] and r[0, 0, 1] == a[0, 2] and r[1, 1, 2] == a[1, 5]
    assert np.array_equal(lm.PermuteOp((1, 0)).compute(a), a.T)
    e = lm.ExpandOp(1, 3).compute(a)  # (2, 3, 6), every copy equal (reference src/Execution.jl:238-248)
    assert e.shape == (2, 3, 6) and np.array_equal(e[:, 2], a)
    b3 = np.ones((4, 2, 6), np.float32)
    assert lm.MatMulOp().compute(b3, a.T).shape == (4, 2, 2)  # ND x 2D (reference src/Execution.jl:12-90)
    with pytest.raises(ValueError, match="mismatch"):
        lm.MatMulOp().compute(a, a)
    assert np.array_equal(lm.AddOp().compute(b3, a[0]), b3 + a[0])
    # on host arrays the fallback has no device to work for: the attention backend has no CPU path
    with pytest.raises(TypeError):
        lm.execute_op(lm.MatMulOp(), a, a.T)


def test_self_attention_layer_graph_and_its_semantics_against_the_reference_replay(lm, oracle):
    """The layer's graph is the reference's own nodes around one fused core; and that decomposition — heads split by a
    column-major reshape, rotary pairs (j, j + D/2), KV head of query head hq = hq % Hkv — reproduces the reference
    layer replayed literally in float64 (repeat_kv, additive mask, softmax), here with the oracle as the core."""
    from layer_reference import reference_layer_f64
    B, S, hidden, n_heads, n_kv_heads, prev_seq = 2, 24, 64, 4, 2, 3
    D = hidden // n_heads
    g = lm.Graph()
    tx = lm.tensor(g, (B, S, hidden))
    layer = lm.SelfAttention(hidden, n_heads, n_kv_heads, g)
    out = layer(tx, prev_seq)
    kinds = [type(n.op).__name__ for n in g.nodes[5:]]
    assert kinds == ["PermuteOp", "MatMulOp", "ReshapeOp", "PermuteOp"] * 3 + ["RotaryEmbeddingOp", "RotaryEmbeddingOp",
                                                                              "FlashAttentionOp", "PermuteOp", "ReshapeOp",
                                                                              "PermuteOp", "MatMulOp"]
    assert out.shape == (B, S, hidden)
    x = oracle.gen_normal((B, S, hidden), 31)
    ws = [oracle.gen_normal(shape, 32 + i, 1.0 / np.sqrt(hidden)) for i, shape in
          enumerate([(hidden, hidden), (n_kv_heads * D, hidden), (n_kv_heads * D, hidden), (hidden, hidden)])]
    want = reference_layer_f64(x, *ws, n_heads, n_kv_heads, prev_seq)

    def heads(w, n):
        h = lm.ReshapeOp((B, S, n, D)).compute(lm.MatMulOp().compute(x, lm.PermuteOp((1, 0)).compute(w)))
        return np.ascontiguousarray(lm.PermuteOp((0, 2, 1, 3)).compute(h))

    q, k, v = heads(ws[0], n_heads), heads(ws[1], n_kv_heads), heads(ws[2], n_kv_heads)
    att = oracle.flash_attn(oracle.rope(q, prev_seq=prev_seq), oracle.rope(k, prev_seq=prev_seq), v, causal=True)
    merged = lm.ReshapeOp((B, S, hidden)).compute(lm.PermuteOp((0, 2, 1, 3)).compute(att))
    got = lm.MatMulOp().compute(merged, ws[3].T)
    assert np.abs(got - want).max() / np.abs(want).max() <= 2e-5
    # the row-major (HuggingFace) conventions would not: blocked head map, or a row-major head split
    att_blocked = oracle.flash_attn(oracle.rope(q, prev_seq=prev_seq), oracle.rope(k, prev_seq=prev_seq), v, causal=True, head_map=1)
    wrong = lm.MatMulOp().compute(lm.ReshapeOp((B, S, hidden)).compute(lm.PermuteOp((0, 2, 1, 3)).compute(att_blocked)), ws[3].T)
    assert np.abs(wrong - want).max() / np.abs(want).max() > 1e-2
