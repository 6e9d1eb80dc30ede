"""The rotary embedding of the queries done inside the flash attention kernels (lmh_attn_params.q_rope): the
reference rotates q and k directly in front of attention (reference src/NN.jl:357-358, apply_rotary_embeddings
:253-303). Checked two ways through the C ABI: against the same library's lmh_rope followed by plain attention (the
fused rotation goes through the same arithmetic, so the two must agree bit for bit), and against the CPU oracle's rope
followed by its attention, to the contract's tolerances."""
import numpy as np
import pytest

from conftest import TOL, rel_err

pytestmark = pytest.mark.gpu

NT = 16


def out_type(dtype):
    return "f32" if dtype == "bf16" else dtype


def run(lm, hip, q, k, v, dtype, causal, rope=None, kv_len=None, pos0=None, head_map=0):
    """rope = None | (prev_seq, interleaved): attention on device copies of q, k, v; returns (result, kernel name)."""
    dq, dk, dv = (lm.to_device(x, hip, dtype) for x in (q, k, v))
    extra = []
    if kv_len is not None:
        extra.append(lm.to_device(np.asarray(kv_len, np.int32), hip))
    if pos0 is not None:
        extra.append(lm.to_device(np.asarray(pos0, np.int32), hip))
    op = lm.FlashAttentionOp(lm.default_scale(q.shape[-1]), causal, head_map, has_kv_len=kv_len is not None,
                             q_rope_base=None if rope is None else 10000.0, q_prev_seq=0 if rope is None else rope[0],
                             q_rope_interleaved=False if rope is None else rope[1], has_q_pos0=pos0 is not None)
    out = lm.HipArray(q.shape, out_type(dtype), hip)
    lm.host.execute_op_inplace(out, op, dq, dk, dv, *extra)
    return out.to_host()


def plan(lm, q, k, dtype, causal, rope):
    p = lm.binding.AttnParams()
    p.out = p.q = p.k = p.v = 4096
    p.B, p.Hq, p.Sq, p.D = q.shape
    p.Hkv, p.Sk = k.shape[1], k.shape[2]
    p.dtype = lm.binding.DTYPE_CODES[dtype]
    p.scale, p.causal, p.out_f32 = lm.default_scale(q.shape[-1]), int(causal), int(out_type(dtype) == "f32")
    if rope:
        p.q_rope, p.q_rope_base = 1, 10000.0
    return lm.binding.flash_attn_plan(p)


def rotated_on_device(lm, hip, q, dtype, prev_seq=0, interleaved=False, pos0=None):
    dq = lm.to_device(q, hip, dtype)
    d0 = None if pos0 is None else lm.to_device(np.asarray(pos0, np.int32), hip)
    return lm.apply_rotary_embeddings(dq, prev_seq=prev_seq, pos0=d0, interleaved=interleaved).to_host()


def inputs(oracle, shape_q, shape_kv, dtype, seed, mul=1.0):
    q = oracle.round_to(oracle.gen_normal(shape_q, seed, mul), dtype)
    k = oracle.round_to(oracle.gen_normal(shape_kv, seed + 1, mul), dtype)
    v = oracle.round_to(oracle.gen_normal(shape_kv, seed + 2, mul), dtype)
    return q, k, v


# (B, Hq, Hkv, Sq, Sk, D, causal, dtype, part of the kernel name the launch must reach)
CASES = [
    (1, 8, 2, 96, 96, 64, True, "f16", "prefill_mfma_kernel<f16, D=64, causal, key groups=1"),
    (1, 4, 4, 300, 300, 96, True, "f16", "prefill_mfma_kernel<f16, D=96, causal, key groups=2"),
    (2, 4, 2, 200, 333, 128, False, "bf16", "prefill_mfma_kernel<bf16, D=128, full"),
    (1, 48, 8, 2048, 2048, 96, True, "f16", "waves=8"),
    (1, 32, 8, 4096, 4096, 96, True, "f16", "prefill_mfma_pair_kernel<f16, D=96, causal>"),
    (1, 64, 64, 2000, 2000, 64, True, "f16", "prefill_mfma_pair_kernel<f16, D=64, causal>"),
    (1, 32, 8, 4096, 1100, 96, False, "f16", "prefill_mfma_pair_kernel<f16, D=96, full>"),
    (1, 64, 64, 2000, 2000, 64, True, "bf16", "prefill_mfma_kernel<bf16, D=64, causal, key groups=1"),
    (1, 32, 8, 4096, 4096, 96, True, "bf16", "prefill_mfma_kernel<bf16, D=96, causal, key groups=1, waves=8"),
    (4, 20, 20, 448, 704, 64, False, "f16", "prefill_mfma_wide_kernel<f16, D=64>"),
    (4, 20, 20, 448, 704, 96, False, "bf16", "prefill_mfma_wide_kernel<bf16, D=96>"),
    (1, 4, 2, 160, 160, 64, True, "f32", "prefill_f32_kernel<D=64, causal"),
    (1, 4, 4, 130, 200, 96, False, "f32", "prefill_f32_kernel<D=96, full"),
    (1, 16, 4, 2048, 2048, 128, True, "f32", "prefill_f32_kernel<D=128, causal, key groups=1"),
    (1, 4, 2, 70, 90, 80, True, "f16", "prefill_valu_kernel"),   # a head dim the register rotation does not take
    (1, 2, 2, 50, 50, 32, True, "f32", "prefill_valu_kernel"),
    (1, 2, 1, 40, 60, 6, False, "bf16", "prefill_valu_kernel"),
]


@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "%s-D%d-%dx%d-%s" % (c[7], c[5], c[3], c[4], "causal" if c[6] else "full"))
def test_fused_q_rope_equals_rope_then_attention(lm, hip, oracle, case, interleaved):
    B, Hq, Hkv, Sq, Sk, D, causal, dtype, kernel = case
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 12000 + D + Sq)
    name = plan(lm, q, k, dtype, causal, True)
    print("kernel:", name, flush=True)
    assert kernel in name, name
    prev = 7
    got = run(lm, hip, q, k, v, dtype, causal, rope=(prev, interleaved))
    # the same library, two launches: rotate (and round) q, then attend. Where both forms reach the same attention
    # kernel the results must be the same bits (a head dim the register rotation does not take sends the fused form to
    # the vector-ALU kernel while the plain form stays on the matrix cores: then they agree to the tolerance)
    q_rot = rotated_on_device(lm, hip, q, dtype, prev_seq=prev, interleaved=interleaved)
    two_step = run(lm, hip, q_rot, k, v, dtype, causal)
    if plan(lm, q, k, dtype, causal, False) == name:
        np.testing.assert_array_equal(got, two_step)
    else:
        assert "prefill_valu_kernel" in name
        assert rel_err(got, two_step) <= TOL[dtype]
    # the oracle: rope, round to the element type, attention
    q_ref = oracle.round_to(oracle.rope(q, prev_seq=prev, interleaved=interleaved), dtype)
    want = oracle.flash_attn(q_ref, k, v, causal=causal, nthreads=NT)
    # fp32: 1e-5 plus the spread of sin / cos between libm and the GPU at these angles (see the rope tests)
    tol = {"f32": 3e-5, "f16": 2e-3, "bf16": 3e-3}[dtype]  # a bf16 q rounds differently where the rotations differ by an ulp
    assert rel_err(got, want) <= tol
    # and the rotation is really applied: without it the result differs
    assert rel_err(run(lm, hip, q, k, v, dtype, causal), want) > 10 * tol


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_fused_q_rope_with_positions_per_sequence_and_ragged_keys(lm, hip, oracle, dtype):
    B, Hq, Hkv, Sq, Sk, D = 3, 8, 4, 100, 150, 128
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 12500)
    pos0 = np.array([0, 31, 900], np.int32)
    lens = np.array([150, 64, 1], np.int32)
    got = run(lm, hip, q, k, v, dtype, False, rope=(0, False), kv_len=lens, pos0=pos0)
    q_rot = rotated_on_device(lm, hip, q, dtype, pos0=pos0)
    np.testing.assert_array_equal(got, run(lm, hip, q_rot, k, v, dtype, False, kv_len=lens))
    q_ref = oracle.round_to(oracle.rope(q, pos0=pos0), dtype)
    want = oracle.flash_attn(q_ref, k, v, causal=False, kv_len=lens, nthreads=NT)
    assert rel_err(got, want) <= {"f32": 2e-4, "f16": 2e-3, "bf16": 3e-3}[dtype]  # fp32: angles up to 1000 rad


@pytest.mark.parametrize("dtype,D", [("f16", 96), ("bf16", 128), ("f32", 64), ("f16", 80)])
def test_self_attention_core_rotates_q_inside_the_attention_launch(lm, hip, oracle, dtype, D):
    """self_attention_core (reference src/NN.jl:352-382): one rotary node (K), one attention node that rotates Q itself;
    head dims outside the fused set keep both rotary nodes. Either way the result is rope + GQA attention."""
    B, Hq, Hkv, S = 1, 8, 2, 130
    q, k, v = inputs(oracle, (B, Hq, S, D), (B, Hkv, S, D), dtype, 12600)
    g = lm.Graph()
    tq, tk, tv = lm.tensor(g, q.shape, dtype), lm.tensor(g, k.shape, dtype), lm.tensor(g, v.shape, dtype)
    out = lm.self_attention_core(tq, tk, tv, causal=True, prev_seq=3, rope_base=10000.0, out_dtype=out_type(dtype))
    n_rope = sum(isinstance(n.op, lm.RotaryEmbeddingOp) for n in g.nodes)
    assert n_rope == (1 if D in lm.FUSED_ROPE_HEAD_DIMS else 2)
    assert (g.nodes[out.id].op.q_rope_base is not None) == (D in lm.FUSED_ROPE_HEAD_DIMS)
    got = lm.execute(g, out.id, {tq.id: q, tk.id: k, tv.id: v}, hip)
    want = oracle.flash_attn(oracle.round_to(oracle.rope(q, prev_seq=3), dtype), oracle.round_to(oracle.rope(k, prev_seq=3), dtype),
                             v, causal=True, nthreads=NT)
    assert rel_err(got, want) <= {"f32": 3e-5, "f16": 3e-3, "bf16": 4e-3}[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32"])
def test_prompt_core_fills_the_cache_and_attends_in_two_launches(lm, hip, oracle, dtype):
    """prompt_self_attention_core: append (K rotated on its way into the cache) + attention over the cache rows with
    the queries rotated inside the kernel; a compiled graph of it is two steps. The caches afterwards hold what the
    decode steps will read."""
    B, Hq, Hkv, T, D, Lmax = 2, 8, 2, 96, 128, 160
    q, kn, vn = inputs(oracle, (B, Hq, T, D), (B, Hkv, T, D), dtype, 12700)
    g = lm.Graph()
    tq, tkn, tvn = lm.tensor(g, q.shape, dtype), lm.tensor(g, kn.shape, dtype), lm.tensor(g, vn.shape, dtype)
    tkc, tvc = lm.tensor(g, (B, Hkv, Lmax, D), dtype), lm.tensor(g, (B, Hkv, Lmax, D), dtype)
    tpos, tlen = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
    out, kc, vc = lm.prompt_self_attention_core(tq, tkn, tvn, tkc, tvc, tpos, tlen, rope_base=10000.0, out_dtype=out_type(dtype))
    cg = lm.compile(g, hip)
    assert len(cg.steps) == 2
    junk = np.full((B, Hkv, Lmax, D), np.nan, np.float32)  # rows past kv_len must not matter
    res = cg({tq.id: q, tkn.id: kn, tvn.id: vn, tkc.id: junk, tvc.id: junk, tpos.id: np.zeros(B, np.int32),
              tlen.id: np.full(B, T, np.int32)})
    k_rot = oracle.round_to(oracle.rope(kn), dtype)
    want = oracle.flash_attn(oracle.round_to(oracle.rope(q), dtype), k_rot, vn, causal=True, nthreads=NT)
    assert rel_err(res[out.id].to_host(), want) <= {"f32": 3e-5, "f16": 3e-3, "bf16": 4e-3}[dtype]
    kc_host = res[kc.id][0].to_host()
    assert rel_err(kc_host[:, :, :T], k_rot) <= (2e-5 if dtype == "f32" else 8e-3)
    np.testing.assert_array_equal(res[kc.id][1].to_host()[:, :, :T], vn)
