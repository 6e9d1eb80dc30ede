"""lmh_decode_step: one decode step of a cached attention layer in two launches — the split kernel over the rows
already in the caches with q rotated as it is loaded, then the merge launch that adds the new row from k_new / v_new
and stores it (K rotated) into the caches. Checked through the C ABI against the CPU oracle (rope, cache append, decode
attention: reference src/NN.jl:253-303, src/Whisper.jl:552-570, :584-620) and against the library's own three-launch
path (lmh_kv_append + lmh_decode_attn)."""
import numpy as np
import pytest

from conftest import TOL, rel_err

pytestmark = pytest.mark.gpu

NT = 16


def step_inputs(oracle, B, Hq, Hkv, Lmax, D, dtype, seed):
    q = oracle.round_to(oracle.gen_normal((B, Hq, 1, D), seed), dtype)
    kn = oracle.round_to(oracle.gen_normal((B, Hkv, 1, D), seed + 1), dtype)
    vn = oracle.round_to(oracle.gen_normal((B, Hkv, 1, D), seed + 2), dtype)
    kc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), seed + 3), dtype)
    vc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), seed + 4), dtype)
    return q, kn, vn, kc, vc


def expected(oracle, q, kn, vn, kc, vc, pos, dtype, rope, interleaved, head_map):
    """The oracle's step: rotate q and k_new at pos[b], round, write row pos[b], attend rows 0 .. pos[b]."""
    B = q.shape[0]
    if rope:
        q = oracle.round_to(oracle.rope(q, pos0=pos, interleaved=interleaved), dtype)
        kn = oracle.round_to(oracle.rope(kn, pos0=pos, interleaved=interleaved), dtype)
    kc, vc = kc.copy(), vc.copy()
    for b in range(B):
        kc[b, :, pos[b]] = kn[b, :, 0]
        vc[b, :, pos[b]] = vn[b, :, 0]
    out = oracle.decode_attn(q[:, :, 0], kc, vc, kv_len=pos + 1, head_map=head_map, nthreads=NT)
    return out, kc, vc


def run_step(lm, hip, q, kn, vn, kc, vc, pos, dtype, rope, interleaved=False, head_map=0, num_splits=0):
    dq = lm.to_device(np.ascontiguousarray(q[:, :, 0]), hip, dtype)
    dkn, dvn, dkc, dvc = (lm.to_device(x, hip, dtype) for x in (kn, vn, kc, vc))
    dpos = lm.to_device(np.asarray(pos, np.int32), hip)
    op = lm.DecodeStepOp(lm.default_scale(q.shape[-1]), head_map, num_splits, "f32", 10000.0 if rope else None, interleaved)
    out, kc2, vc2 = lm.execute_op(op, dq, dkc, dvc, dkn, dvn, dpos)
    assert kc2 is dkc and vc2 is dvc
    np.testing.assert_array_equal(dq.to_host(), q[:, :, 0])  # q itself is left as it was
    return out.to_host(), dkc.to_host(), dvc.to_host()


CASES = [  # B, Hq, Hkv, Lmax, D, dtype, rope, interleaved, head_map
    (2, 8, 2, 700, 64, "f16", True, False, 0),
    (3, 32, 8, 3000, 128, "bf16", True, False, 0),
    (3, 32, 8, 3000, 128, "bf16", True, False, 1),
    (2, 4, 4, 900, 256, "f16", True, False, 0),
    (2, 12, 4, 1100, 96, "f16", True, True, 0),    # head dim 96: in registers only with the interleaved pairing
    (2, 12, 4, 1100, 96, "bf16", False, False, 0),  # no rotary embedding
    (1, 40, 2, 600, 128, "f16", True, False, 0),    # 20 query heads per KV head: two slices of 16
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B%d-H%d:%d-L%d-D%d-%s" % c[:6])
def test_decode_step_against_the_oracle(lm, hip, oracle, case):
    B, Hq, Hkv, Lmax, D, dtype, rope, interleaved, head_map = case
    q, kn, vn, kc, vc = step_inputs(oracle, B, Hq, Hkv, Lmax, D, dtype, 16000 + D + Lmax)
    rng = np.random.default_rng(16001)
    pos = rng.integers(1, Lmax, size=B).astype(np.int32)
    pos[0] = Lmax - 1  # the last row of a cache
    if B > 1:
        pos[1] = 0     # an empty cache: the result is v_new
    kcp, vcp = kc.copy(), vc.copy()
    for b in range(B):  # rows from pos[b] on are not part of the sequence yet: poison them
        kcp[b, :, pos[b]:] = np.nan
        vcp[b, :, pos[b]:] = np.nan
    got, kc_after, vc_after = run_step(lm, hip, q, kn, vn, kcp, vcp, pos, dtype, rope, interleaved, head_map)
    want, kc_want, vc_want = expected(oracle, q, kn, vn, kc, vc, pos, dtype, rope, interleaved, head_map)
    assert np.isfinite(got).all()
    assert rel_err(got, want) <= TOL[dtype]
    if B > 1:  # (fp32 output of exactly one row with weight 1)
        G = Hq // Hkv
        kv_of = [(h // G if head_map == 1 else h % Hkv) for h in range(Hq)]
        np.testing.assert_array_equal(got[1], vn[1, kv_of, 0])
    for b in range(B):
        # the appended row: V bit for bit, K to the rotation's rounding (one ulp of the element type where sin / cos differ)
        np.testing.assert_array_equal(vc_after[b, :, pos[b]], vn[b, :, 0])
        assert rel_err(kc_after[b, :, pos[b]], kc_want[b, :, pos[b]]) <= (8e-3 if rope else 0)
        # nothing else was touched
        np.testing.assert_array_equal(kc_after[b, :, :pos[b]], kc[b, :, :pos[b]])
        assert np.isnan(kc_after[b, :, pos[b] + 1:]).all() and np.isnan(vc_after[b, :, pos[b] + 1:]).all()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_decode_step_equals_append_then_attend(lm, hip, oracle, dtype):
    """Against the library's own three launches on the same inputs: the caches must come out bit-identical (the same
    rotation arithmetic), the result within the merge order's rounding."""
    B, Hq, Hkv, Lmax, D = 4, 32, 8, 2048, 128
    q, kn, vn, kc, vc = step_inputs(oracle, B, Hq, Hkv, Lmax, D, dtype, 16500)
    pos = np.array([5, 2047, 1000, 64], np.int32)
    got, kc1, vc1 = run_step(lm, hip, q, kn, vn, kc, vc, pos, dtype, True)
    dq = lm.to_device(q, hip, dtype)
    dkn, dvn, dkc, dvc = (lm.to_device(x, hip, dtype) for x in (kn, vn, kc, vc))
    dpos = lm.to_device(pos, hip)
    lm.kv_append(dkc, dvc, dkn, dvn, dpos, rope_k=True, q=dq)
    out = lm.execute_op(lm.DecodeAttentionOp(lm.default_scale(D), 0, 0, "f32"), dq.view((B, Hq, D)), dkc, dvc, lm.to_device(pos + 1, hip))
    np.testing.assert_array_equal(kc1, dkc.to_host())
    np.testing.assert_array_equal(vc1, dvc.to_host())
    assert rel_err(got, out.to_host()) <= 2e-6


def test_decode_step_graph_steps_through_positions(lm, hip, oracle):
    """cached_self_attention_core(fused=True) is one node; one compiled graph serves every position, and the caches it
    holds afterwards are the rotated K and the raw V of all steps (as in the two-node form)."""
    B, Hq, Hkv, S, D, Lmax, dtype = 2, 8, 2, 20, 64, 512, "f16"
    q = oracle.round_to(oracle.gen_normal((B, Hq, S, D), 16600), dtype)
    k = oracle.round_to(oracle.gen_normal((B, Hkv, S, D), 16601), dtype)
    v = oracle.round_to(oracle.gen_normal((B, Hkv, S, D), 16602), dtype)
    want = oracle.flash_attn(oracle.round_to(oracle.rope(q), dtype), oracle.round_to(oracle.rope(k), dtype), v, causal=True)
    g = lm.Graph()
    tq, tkn, tvn = lm.tensor(g, (B, Hq, 1, D), dtype), lm.tensor(g, (B, Hkv, 1, D), dtype), lm.tensor(g, (B, Hkv, 1, D), dtype)
    tkc, tvc = lm.tensor(g, (B, Hkv, Lmax, D), dtype), lm.tensor(g, (B, Hkv, Lmax, D), dtype)
    tpos, tlen = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
    out, kc2, vc2 = lm.cached_self_attention_core(tq, tkn, tvn, tkc, tvc, tpos, tlen, rope_base=10000.0, out_dtype="f32", fused=True)
    assert isinstance(g.nodes[out.id].op, lm.DecodeStepOp) and kc2.id == out.id and kc2.index == 1
    cg = lm.compile(g, hip)
    assert len(cg.steps) == 1
    for t in range(S):
        if t == 3:
            cg.capture()  # the step can be recorded like the two-node form
        res = cg({tq.id: np.ascontiguousarray(q[:, :, t:t + 1]), tkn.id: np.ascontiguousarray(k[:, :, t:t + 1]),
                  tvn.id: np.ascontiguousarray(v[:, :, t:t + 1]), tpos.id: np.full(B, t, np.int32)})
        assert rel_err(res[out.id][0].to_host(), want[:, :, t]) <= TOL[dtype], t
    cg.release()
    assert rel_err(res[out.id][1].to_host()[:, :, :S], oracle.round_to(oracle.rope(k), dtype)) <= 8e-3
    np.testing.assert_array_equal(res[out.id][2].to_host()[:, :, :S], v)


def test_decode_step_refuses_what_it_cannot_take(lm, hip, oracle):
    B, Hq, Hkv, Lmax = 1, 4, 4, 256
    for dtype, D, interleaved in (("f32", 64, False), ("f16", 96, False), ("f16", 72, False)):
        q, kn, vn, kc, vc = step_inputs(oracle, B, Hq, Hkv, Lmax, D, dtype, 16700)
        assert not lm.decode_step_supported(dtype, D, True, interleaved)
        with pytest.raises(lm.LuminalHipError) as e:
            run_step(lm, hip, q, kn, vn, kc, vc, np.array([3], np.int32), dtype, True, interleaved)
        assert e.value.code == lm.binding.LMH_E_UNSUPPORTED
    # the builder falls back to append + attend where the fused step does not apply
    g = lm.Graph()
    tq, tkn, tvn = lm.tensor(g, (B, Hq, 1, 96), "f16"), lm.tensor(g, (B, Hkv, 1, 96), "f16"), lm.tensor(g, (B, Hkv, 1, 96), "f16")
    tkc, tvc = lm.tensor(g, (B, Hkv, Lmax, 96), "f16"), lm.tensor(g, (B, Hkv, Lmax, 96), "f16")
    tpos, tlen = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
    out, _, _ = lm.cached_self_attention_core(tq, tkn, tvn, tkc, tvc, tpos, tlen, rope_base=10000.0, fused=True)
    assert isinstance(g.nodes[out.id].op, lm.DecodeAttentionOp)
