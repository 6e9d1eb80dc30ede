"""Parity of the HIP kernels (called through the C ABI) against the CPU oracle and the golden
vectors, on an MI355X. Tolerances are the contract's: max|err| / max|oracle| <= 1e-5 for fp32 and
<= 2e-3 for fp16 / bf16, with the oracle evaluated in fp32 on inputs already rounded to the
element type."""
import numpy as np
import pytest

from conftest import TOL, rel_err

pytestmark = pytest.mark.gpu

NT = 16  # oracle threads (rows are independent; results do not depend on it)


def out_type(dtype, out_dtype):
    """bf16 results are taken in fp32 unless a test asks otherwise: rounding a result to bf16 costs up
    to 2^-8 of its magnitude by itself, more than the 2e-3 budget (test_bf16_output_is_rounded_fp32
    covers the bf16-out path)."""
    if out_dtype is not None:
        return out_dtype
    return "f32" if dtype == "bf16" else dtype


def run_flash(lm, hip, q, k, v, dtype, causal, scale=None, head_map=0, kv_len=None, out_dtype=None):
    od = out_type(dtype, out_dtype)
    g = lm.Graph()
    tq, tk, tv = lm.tensor(g, q.shape, dtype), lm.tensor(g, k.shape, dtype), lm.tensor(g, v.shape, dtype)
    if kv_len is None:
        out = lm.flash_attention(tq, tk, tv, scale=scale, causal=causal, head_map=head_map, out_dtype=od)
        return lm.execute(g, out.id, {tq.id: q, tk.id: k, tv.id: v}, hip)
    # kv_len is an extension of the op: call the in-place executor directly
    dq, dk, dv = (lm.to_device(x, hip, dtype) for x in (q, k, v))
    dl = lm.to_device(np.asarray(kv_len, np.int32), hip)
    op = lm.FlashAttentionOp(lm.default_scale(q.shape[-1]) if scale is None else scale, causal, head_map)
    out = lm.HipArray(q.shape, od, hip)
    lm.host.execute_op_inplace(out, op, dq, dk, dv, dl)
    return out.to_host()


def run_decode(lm, hip, q, kc, vc, dtype, kv_len=None, scale=None, head_map=0, num_splits=0, out_dtype=None):
    dq, dk, dv = (lm.to_device(x, hip, dtype) for x in (q, kc, vc))
    dl = None if kv_len is None else lm.to_device(np.asarray(kv_len, np.int32), hip)
    op = lm.DecodeAttentionOp(lm.default_scale(q.shape[-1]) if scale is None else scale, head_map, num_splits)
    out = lm.HipArray(q.shape, out_type(dtype, out_dtype), hip)
    args = (dq, dk, dv) if dl is None else (dq, dk, dv, dl)
    lm.host.execute_op_inplace(out, op, *args)
    return out.to_host()


def inputs(oracle, shape_q, shape_kv, dtype, seed, mul=1.0):
    q = oracle.round_to(oracle.gen_normal(shape_q, seed, mul), dtype)
    k = oracle.round_to(oracle.gen_normal(shape_kv, seed + 1, mul), dtype)
    v = oracle.round_to(oracle.gen_normal(shape_kv, seed + 2, mul), dtype)
    return q, k, v


# ---------------------------------------------------------------------------------------------
# golden vectors (independent numpy float64), every element type
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_golden_vectors(lm, hip, golden, dtype):
    for name, c in golden.items():
        print("case", name, dtype, flush=True)
        if name.startswith("decode"):
            got = run_decode(lm, hip, c["q"][:, :, 0], c["k"], c["v"], dtype, kv_len=c["kv_len"], scale=c["scale"])
            want = c["out"][:, :, 0]
        else:
            got = run_flash(lm, hip, c["q"], c["k"], c["v"], dtype, c["causal"], scale=c["scale"], kv_len=c["kv_len"])
            want = c["out"]
        assert rel_err(got, want) <= TOL[dtype], (name, dtype)


def test_reference_test_shape_criterion(lm, hip, oracle):
    # the reference's own check: flash ~= manual attention at rtol 1e-4 on B=H=1, S=8, D=16
    # (reference tests/test_flash_attention_verification.jl:24-49)
    q, k, v = inputs(oracle, (1, 1, 8, 16), (1, 1, 8, 16), "f32", 100)
    for causal in (False, True):
        got = run_flash(lm, hip, q, k, v, "f32", causal)
        np.testing.assert_allclose(got, oracle.naive_attention_np(q, k, v, causal=causal), rtol=1e-4, atol=1e-6)
        assert rel_err(got, oracle.flash_attn(q, k, v, causal=causal)) <= 1e-5


# ---------------------------------------------------------------------------------------------
# the five benchmark configurations at full size
# ---------------------------------------------------------------------------------------------
def test_config1_llama_example_fp32_causal(lm, hip, oracle):
    q, k, v = inputs(oracle, (1, 8, 128, 64), (1, 8, 128, 64), "f32", 1000)
    got = run_flash(lm, hip, q, k, v, "f32", True, scale=0.125)
    assert rel_err(got, oracle.flash_attn(q, k, v, scale=0.125, causal=True)) <= 1e-5
    np.testing.assert_array_equal(got[:, :, 0], v[:, :, 0])  # first causal row is V[0] exactly


def test_config2_phi3_prefill_fp16_causal_d96(lm, hip, oracle):
    shape = (1, 32, 4096, 96)
    q, k, v = inputs(oracle, shape, shape, "f16", 2000, mul=0.5)
    got = run_flash(lm, hip, q, k, v, "f16", True)
    want = oracle.flash_attn(q, k, v, causal=True, nthreads=NT)
    assert rel_err(got, want) <= 2e-3


def test_config3_whisper_cross_attention_fp16(lm, hip, oracle):
    q, k, v = inputs(oracle, (4, 20, 448, 64), (4, 20, 1500, 64), "f16", 3000)
    got = run_flash(lm, hip, q, k, v, "f16", False)
    want = oracle.flash_attn(q, k, v, causal=False, nthreads=NT)
    assert rel_err(got, want) <= 2e-3


@pytest.mark.parametrize("head_map", [0, 1])
def test_config4_llama_gqa_decode_bf16(lm, hip, oracle, head_map):
    B, Hq, Hkv, L, D = 16, 32, 8, 4096, 128
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), "bf16", 4000)
    lens = np.full(B, L, np.int32)
    got = run_decode(lm, hip, q, k, v, "bf16", kv_len=lens, head_map=head_map)
    want = oracle.decode_attn(q, k, v, kv_len=lens, head_map=head_map, nthreads=NT)
    assert rel_err(got, want) <= 2e-3
    # the two head maps are different functions of the same inputs
    other = oracle.decode_attn(q, k, v, kv_len=lens, head_map=1 - head_map, nthreads=NT)
    assert rel_err(got, other) > 1e-2


def test_config5_long_ragged_gqa_decode_bf16(lm, hip, oracle):
    """B=64, Hq=32, Hkv=8, D=128, kv_len ~ U[8192, 32768]; the cache tail past kv_len[b] is NaN."""
    B, Hq, Hkv, Lmax, D = 64, 32, 8, 32768, 128
    lens = oracle.gen_uniform_int(B, 5000, 8192, 32768)
    q = oracle.round_to(oracle.gen_normal((B, Hq, D), 5001), "bf16")
    dk = lm.HipArray((B, Hkv, Lmax, D), "bf16", hip).fill_bytes(0xFF)  # 0xFFFF = NaN
    dv = lm.HipArray((B, Hkv, Lmax, D), "bf16", hip).fill_bytes(0xFF)
    want = np.empty((B, Hq, D), np.float32)
    row_bytes = D * 2
    for b in range(B):
        n = int(lens[b])
        kb = oracle.round_to(oracle.gen_normal((1, Hkv, n, D), 6000 + 2 * b), "bf16")
        vb = oracle.round_to(oracle.gen_normal((1, Hkv, n, D), 6001 + 2 * b), "bf16")
        want[b] = oracle.decode_attn(q[b:b + 1], kb, vb, nthreads=NT)[0]
        kbits, vbits = lm.encode(kb, "bf16"), lm.encode(vb, "bf16")
        for h in range(Hkv):
            off = ((b * Hkv + h) * Lmax) * row_bytes
            lm.binding.memcpy_h2d(dk.ptr + off, kbits[0, h].ctypes.data, n * row_bytes)
            lm.binding.memcpy_h2d(dv.ptr + off, vbits[0, h].ctypes.data, n * row_bytes)
    dq = lm.to_device(q, hip, "bf16")
    dl = lm.to_device(lens, hip)
    results = {}
    for splits in (0, 8, 57):
        out = lm.HipArray((B, Hq, D), "f32", hip)
        lm.host.execute_op_inplace(out, lm.DecodeAttentionOp(lm.default_scale(D), 0, splits), dq, dk, dv, dl)
        results[splits] = out.to_host()
        assert rel_err(results[splits], want) <= 2e-3, splits
    # split-count invariance (log-sum-exp merge identity): same answer up to fp32 reassociation
    assert rel_err(results[8], results[0]) <= 1e-5
    assert rel_err(results[57], results[0]) <= 1e-5


# ---------------------------------------------------------------------------------------------
# shape / feature sweeps
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("D", [16, 24, 32, 64, 80, 96, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_fp32_head_dims(lm, hip, oracle, D, causal):
    q, k, v = inputs(oracle, (2, 3, 70, D), (2, 3, 70, D), "f32", 7000 + D)
    assert rel_err(run_flash(lm, hip, q, k, v, "f32", causal), oracle.flash_attn(q, k, v, causal=causal)) <= 1e-5


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("D", [136, 160, 192, 256])
def test_head_dims_above_128_run_on_the_vector_kernel(lm, hip, oracle, dtype, D):
    # decode accepts head dims up to 256; prefill does too (a model with D = 256 must be able to do both)
    q, k, v = inputs(oracle, (2, 4, 70, D), (2, 2, 90, D), dtype, 7150 + D)
    lens = np.array([90, 41], np.int32)
    for causal in (False, True):
        got = run_flash(lm, hip, q, k, v, dtype, causal, kv_len=lens)
        assert rel_err(got, oracle.flash_attn(q, k, v, causal=causal, kv_len=lens)) <= TOL[dtype]


@pytest.mark.parametrize("Sq,Sk", [(1, 1), (1, 77), (7, 7), (64, 64), (65, 130), (130, 65), (257, 300)])
@pytest.mark.parametrize("causal", [False, True])
def test_fp32_sequence_shapes(lm, hip, oracle, Sq, Sk, causal):
    q, k, v = inputs(oracle, (1, 2, Sq, 64), (1, 2, Sk, 64), "f32", 7100 + Sq)
    assert rel_err(run_flash(lm, hip, q, k, v, "f32", causal), oracle.flash_attn(q, k, v, causal=causal)) <= 1e-5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("D", [64, 96, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (1, 200), (64, 64), (127, 127), (128, 128), (129, 129), (300, 1000), (1000, 300), (513, 513)])
def test_mfma_shapes(lm, hip, oracle, dtype, D, causal, Sq, Sk):
    q, k, v = inputs(oracle, (2, 3, Sq, D), (2, 3, Sk, D), dtype, 7200 + Sq + D)
    got = run_flash(lm, hip, q, k, v, dtype, causal)
    assert rel_err(got, oracle.flash_attn(q, k, v, causal=causal, nthreads=NT)) <= 2e-3


@pytest.mark.parametrize("D", [64, 96, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("Sq,Sk", [(1, 1), (1, 200), (31, 33), (64, 64), (127, 127), (128, 128), (129, 129), (300, 1000), (1000, 300), (513, 513)])
def test_fp32_mfma_shapes(lm, hip, oracle, D, causal, Sq, Sk):
    # the fp32 matrix-core kernel (head dims 64 / 96 / 128) at the fp32 budget
    q, k, v = inputs(oracle, (2, 3, Sq, D), (2, 3, Sk, D), "f32", 7300 + Sq + D)
    got = run_flash(lm, hip, q, k, v, "f32", causal)
    assert rel_err(got, oracle.flash_attn(q, k, v, causal=causal, nthreads=NT)) <= 1e-5


def test_fp32_large_logits_and_late_maximum(lm, hip, oracle):
    # scores far apart (scale 1, |q.k| up to ~60) and a maximum that arrives in the last tile exercise the
    # lazily raised running max of the fp32 kernel; the oracle follows the reference's exact recurrence
    B, H, S, D = 1, 2, 200, 64
    q, k, v = inputs(oracle, (B, H, S, D), (B, H, S, D), "f32", 7400)
    k[:, :, -1] *= 6.0
    for causal in (False, True):
        got = run_flash(lm, hip, q, k, v, "f32", causal, scale=1.0)
        assert rel_err(got, oracle.flash_attn(q, k, v, scale=1.0, causal=causal)) <= 1e-5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("H,S", [(2, 200), (2, 700), (160, 520)])  # 128-row, key-split, and 128-row workgroups in a full launch
def test_half_large_logits_and_late_maximum(lm, hip, oracle, dtype, H, S):
    # as above for the half-precision kernels: P is held against a stale max until a row outgrows it by 2^8
    q, k, v = inputs(oracle, (1, H, S, 64), (1, H, S, 64), dtype, 7410)
    k[:, :, -1] = oracle.round_to(k[:, :, -1] * 6.0, dtype)
    k[:, :, S // 2] = oracle.round_to(k[:, :, S // 2] * 3.0, dtype)
    for causal in (False, True):
        got = run_flash(lm, hip, q, k, v, dtype, causal, scale=1.0)
        assert rel_err(got, oracle.flash_attn(q, k, v, scale=1.0, causal=causal, nthreads=NT)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("head_map", [0, 1])
def test_gqa_prefill_both_head_maps(lm, hip, oracle, dtype, head_map):
    q, k, v = inputs(oracle, (2, 8, 150, 64), (2, 2, 150, 64), dtype, 7300)
    got = run_flash(lm, hip, q, k, v, dtype, True, head_map=head_map)
    assert rel_err(got, oracle.flash_attn(q, k, v, causal=True, head_map=head_map, nthreads=NT)) <= TOL[dtype]
    assert rel_err(got, oracle.flash_attn(q, k, v, causal=True, head_map=1 - head_map, nthreads=NT)) > 1e-2


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_prefill_ragged_kv_len_with_poisoned_tail(lm, hip, oracle, dtype):
    B, H, Sq, Sk, D = 3, 2, 40, 200, 64
    q, k, v = inputs(oracle, (B, H, Sq, D), (B, H, Sk, D), dtype, 7400)
    lens = np.array([200, 65, 1], np.int32)
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.nan
    got = run_flash(lm, hip, q, kp, vp, dtype, False, kv_len=lens)
    assert rel_err(got, oracle.flash_attn(q, k, v, kv_len=lens)) <= TOL[dtype]


@pytest.mark.parametrize("dtype,D", [("f32", 64), ("f16", 64), ("bf16", 96), ("f16", 80), ("f32", 40)])
def test_prefill_sequence_without_keys_is_written_as_zeros(lm, hip, oracle, dtype, D):
    # kv_len[b] == 0 does not occur in the reference (its 0/0 would be NaN); every kernel writes zeros for it
    B, H, Sq, Sk = 3, 2, 70, 130
    q, k, v = inputs(oracle, (B, H, Sq, D), (B, H, Sk, D), dtype, 7450)
    lens = np.array([130, 0, 5], np.int32)
    got = run_flash(lm, hip, q, k, v, dtype, False, kv_len=lens)
    want = oracle.flash_attn(q, k, v, kv_len=np.array([130, 1, 5], np.int32))
    assert np.all(got[1] == 0)
    keep = [0, 2]
    assert rel_err(got[keep], want[keep]) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("D", [64, 96, 128])
@pytest.mark.parametrize("causal", [False, True])
def test_prefill_small_launch_splits_keys_between_wave_pairs(lm, hip, oracle, dtype, D, causal):
    # few workgroups and >= 256 keys: 64-row workgroups whose wave pairs take alternate 32-key blocks and are
    # merged at the end. Lengths put the last key in the first block, the second block, on a block edge, and nowhere.
    B, Hq, Hkv, Sq, Sk = 7, 4, 2, 150, 700
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 7470 + D)
    lens = np.array([700, 20, 33, 64, 97, 0, 641], np.int32)
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.nan
    got = run_flash(lm, hip, q, kp, vp, dtype, causal, kv_len=lens)
    want = oracle.flash_attn(q, k, v, causal=causal, kv_len=np.maximum(lens, 1), nthreads=NT)
    assert np.all(got[5] == 0)
    keep = [0, 1, 2, 3, 4, 6]
    assert rel_err(got[keep], want[keep]) <= TOL[dtype]


WIDE_CASES = [
    # dtype, out dtype, B, Hq, Hkv, Sq, Sk, D, head_map, kv_len (None = all keys)
    ("bf16", "f32", 2, 20, 10, 430, 777, 64, 0, None),       # 6 workgroups per head: 3, 3, 2, 2, 2, 2 row blocks, the last one ragged
    ("f16", "f32", 16, 8, 8, 190, 1000, 96, 0, [1000, 0, 1, 31, 32, 33, 95, 96, 97, 640, 999, 128, 129, 500, 767, 768]),
    ("bf16", "bf16", 1, 256, 256, 96, 700, 80, 0, None),     # one workgroup per head, head dim padded to 96
    ("f16", "f16", 4, 20, 20, 448, 1500, 64, 0, [1500, 1499, 97, 0]),  # 5 row blocks on 16 waves: two split two ways, three split four ways
    ("f16", "f32", 2, 24, 6, 448, 900, 64, 1, [900, 650]),   # blocked GQA map; 3, 3, 3, 3, 2 row blocks
    ("bf16", "f32", 4, 20, 4, 448, 1500, 96, 0, None),
    ("f16", "f32", 2, 32, 32, 576, 1200, 64, 0, None),       # 5, 5, 4, 4 row blocks: four key groups each where there are 4
    ("f16", "f16", 1, 40, 8, 440, 800, 40, 0, [799]),        # head dim 40 on the D = 64 tiling
    ("f16", "f32", 4, 20, 20, 672, 1500, 64, 0, [1500, 1499, 97, 0]),  # 7 row blocks: six split two ways, one four ways
    ("bf16", "f32", 2, 40, 10, 650, 900, 96, 1, [900, 129]),  # 7, 7, 7 row blocks, the last ragged; 128-key tiles end inside the keys
]


@pytest.mark.parametrize("dtype,out_dtype,B,Hq,Hkv,Sq,Sk,D,head_map,lens", WIDE_CASES)
def test_prefill_one_wide_workgroup_per_cu(lm, hip, oracle, dtype, out_dtype, B, Hq, Hkv, Sq, Sk, D, head_map, lens):
    """Non-causal launches with fewer 64-row workgroups than fill the chip evenly: one workgroup per CU of up to 8 row
    blocks x up to 6 key groups, partial results folded through LDS. Ragged kv_len with a poisoned tail (lengths on
    and around block and tile edges, 0 and 1), GQA under both head maps, query counts that end inside a block."""
    assert "prefill_mfma_wide_kernel" in lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, False)
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 7480 + D + B, 0.8)
    kp, vp = k.copy(), v.copy()
    if lens is not None:
        lens = np.array(lens, np.int32)
        for b, n in enumerate(lens):
            kp[b, :, n:] = np.nan
            vp[b, :, n:] = np.nan
    got = run_flash(lm, hip, q, kp, vp, dtype, False, head_map=head_map, kv_len=lens, out_dtype=out_dtype)
    tol = TOL[dtype] + (2.0 ** -8 if out_dtype == "bf16" else 0.0)  # a bf16 result carries its own rounding
    hq = np.arange(0, Hq, max(1, Hq // 8))  # a spread of heads keeps the CPU oracle at a few seconds
    if Hq == Hkv:
        kv_of = hq
    else:
        kv_of = hq // (Hq // Hkv) if head_map == 1 else hq % Hkv
    want_len = None if lens is None else np.maximum(lens, 1)
    want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=False, kv_len=want_len, nthreads=NT)
    keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
    assert np.isfinite(got).all()
    assert rel_err(got[keep][:, hq], want[keep]) <= tol
    if lens is not None:
        for b in np.nonzero(lens == 0)[0]:
            assert np.all(got[b] == 0)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_prefill_wide_workgroups_large_logits_and_late_maximum(lm, hip, oracle, dtype):
    # the key groups of a row block hold different running maxima (scale 1, one key x 6 in the last tile, one x 3 in the
    # middle) when they are folded
    B, H, Sq, Sk, D = 1, 40, 448, 700, 64
    assert "prefill_mfma_wide_kernel" in lm.flash_attention_plan((B, H, Sq, D), (B, H, Sk, D), dtype, False)
    q, k, v = inputs(oracle, (B, H, Sq, D), (B, H, Sk, D), dtype, 7495)
    k[:, :, -1] = oracle.round_to(k[:, :, -1] * 6.0, dtype)
    k[:, :, Sk // 2] = oracle.round_to(k[:, :, Sk // 2] * 3.0, dtype)
    got = run_flash(lm, hip, q, k, v, dtype, False, scale=1.0)
    hs = np.arange(0, H, 5)
    want = oracle.flash_attn(q[:, hs], k[:, hs], v[:, hs], scale=1.0, causal=False, nthreads=NT)
    assert rel_err(got[:, hs], want) <= TOL[dtype]


@pytest.mark.parametrize("causal", [False, True])
def test_prefill_small_and_large_launches_agree(lm, hip, oracle, causal):
    # the same two heads alone (key-split workgroups) and as part of a launch that fills the chip (128-row workgroups)
    S, D = 512, 96
    q, k, v = inputs(oracle, (1, 160, S, D), (1, 160, S, D), "f16", 7490, 0.5)
    small = run_flash(lm, hip, q[:, :2], k[:, :2], v[:, :2], "f16", causal, out_dtype="f32")
    large = run_flash(lm, hip, q, k, v, "f16", causal, out_dtype="f32")
    want = oracle.flash_attn(q[:, :2], k[:, :2], v[:, :2], causal=causal, nthreads=NT)
    assert rel_err(small, want) <= TOL["f16"]
    assert rel_err(large[:, :2], want) <= TOL["f16"]
    assert rel_err(small, large[:, :2]) <= TOL["f16"]


@pytest.mark.parametrize("dtype,D,causal,B", [("f16", 96, False, 2), ("f16", 96, True, 4), ("bf16", 64, True, 4),
                                              ("f16", 64, False, 2), ("bf16", 96, False, 2), ("f16", 80, True, 4),
                                              ("bf16", 40, False, 2), ("f16", 128, False, 2), ("f16", 128, True, 4),
                                              ("f16", 112, True, 4),
                                              # causal, 512 workgroups = two rounds of one per CU: 128-key tiles at D = 96
                                              ("f16", 96, True, 2), ("bf16", 96, True, 2), ("f16", 88, True, 2)])
def test_prefill_large_launch_runs_256_row_workgroups(lm, hip, oracle, dtype, D, causal, B):
    """From 512 (non-causal) / 1024 (causal) workgroups of 256 query rows on, eight waves share every staged K/V tile
    (fp16 and bf16 at head dims up to 96, fp16 above). GQA, ragged kv_len with a poisoned tail, a query count that is no multiple of 256; every
    eighth head is checked against the oracle, and two heads against the same heads launched alone (key-split
    128-row workgroups)."""
    Hq, Hkv = (32, 16) if causal else (32, 8)
    Sq, Sk = (2048 - 37, 2048 - 37) if causal else (2048 - 200, 1500)
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 7500 + D, 0.7)
    lens = np.array([Sk, Sk - 63, 1, Sk - 700][:B], np.int32)
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.nan
    got = run_flash(lm, hip, q, kp, vp, dtype, causal, kv_len=lens, out_dtype="f32")
    assert np.isfinite(got).all()
    hq = np.arange(0, Hq, 8)
    want = oracle.flash_attn(q[:, hq], k[:, hq % Hkv], v[:, hq % Hkv], causal=causal, kv_len=lens, nthreads=NT)
    assert rel_err(got[:, hq], want) <= TOL[dtype]
    alone = run_flash(lm, hip, q[:1, :2], kp[:1, :2], vp[:1, :2], dtype, causal, kv_len=lens[:1], out_dtype="f32")
    assert rel_err(alone, got[:1, :2]) <= TOL[dtype]


@pytest.mark.parametrize("dtype,D", [("f16", 96), ("bf16", 96), ("f16", 64), ("f16", 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_prefill_many_heads_few_queries_on_256_row_workgroups(lm, hip, oracle, dtype, D, causal):
    """512 (b, head) pairs with 150 queries each: the launch is large enough for the eight-wave workgroups, three of
    whose waves then own no query at all (they still stage tiles and meet the barriers); keys end inside a tile."""
    B, H, Sq, Sk = 8, 64, 150, 300
    q, k, v = inputs(oracle, (B, H, Sq, D), (B, H, Sk, D), dtype, 7600 + D, 0.8)
    got = run_flash(lm, hip, q, k, v, dtype, causal, out_dtype="f32")
    assert np.isfinite(got).all()
    hs = np.arange(0, H, 16)
    want = oracle.flash_attn(q[:, hs], k[:, hs], v[:, hs], causal=causal, nthreads=NT)
    assert rel_err(got[:, hs], want) <= TOL[dtype]


@pytest.mark.parametrize("D", [64, 96, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("B", [1, 9])  # 4 heads: 8 or 72 workgroups of 128 rows -> four-way (D = 64) / two-way key split
def test_fp32_tiny_launch_splits_keys_between_waves(lm, hip, oracle, D, causal, B):
    Hq, Hkv, Sq, Sk = 4, 2, 100, 300
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), "f32", 7480 + D)
    lens = np.array(([300, 20, 33, 64, 97, 0, 129, 256, 290])[:B], np.int32)
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.nan
    got = run_flash(lm, hip, q, kp, vp, "f32", causal, kv_len=lens)
    want = oracle.flash_attn(q, k, v, causal=causal, kv_len=np.maximum(lens, 1), nthreads=NT)
    keep = [b for b in range(B) if lens[b] > 0]
    for b in range(B):
        if lens[b] == 0:
            assert np.all(got[b] == 0)
    assert rel_err(got[keep], want[keep]) <= TOL["f32"]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("D", [8, 40, 72, 80, 104, 120])
@pytest.mark.parametrize("Sq,Sk", [(70, 70), (200, 700)])  # the second takes the key-split workgroups
def test_head_dims_between_the_tilings_run_padded_on_the_matrix_cores(lm, hip, oracle, dtype, D, Sq, Sk):
    q, k, v = inputs(oracle, (2, 4, Sq, D), (2, 2, Sk, D), dtype, 7460 + D)
    lens = np.array([Sk, Sk // 3], np.int32)
    kp, vp = k.copy(), v.copy()
    kp[1, :, lens[1]:] = np.nan
    vp[1, :, lens[1]:] = np.nan
    for causal in (False, True):
        got = run_flash(lm, hip, q, kp, vp, dtype, causal, kv_len=lens)
        assert rel_err(got, oracle.flash_attn(q, k, v, causal=causal, kv_len=lens, nthreads=NT)) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_unusual_head_dim_and_scale_take_the_vector_path(lm, hip, oracle, dtype):
    q, k, v = inputs(oracle, (1, 2, 90, 20), (1, 2, 90, 20), dtype, 7500)  # not a multiple of 8
    assert rel_err(run_flash(lm, hip, q, k, v, dtype, True), oracle.flash_attn(q, k, v, causal=True)) <= 2e-3
    q, k, v = inputs(oracle, (1, 2, 90, 64), (1, 2, 90, 64), dtype, 7501)
    for scale in (-0.2, 0.0):
        assert rel_err(run_flash(lm, hip, q, k, v, dtype, True, scale=scale),
                       oracle.flash_attn(q, k, v, causal=True, scale=scale)) <= 2e-3


def test_whisper_split_scale_equals_single_scale(lm, hip, oracle):
    # Whisper multiplies q and k by D^-0.25 each (reference src/Whisper.jl:305-307); the fused op takes
    # unscaled q, k and scale = 1/sqrt(D). Same function up to fp32 rounding.
    q, k, v = inputs(oracle, (1, 4, 30, 64), (1, 4, 100, 64), "f32", 7600)
    s = np.float32(64) ** np.float32(-0.25)
    split = run_flash(lm, hip, q * s, k * s, v, "f32", False, scale=1.0)
    fused = run_flash(lm, hip, q, k, v, "f32", False)
    assert rel_err(split, fused) <= 1e-5


@pytest.mark.parametrize("dtype,D", [("f32", 64), ("f32", 128), ("f16", 64), ("f16", 96), ("bf16", 128), ("bf16", 256), ("f16", 8)])
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 4), (8, 2), (8, 1), (12, 2), (16, 1)])
def test_decode_group_sizes_and_dims(lm, hip, oracle, dtype, D, Hq, Hkv):
    B, L = 3, 333
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), dtype, 7700 + D + Hq)
    lens = np.array([333, 100, 1], np.int32)
    for hm in (0, 1):
        for splits in (1, 3):
            got = run_decode(lm, hip, q, k, v, dtype, kv_len=lens, head_map=hm, num_splits=splits)
            want = oracle.decode_attn(q, k, v, kv_len=lens, head_map=hm)
            assert rel_err(got, want) <= TOL[dtype], (hm, splits)


def test_decode_equals_last_row_of_causal_prefill_on_gpu(lm, hip, oracle):
    B, Hq, Hkv, L, D = 2, 8, 2, 257, 128
    q, k, v = inputs(oracle, (B, Hq, L, D), (B, Hkv, L, D), "bf16", 7800)
    full = run_flash(lm, hip, q, k, v, "bf16", True)
    dec = run_decode(lm, hip, np.ascontiguousarray(q[:, :, L - 1]), k, v, "bf16")
    assert rel_err(dec, full[:, :, L - 1]) <= 4e-3  # two results, each within 2e-3 of the oracle


def test_decode_alternating_batches_on_one_workspace_repeat_bitwise(lm, hip, oracle):
    """Two different ragged batches alternate on the one split-KV workspace, 12 times each: a merge that picked
    up a partial of the other batch (one call earlier) or an unset slot would not reproduce the first result bit
    for bit."""
    B, Hq, Hkv, L, D = 24, 32, 8, 2048, 128
    lens = (np.arange(B) * 83 % L + 1).astype(np.int32)  # 1 .. L, ragged
    sets = []
    for seed in (9700, 9710):
        q = oracle.round_to(oracle.gen_normal((B, Hq, D), seed), "bf16")
        kc = oracle.round_to(oracle.gen_normal((B, Hkv, L, D), seed + 1), "bf16")
        vc = oracle.round_to(oracle.gen_normal((B, Hkv, L, D), seed + 2), "bf16")
        want = oracle.decode_attn(q, kc, vc, kv_len=lens, nthreads=NT)
        sets.append((tuple(lm.to_device(x, hip, "bf16") for x in (q, kc, vc)), want))
    dl = lm.to_device(lens, hip)
    op = lm.DecodeAttentionOp(lm.default_scale(D), 0, 16)  # 16 splits of 128 keys
    first = [None, None]
    for rep in range(12):
        for i, ((dq, dk, dv), want) in enumerate(sets):
            out = lm.HipArray((B, Hq, D), "f32", hip)
            lm.host.execute_op_inplace(out, op, dq, dk, dv, dl)
            got = out.to_host()
            if first[i] is None:
                first[i] = got
                assert rel_err(got, want) <= TOL["bf16"]
            else:
                assert np.array_equal(got, first[i]), (rep, i)


def test_decode_without_kv_len_and_poisoned_tail(lm, hip, oracle):
    B, Hq, Hkv, L, D = 2, 8, 2, 1000, 128
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), "bf16", 7900)
    assert rel_err(run_decode(lm, hip, q, k, v, "bf16"), oracle.decode_attn(q, k, v)) <= 2e-3
    lens = np.array([999, 130], np.int32)
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.nan
    for splits in (0, 1, 5):
        got = run_decode(lm, hip, q, kp, vp, "bf16", kv_len=lens, num_splits=splits)
        assert rel_err(got, oracle.decode_attn(q, k, v, kv_len=lens)) <= 2e-3


@pytest.mark.parametrize("dtype,D,out_dtype", [("bf16", 128, "f32"), ("f16", 64, "f16"), ("f32", 64, "f32"), ("bf16", 72, "bf16")])
@pytest.mark.parametrize("splits", [1, 0, 3])
def test_decode_sequence_without_keys_is_written_as_zeros(lm, hip, oracle, dtype, D, out_dtype, splits):
    # kv_len[b] == 0 (a fresh cache) does not occur in the reference; like every prefill kernel, every decode path
    # (matrix-core and vector kernel, with and without a merge pass) writes zeros for it instead of leaving the rows unset
    B, Hq, Hkv, L = 4, 8, 2, 600
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), dtype, 7950 + D)
    lens = np.array([600, 0, 37, 0], np.int32)
    dq, dk, dv = (lm.to_device(x, hip, dtype) for x in (q, k, v))
    out = lm.HipArray((B, Hq, D), out_dtype, hip).fill_bytes(0xFF)  # NaN bit patterns: unwritten rows would show
    op = lm.DecodeAttentionOp(lm.default_scale(D), 0, splits)
    lm.host.execute_op_inplace(out, op, dq, dk, dv, lm.to_device(lens, hip))
    got = out.to_host()
    assert np.all(got[[1, 3]] == 0)
    want = oracle.decode_attn(q, k, v, kv_len=np.maximum(lens, 1))
    assert rel_err(got[[0, 2]], want[[0, 2]]) <= (8e-3 if out_dtype == "bf16" else TOL[dtype])


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_half_output_is_the_rounded_fp32_output(lm, hip, oracle, dtype):
    """out_f32 = 0 writes the same result rounded once to the input element type. The two code paths
    may differ in the last fp32 bit (the compiler schedules the final multiply separately), which
    moves a value across a rounding boundary now and then: allow one unit in the last place on a
    tiny fraction of the elements."""
    ulp = 2.0 ** -10 if dtype == "f16" else 2.0 ** -7

    def check(narrow, wide):
        want = oracle.round_to(wide, dtype)
        assert np.mean(narrow != want) < 1e-3
        assert np.all(np.abs(narrow - want) <= ulp * np.maximum(np.abs(want), 2.0 ** -14))

    q, k, v = inputs(oracle, (1, 4, 200, 128), (1, 4, 200, 128), dtype, 8500)
    check(run_flash(lm, hip, q, k, v, dtype, True, out_dtype=dtype), run_flash(lm, hip, q, k, v, dtype, True, out_dtype="f32"))
    qd, kd, vd = inputs(oracle, (3, 8, 128), (3, 2, 900, 128), dtype, 8600)
    for splits in (1, 4):
        check(run_decode(lm, hip, qd, kd, vd, dtype, num_splits=splits, out_dtype=dtype),
              run_decode(lm, hip, qd, kd, vd, dtype, num_splits=splits, out_dtype="f32"))


def test_strided_tensors(lm, hip, oracle):
    # K and V interleaved in one [B, H, S, 2, D] buffer: row stride 2*D, exercised through explicit strides
    B, H, S, D = 2, 4, 100, 64
    q, k, v = inputs(oracle, (B, H, S, D), (B, H, S, D), "f16", 8000)
    kv = np.stack([k, v], axis=3)  # [B,H,S,2,D]
    dkv = lm.to_device(kv, hip, "f16")
    dq = lm.to_device(q, hip, "f16")
    out = lm.HipArray(q.shape, "f16", hip)
    p = lm.binding.AttnParams()
    p.out, p.q, p.k, p.v = out.ptr, dq.ptr, dkv.ptr, dkv.ptr + D * 2
    p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D = B, H, H, S, S, D
    for arr in (p.k_stride, p.v_stride):
        arr[0], arr[1], arr[2] = H * S * 2 * D, S * 2 * D, 2 * D
    p.dtype, p.scale, p.causal, p.head_map = lm.binding.LMH_F16, lm.default_scale(D), 1, 0
    lm.binding.flash_attn_fwd(p)
    assert rel_err(out.to_host(), oracle.flash_attn(q, k, v, causal=True)) <= 2e-3


def test_strided_tensors_on_the_wide_workgroups(lm, hip, oracle):
    # cross attention over K and V interleaved in one [B, H, Sk, 2, D] buffer, Q and the output as [B, Sq, H, D]
    # (head stride D, row stride H*D): every stride differs from the contiguous one
    B, H, Sq, Sk, D = 2, 20, 448, 800, 64
    q, k, v = inputs(oracle, (B, H, Sq, D), (B, H, Sk, D), "f16", 8100)
    dkv = lm.to_device(np.stack([k, v], axis=3), hip, "f16")
    dq = lm.to_device(np.ascontiguousarray(q.transpose(0, 2, 1, 3)), hip, "f16")  # [B, Sq, H, D]
    out = lm.HipArray((B, Sq, H, D), "f16", hip)
    p = lm.binding.AttnParams()
    p.out, p.q, p.k, p.v = out.ptr, dq.ptr, dkv.ptr, dkv.ptr + D * 2
    p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D = B, H, H, Sq, Sk, D
    for arr in (p.k_stride, p.v_stride):
        arr[0], arr[1], arr[2] = H * Sk * 2 * D, Sk * 2 * D, 2 * D
    for arr in (p.q_stride, p.o_stride):
        arr[0], arr[1], arr[2] = Sq * H * D, D, H * D
    p.dtype, p.scale, p.causal, p.head_map = lm.binding.LMH_F16, lm.default_scale(D), 0, 0
    assert "prefill_mfma_wide_kernel" in lm.binding.flash_attn_plan(p)
    lm.binding.flash_attn_fwd(p)
    got = out.to_host().transpose(0, 2, 1, 3)
    assert rel_err(got, oracle.flash_attn(q, k, v, causal=False, nthreads=NT)) <= 2e-3


def test_compiled_graph_reuses_buffers(lm, hip, oracle):
    # compile() pre-allocates one buffer per node and runs in place (reference src/Compiler.jl:218-255)
    B, H, S, D = 1, 4, 96, 64
    g = lm.Graph()
    tq, tk, tv = (lm.tensor(g, (B, H, S, D), "f16") for _ in range(3))
    out = lm.flash_attention(tq, tk, tv, causal=True)
    cg = lm.compile(g, hip)
    ptr_before = cg.results[out.id].ptr
    for seed in (8100, 8200):
        q, k, v = inputs(oracle, (B, H, S, D), (B, H, S, D), "f16", seed)
        res = cg({tq.id: q, tk.id: k, tv.id: v}, hip)
        assert rel_err(lm.from_device(res[out.id]), oracle.flash_attn(q, k, v, causal=True)) <= 2e-3
    assert cg.results[out.id].ptr == ptr_before


def test_rerun_is_bitwise_deterministic(lm, hip, oracle):
    q, k, v = inputs(oracle, (1, 4, 500, 96), (1, 4, 500, 96), "f16", 8300)
    a = run_flash(lm, hip, q, k, v, "f16", True)
    b = run_flash(lm, hip, q, k, v, "f16", True)
    np.testing.assert_array_equal(a, b)
    qd, kd, vd = inputs(oracle, (4, 8, 128), (4, 2, 3000, 128), "bf16", 8400)
    np.testing.assert_array_equal(run_decode(lm, hip, qd, kd, vd, "bf16"), run_decode(lm, hip, qd, kd, vd, "bf16"))


# ---------------------------------------------------------------------------------------------
# rotary embedding and KV-cache append
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("D", [64, 96, 20])  # 20: no 16-byte chunks, one element per thread
def test_rope(lm, hip, oracle, dtype, interleaved, D):
    B, H, S = 2, 3, 37
    x = oracle.round_to(oracle.gen_normal((B, H, S, D), 9000), dtype)
    dx = lm.to_device(x, hip, dtype)
    got = lm.apply_rotary_embeddings(dx, prev_seq=100, interleaved=interleaved).to_host()
    want = oracle.round_to(oracle.rope(x, prev_seq=100, interleaved=interleaved), dtype)
    # fp32: 1e-5 of the output range plus the spread of sin/cos at ~100 rad between libm and the GPU
    tol = {"f32": 2e-5, "f16": 2e-3, "bf16": 8e-3}[dtype]  # bf16 output rounding alone is up to 2^-8
    assert rel_err(got, want) <= tol
    # per-sequence positions, in place
    pos0 = np.array([5, 2000], np.int32)
    lm.apply_rotary_embeddings(dx, pos0=lm.to_device(pos0, hip), out=dx, interleaved=interleaved)
    want = oracle.round_to(oracle.rope(x, pos0=pos0, interleaved=interleaved), dtype)
    assert rel_err(dx.to_host(), want) <= tol * (10 if dtype == "f32" else 1)  # 2000 rad: fp32 angle rounding


def test_rope_reference_graph_replay_fp32(lm, hip, oracle):
    x = oracle.gen_normal((1, 8, 128, 64), 9100)
    got = lm.apply_rotary_embeddings(lm.to_device(x, hip), prev_seq=0).to_host()
    assert rel_err(got, oracle.rope_column_major_replay(x, prev_seq=0)) <= 2e-5


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("D", [128, 24, 20])  # 24: 16-byte chunks for fp32 only; 20: for neither
@pytest.mark.parametrize("interleaved", [False, True])
def test_kv_append_in_place(lm, hip, oracle, dtype, D, interleaved):
    B, Hkv, Lmax, T = 3, 2, 50, 2
    kc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9200), dtype)
    vc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9201), dtype)
    kn = oracle.round_to(oracle.gen_normal((B, Hkv, T, D), 9202), dtype)
    vn = oracle.round_to(oracle.gen_normal((B, Hkv, T, D), 9203), dtype)
    pos = np.array([0, 17, 49], np.int32)  # the last sequence has room for one of its two rows
    dk, dv, dkn, dvn = (lm.to_device(a, hip, dtype) for a in (kc, vc, kn, vn))
    lm.kv_append(dk, dv, dkn, dvn, lm.to_device(pos, hip))
    np.testing.assert_array_equal(dk.to_host(), oracle.kv_append(kc, kn, pos))
    np.testing.assert_array_equal(dv.to_host(), oracle.kv_append(vc, vn, pos))
    # fused rotary embedding of K: equals rope at the row position, then append; V untouched
    dk2, dv2 = lm.to_device(kc, hip, dtype), lm.to_device(vc, hip, dtype)
    lm.kv_append(dk2, dv2, dkn, dvn, lm.to_device(pos, hip), rope_k=True, interleaved=interleaved)
    kn_rot = oracle.round_to(oracle.rope(kn, pos0=pos, interleaved=interleaved), dtype)
    tol = 2e-5 if dtype == "f32" else 8e-3
    assert rel_err(dk2.to_host(), oracle.kv_append(kc, kn_rot, pos)) <= tol
    np.testing.assert_array_equal(dv2.to_host(), oracle.kv_append(vc, vn, pos))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("interleaved", [False, True])
@pytest.mark.parametrize("T,D,rope_k", [(1, 128, True), (1, 20, False), (3, 64, True), (250, 64, True)])
def test_kv_append_rotates_the_queries_in_the_same_call(lm, hip, oracle, dtype, interleaved, T, D, rope_k):
    """The decode step's q rides along with the cache append: rotated in place at pos[b] + t, what the rotary kernel
    alone produces (to an ulp) and within tolerance of the oracle; the caches come out as without q."""
    B, Hq, Hkv, Lmax = 3, 8, 2, 400
    kc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9270), dtype)
    vc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9271), dtype)
    kn = oracle.round_to(oracle.gen_normal((B, Hkv, T, D), 9272), dtype)
    vn = oracle.round_to(oracle.gen_normal((B, Hkv, T, D), 9273), dtype)
    q = oracle.round_to(oracle.gen_normal((B, Hq, T, D), 9274), dtype)
    pos = np.array([0, 17, 149], np.int32)
    dpos = lm.to_device(pos, hip)
    dk, dv, dkn, dvn, dq = (lm.to_device(a, hip, dtype) for a in (kc, vc, kn, vn, q))
    lm.kv_append(dk, dv, dkn, dvn, dpos, rope_k=rope_k, interleaved=interleaved, q=dq)
    dk2, dv2, dq2 = (lm.to_device(a, hip, dtype) for a in (kc, vc, q))
    lm.kv_append(dk2, dv2, dkn, dvn, dpos, rope_k=rope_k, interleaved=interleaved)
    lm.apply_rotary_embeddings(dq2, pos0=dpos, out=dq2, interleaved=interleaved)
    np.testing.assert_array_equal(dk.to_host(), dk2.to_host())
    np.testing.assert_array_equal(dv.to_host(), dv2.to_host())
    # the two kernels contract x0*cos - x1*sin differently: equal to an ulp of the element type
    assert rel_err(dq.to_host(), dq2.to_host()) <= {"f32": 1e-6, "f16": 1e-3, "bf16": 8e-3}[dtype]
    tol = {"f32": 1e-4, "f16": 2e-3, "bf16": 8e-3}[dtype]
    assert rel_err(dq.to_host(), oracle.rope(q, pos0=pos, interleaved=interleaved)) <= tol
    assert rel_err(dq.to_host(), q) > 1e-2  # it did rotate
    with pytest.raises(ValueError):
        lm.kv_append(dk, dv, dkn, dvn, dpos, q=lm.to_device(q[:, :, :, : D // 2], hip, dtype))


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("interleaved", [False, True])
def test_kv_append_whole_prompt(lm, hip, oracle, dtype, interleaved):
    # enough rows for the 16-byte-chunk kernel; the last sequence runs into the end of the cache
    B, Hkv, Lmax, D, T = 3, 4, 400, 64, 250
    kc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9250), dtype)
    vc = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9251), dtype)
    kn = oracle.round_to(oracle.gen_normal((B, Hkv, T, D), 9252), dtype)
    vn = oracle.round_to(oracle.gen_normal((B, Hkv, T, D), 9253), dtype)
    pos = np.array([0, 150, 300], np.int32)
    dk, dv, dkn, dvn = (lm.to_device(a, hip, dtype) for a in (kc, vc, kn, vn))
    lm.kv_append(dk, dv, dkn, dvn, lm.to_device(pos, hip))
    np.testing.assert_array_equal(dk.to_host(), oracle.kv_append(kc, kn, pos))
    np.testing.assert_array_equal(dv.to_host(), oracle.kv_append(vc, vn, pos))
    dk2, dv2 = lm.to_device(kc, hip, dtype), lm.to_device(vc, hip, dtype)
    lm.kv_append(dk2, dv2, dkn, dvn, lm.to_device(pos, hip), rope_k=True, interleaved=interleaved)
    kn_rot = oracle.round_to(oracle.rope(kn, pos0=pos, interleaved=interleaved), dtype)
    tol = {"f32": 1e-4, "f16": 2e-3, "bf16": 8e-3}[dtype]  # fp32: angles up to 550 rad, fp32 angle rounding
    assert rel_err(dk2.to_host(), oracle.kv_append(kc, kn_rot, pos)) <= tol
    np.testing.assert_array_equal(dv2.to_host(), oracle.kv_append(vc, vn, pos))


def test_kv_cache_state_allocation_and_row_placement(lm, hip):
    """The reference's own cache tests (tests/test_kv_cache.jl:13-29 "KVCacheState allocation", :54-70 "_kv_scatter
    places token at correct position") on the in-place form: a fresh cache is zero with step_pos 0 and the shape
    (batch, heads, max_seq, head_dim); a row written at position 0, 1 or the last slot lands there and nowhere else,
    the cache keeps its shape; appending to a full cache is refused."""
    cache = lm.KVCacheState(1, 6, 64, max_seq=10, dtype="f32", device=hip)
    assert cache.step_pos == 0 and cache.max_seq == 10
    assert cache.k.shape == cache.v.shape == (1, 6, 10, 64)
    assert not cache.k.to_host().any() and not cache.v.to_host().any()
    for pos in (0, 1, 3):  # the reference's minimal dims: (batch=1, heads=1, max_seq=4, head_dim=2)
        past = lm.to_device(np.zeros((1, 1, 4, 2), np.float32), hip)
        past_v = lm.to_device(np.zeros((1, 1, 4, 2), np.float32), hip)
        new = lm.to_device(np.array([[[[1.5, -2.5]]]], np.float32), hip)
        lm.kv_append(past, past_v, new, new, pos)
        want = np.zeros((1, 1, 4, 2), np.float32)
        want[0, 0, pos] = [1.5, -2.5]
        assert past.shape == (1, 1, 4, 2)
        np.testing.assert_array_equal(past.to_host(), want)
        np.testing.assert_array_equal(past_v.to_host(), want)
    for _ in range(10):
        cache.append(lm.to_device(np.ones((1, 6, 1, 64), np.float32), hip), lm.to_device(np.ones((1, 6, 1, 64), np.float32), hip))
    assert cache.step_pos == 10
    with pytest.raises(ValueError, match="full"):
        cache.append(lm.to_device(np.ones((1, 6, 1, 64), np.float32), hip), lm.to_device(np.ones((1, 6, 1, 64), np.float32), hip))


def test_incremental_decode_equals_causal_prefill(lm, hip, oracle):
    """Token-by-token decode through KVCacheState (append + fused cached attention) reproduces causal
    prefill row by row — the end-to-end property the reference's cached path is built on
    (reference src/Whisper.jl:584-620 with the cache update of :552-570)."""
    B, Hq, Hkv, S, D = 2, 8, 2, 40, 64
    q, k, v = inputs(oracle, (B, Hq, S, D), (B, Hkv, S, D), "f32", 9300)
    want = oracle.flash_attn(q, k, v, causal=True)
    cache = lm.KVCacheState(B, Hkv, D, max_seq=64, dtype="f32", device=hip)
    for t in range(S):
        cache.append(lm.to_device(np.ascontiguousarray(k[:, :, t:t + 1]), hip), lm.to_device(np.ascontiguousarray(v[:, :, t:t + 1]), hip))
        out = cache.attend(lm.to_device(np.ascontiguousarray(q[:, :, t]), hip)).to_host()
        assert rel_err(out, want[:, :, t]) <= 1e-5, t
    assert cache.step_pos == S


def test_plain_c_client_of_the_abi(hip):
    """The C ABI driven from C, not Python: tests/c_host/abi_client (built beforehand by `__graft_entry__.build()` or
    `python tests/c_host/build.py`) runs cross attention, causal GQA attention and split-KV decode in fp32 against its
    own float64 softmax and exits 0 when all are within 1e-5."""
    import os
    import subprocess
    binary = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_host", "abi_client")
    if not os.path.exists(binary):
        pytest.skip("tests/c_host/abi_client is not built (python tests/c_host/build.py needs gcc and the ROCm libraries)")
    res = subprocess.run([binary], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0, res.stdout


def test_calibration_kernels(lm, hip):
    # measurement aids: the copy kernel copies, the bare MFMA loop reports its flops and checks its arguments
    n = 1 << 16
    src = lm.HipArray((n,), "f32", hip).copy_from_host(np.arange(n, dtype=np.float32))
    dst = lm.HipArray((n,), "f32", hip).fill_bytes(0)
    lm.binding.calib_copy(dst.ptr, src.ptr, n * 4)
    assert np.array_equal(dst.to_host(), np.arange(n, dtype=np.float32))
    sink = lm.HipArray((512 * 256,), "f32", hip).fill_bytes(0xFF)
    ones = lm.HipArray((1 << 12,), "f16", hip).copy_from_host(np.ones(1 << 12, np.float16))
    flops = lm.binding.calib_mfma(sink.ptr, ones.ptr, 1 << 13, 3)
    assert flops == 512 * 4 * 3 * 8 * 2 * 32 * 32 * 16
    got = sink.to_host()
    # every accumulator element is a sum of 16 products 1*1 per MFMA: 6 MFMAs per accumulator, 64 elements per lane
    assert np.all(got == 64 * 16 * 6)
    with pytest.raises(lm.LuminalHipError):
        lm.binding.calib_mfma(sink.ptr, ones.ptr, 24, 1)
    # the instruction-mix streams: with operands of ones and no vector work, each of the 4 accumulators takes
    # 2 MFMAs per iteration, 16 products per element, and the 8 vector registers stay at 1
    sink.fill_bytes(0xFF)
    flops = lm.binding.calib_mix(sink.ptr, ones.ptr, 1 << 13, 3, 0)
    assert flops == 256 * 8 * 3 * 8 * 2 * 32 * 32 * 16
    assert np.all(sink.to_host() == 64 * 16 * 2 * 3 + 8)
    big = lm.HipArray((512 * 512,), "f32", hip).fill_bytes(0xFF)
    assert lm.binding.calib_mix(big.ptr, ones.ptr, 1 << 13, 3, 0, 4) == 2 * flops  # two workgroups per CU
    assert np.all(big.to_host() == 64 * 16 * 2 * 3 + 8)
    for mix in (2, 5, 7, 8):  # LDS fragments are ones too, so the matrix part is unchanged; the vector part is bounded (7, 8: accumulators in AGPRs)
        sink.fill_bytes(0xFF)
        lm.binding.calib_mix(sink.ptr, ones.ptr, 1 << 13, 3, mix)
        got = sink.to_host()
        assert np.all(np.isfinite(got)) and np.all(np.abs(got - 64 * 16 * 2 * 3) < 4096)
    with pytest.raises(lm.LuminalHipError):
        lm.binding.calib_mix(sink.ptr, ones.ptr, 1 << 13, 3, 9)
    with pytest.raises(lm.LuminalHipError):
        lm.binding.calib_mix(sink.ptr, ones.ptr, 1 << 13, 3, 0, 3)


def test_compiled_decode_step_graph_serves_every_position(lm, hip, oracle):
    """One compiled graph — in-place cache append that rotates q and, on the way in, K; fused cached
    attention — is built once and stepped through all positions with `pos` / `kv_len` as device tensors
    (the reference compiles one graph per position, src/Decoding.jl:98-106). Every step must equal the matching
    row of causal attention over the rotated sequence (reference src/NN.jl:352-382 as a whole)."""
    B, Hq, Hkv, S, D, Lmax = 2, 8, 2, 24, 64, 32
    q, k, v = inputs(oracle, (B, Hq, S, D), (B, Hkv, S, D), "f32", 9400)
    want = oracle.flash_attn(oracle.rope(q), oracle.rope(k), v, causal=True)
    g = lm.Graph()
    tq, tkn, tvn = lm.tensor(g, (B, Hq, 1, D)), lm.tensor(g, (B, Hkv, 1, D)), lm.tensor(g, (B, Hkv, 1, D))
    tkc, tvc = lm.tensor(g, (B, Hkv, Lmax, D)), lm.tensor(g, (B, Hkv, Lmax, D))
    tpos, tlen = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
    out, kc2, vc2 = lm.cached_self_attention_core(tq, tkn, tvn, tkc, tvc, tpos, tlen, rope_base=10000.0)
    cg = lm.compile(g, hip)
    n_steps_built = len(cg.steps)
    for t in range(S):
        res = cg({tq.id: np.ascontiguousarray(q[:, :, t:t + 1]), tkn.id: np.ascontiguousarray(k[:, :, t:t + 1]),
                  tvn.id: np.ascontiguousarray(v[:, :, t:t + 1]), tpos.id: np.full(B, t, np.int32),
                  tlen.id: np.full(B, t + 1, np.int32)})
        got = res[out.id].to_host()
        assert rel_err(got, want[:, :, t]) <= 2e-5, t
    assert len(cg.steps) == n_steps_built == 2  # append with the rotations, attention: nothing was rebuilt per position
    # the cache the graph holds is the rotated K and the raw V of all steps
    kc_host = res[kc2.id][0].to_host()
    assert rel_err(kc_host[:, :, :S], oracle.rope(k)) <= 2e-5
    assert np.array_equal(res[kc2.id][1].to_host()[:, :, :S], v)


@pytest.mark.parametrize("dtype,Lmax", [("f32", 32), ("bf16", 4096)])  # the long cache takes the split-KV kernels + merge
def test_decode_step_recorded_as_one_hip_graph(lm, hip, oracle, dtype, Lmax):
    """The same step graph, recorded once into a HIP graph after the first position and replayed for every later
    one, must give bit for bit what an unrecorded twin gives, with the program's own eager launches and
    synchronisations between the replays (reference src/Compiler.jl:250-255: the compiled step closure)."""
    B, Hq, Hkv, S, D = 2, 8, 2, 20, 64
    q, k, v = inputs(oracle, (B, Hq, S, D), (B, Hkv, S, D), dtype, 9450)
    want = oracle.flash_attn(oracle.round_to(oracle.rope(q), dtype), oracle.round_to(oracle.rope(k), dtype), v, causal=True)

    def build():
        g = lm.Graph()
        tq, tkn, tvn = lm.tensor(g, (B, Hq, 1, D), dtype), lm.tensor(g, (B, Hkv, 1, D), dtype), lm.tensor(g, (B, Hkv, 1, D), dtype)
        tkc, tvc = lm.tensor(g, (B, Hkv, Lmax, D), dtype), lm.tensor(g, (B, Hkv, Lmax, D), dtype)
        tpos, tlen = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
        out, _, _ = lm.cached_self_attention_core(tq, tkn, tvn, tkc, tvc, tpos, tlen, rope_base=10000.0, out_dtype="f32")
        return lm.compile(g, hip), (tq, tkn, tvn, tpos, tlen), out

    cg, ids, out = build()
    twin, ids2, out2 = build()

    def feed(handles, t):
        tq, tkn, tvn, tpos, tlen = handles
        return {tq.id: lm.to_device(np.ascontiguousarray(q[:, :, t:t + 1]), hip, dtype),
                tkn.id: lm.to_device(np.ascontiguousarray(k[:, :, t:t + 1]), hip, dtype),
                tvn.id: lm.to_device(np.ascontiguousarray(v[:, :, t:t + 1]), hip, dtype),
                tpos.id: np.full(B, t, np.int32), tlen.id: np.full(B, t + 1, np.int32)}

    xq, xk, xv = inputs(oracle, (1, 4, 200, 64), (1, 4, 200, 64), "f16", 9460)
    x_want = oracle.flash_attn(xq, xk, xv, causal=True)
    tol = 2e-5 if dtype == "f32" else 1e-2  # bf16: q and k are rounded again after the rotation
    for t in range(S):
        if t == 1:
            cg.capture()  # step 0 ran eagerly; this call records and replays, the later ones replay
        got = cg(feed(ids, t))[out.id].to_host()
        assert ("hip_exec" in cg.cache) == (t >= 1)
        ref = twin(feed(ids2, t))[out2.id].to_host()
        assert np.array_equal(got, ref), t
        assert rel_err(got, want[:, :, t]) <= tol, t
        # unrelated eager work and a synchronisation between the replays
        assert rel_err(run_flash(lm, hip, xq, xk, xv, "f16", True), x_want) <= TOL["f16"]
        lm.binding.sync()
    cg.release()
    assert "hip_exec" not in cg.cache
    got = cg(feed(ids, S - 1))[out.id].to_host()  # step by step again after release
    assert rel_err(got, want[:, :, S - 1]) <= tol


@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_self_attention_core_is_rope_plus_gqa_flash(lm, hip, oracle, dtype):
    """Prefill form of the attention layer core: rotary nodes on Q and K, then one flash node reading the Hkv heads
    directly; equals the oracle's rope followed by GQA attention in the head order repeat_kv produces."""
    B, Hq, Hkv, S, D = 1, 8, 2, 96, 64
    q, k, v = inputs(oracle, (B, Hq, S, D), (B, Hkv, S, D), dtype, 9500)
    want = oracle.flash_attn(oracle.round_to(oracle.rope(q, prev_seq=5), dtype), oracle.round_to(oracle.rope(k, prev_seq=5), dtype), v, causal=True)
    g = lm.Graph()
    tq, tk, tv = lm.tensor(g, q.shape, dtype), lm.tensor(g, k.shape, dtype), lm.tensor(g, v.shape, dtype)
    out = lm.self_attention_core(tq, tk, tv, causal=True, prev_seq=5, rope_base=10000.0, out_dtype=out_type(dtype, None))
    got = lm.execute(g, out.id, {tq.id: q, tk.id: k, tv.id: v}, hip)
    assert rel_err(got, want) <= (2e-5 if dtype == "f32" else 3e-3)


def test_decode_batch_above_the_persistent_kernel_limit(lm, hip, oracle):
    # more than 1024 sequences: the matrix-core decode kernel keeps its per-sequence prefix sums in LDS and hands
    # larger batches to the vector kernel; same results expected, ragged lengths included
    B, Hq, Hkv, L, D = 1100, 4, 2, 96, 64
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), "bf16", 9600)
    lens = oracle.gen_uniform_int(B, 9601, 1, L).astype(np.int32)
    got = run_decode(lm, hip, q, k, v, "bf16", kv_len=lens)
    assert rel_err(got, oracle.decode_attn(q, k, v, kv_len=lens, nthreads=NT)) <= 2e-3
    # and exactly at the limit the persistent kernel still runs
    got = run_decode(lm, hip, q[:1024], k[:1024], v[:1024], "bf16", kv_len=lens[:1024], num_splits=2)
    assert rel_err(got, oracle.decode_attn(q[:1024], k[:1024], v[:1024], kv_len=lens[:1024], nthreads=NT)) <= 2e-3


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_sequence_four_times_the_longest_benchmark_checked_through_properties(lm, hip, oracle, dtype):
    """S = 16384, causal, D = 128: too long for the scalar oracle on every row, so the result is checked through what
    does not depend on the size: rows below n depend on the first n keys only (oracle on that prefix), single rows
    anywhere against float64 numpy, and a constant V comes back as that constant."""
    B, H, S, D = 1, 4, 16384, 128
    q, k, v = inputs(oracle, (B, H, S, D), (B, H, S, D), dtype, 9650, mul=0.7)
    got = run_flash(lm, hip, q, k, v, dtype, True)
    n = 1024
    want = oracle.flash_attn(q[:, :, :n], k[:, :, :n], v[:, :, :n], causal=True, nthreads=NT)
    assert rel_err(got[:, :, :n], want) <= TOL[dtype]
    scale = 1.0 / np.sqrt(D)
    rows = [n, 4095, 4096, 8191, 12345, S - 129, S - 128, S - 1]
    want = np.empty((B, H, len(rows), D))
    for r, i in enumerate(rows):
        s = np.einsum("bhkd,bhd->bhk", k[:, :, :i + 1].astype(np.float64), q[:, :, i].astype(np.float64)) * scale
        w = np.exp(s - s.max(-1, keepdims=True))
        want[:, :, r] = np.einsum("bhk,bhkd->bhd", w, v[:, :, :i + 1].astype(np.float64)) / w.sum(-1)[..., None]
    assert rel_err(got[:, :, rows], want) <= TOL[dtype]
    const = np.full_like(v, 0.75)
    got = run_flash(lm, hip, q, k, const, dtype, True)
    # fp32: sum and weighted sum each carry ~sqrt(S) * 2^-24 of rounding, as the oracle's own fp32 loop would
    assert np.abs(got - 0.75).max() <= (1e-5 if dtype == "f32" else 1e-3)


def test_decode_over_a_cache_four_times_the_longest_benchmark_sequence(lm, hip, oracle):
    """kv_len = 131072 (and one short neighbour in the same batch), bf16, GQA 4: float64 numpy on every head."""
    B, Hq, Hkv, L, D = 2, 32, 8, 131072, 128
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), "bf16", 9660)
    lens = np.array([L, 777], np.int32)
    got = run_decode(lm, hip, q, k, v, "bf16", kv_len=lens)
    want = np.empty((B, Hq, D))
    for b in range(B):
        for hq in range(Hq):
            kk, vv = k[b, hq % Hkv, :lens[b]].astype(np.float64), v[b, hq % Hkv, :lens[b]].astype(np.float64)
            s = kk @ q[b, hq].astype(np.float64) / np.sqrt(D)
            w = np.exp(s - s.max())
            want[b, hq] = w @ vv / w.sum()
    assert rel_err(got, want) <= 2e-3
    for b in range(B):  # each sequence on its own scale: the long one averages 131072 rows, the short one 777
        assert rel_err(got[b], want[b]) <= 2e-3


def _padded(lm, hip, x, dtype, row_pad, rng):
    """Upload x (B,H,S,D) into a buffer whose rows are D + row_pad apart (padding filled with NaN);
    returns (array, element strides (b, h, s))."""
    B, H, S, D = x.shape
    buf = np.full((B, H, S, D + row_pad), np.nan, np.float32)
    buf[..., :D] = x
    return lm.to_device(buf, hip, dtype), (H * S * (D + row_pad), S * (D + row_pad), D + row_pad)


@pytest.mark.parametrize("seed", range(32))
def test_prefill_random_shapes_strides_and_options(lm, hip, oracle, seed):
    """Seeded sweep over what the entry point dispatches on: element type, head dim (matrix-core and vector kernels),
    GQA group and head map, causal, ragged kv_len, row strides (16-byte aligned and not), fp32 output of half inputs.
    Seeds from 24 on draw launches of more than a thousand 256-row workgroups (the eight-wave instantiations)."""
    rng = np.random.default_rng(9700 + seed)
    dtype = ["f32", "f16", "bf16"][seed % 3]
    D = int(rng.choice([16, 32, 40, 64, 80, 96, 128]))
    if seed < 24:
        Hkv = int(rng.integers(1, 4)); G = int(rng.choice([1, 2, 4])); Hq = Hkv * G
        B = int(rng.integers(1, 4))
        Sq, Sk = int(rng.integers(1, 260)), int(rng.integers(1, 330))
    else:
        dtype = ["f16", "bf16"][seed % 2]
        Hkv = int(rng.integers(11, 17)); G = int(rng.choice([2, 4])); Hq = Hkv * G
        B = 352 // Hq + 1
        Sq, Sk = int(rng.integers(513, 700)), int(rng.integers(260, 800))
    causal = bool(rng.integers(0, 2)); head_map = int(rng.integers(0, 2))
    pad_q, pad_kv = int(rng.choice([0, 8, 3])), int(rng.choice([0, 8, 16, 5]))
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 9800 + seed)
    lens = rng.integers(1, Sk + 1, size=B).astype(np.int32) if rng.integers(0, 2) else None
    dq, qs = _padded(lm, hip, q, dtype, pad_q, rng)
    dk, ks = _padded(lm, hip, k, dtype, pad_kv, rng)
    dv, vs = _padded(lm, hip, v, dtype, pad_kv, rng)
    odt = "f32" if dtype == "bf16" or rng.integers(0, 2) else dtype
    out = lm.HipArray((B, Hq, Sq, D), odt, hip)
    dl = None if lens is None else lm.to_device(lens, hip)
    p = lm.binding.AttnParams()
    p.out, p.q, p.k, p.v = out.ptr, dq.ptr, dk.ptr, dv.ptr
    p.kv_len = dl.ptr if dl is not None else None
    p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D = B, Hq, Hkv, Sq, Sk, D
    for arr, st in ((p.q_stride, qs), (p.k_stride, ks), (p.v_stride, vs)):
        arr[0], arr[1], arr[2] = st
    p.dtype, p.scale, p.causal, p.head_map = lm.binding.DTYPE_CODES[dtype], lm.default_scale(D), int(causal), head_map
    p.out_f32 = int(odt == "f32")
    lm.binding.flash_attn_fwd(p)
    want = oracle.flash_attn(q, k, v, causal=causal, head_map=head_map, kv_len=lens, nthreads=NT)
    case = dict(dtype=dtype, D=D, B=B, Hq=Hq, Hkv=Hkv, Sq=Sq, Sk=Sk, causal=causal, head_map=head_map, pad_q=pad_q, pad_kv=pad_kv,
                lens=None if lens is None else lens.tolist(), out=odt)
    tol = TOL[dtype] if odt == "f32" or dtype == "f32" else 3e-3  # a half-precision result adds its own rounding
    assert rel_err(out.to_host(), want) <= tol, case


@pytest.mark.parametrize("seed", range(12))
def test_decode_random_shapes_and_options(lm, hip, oracle, seed):
    rng = np.random.default_rng(9900 + seed)
    dtype = ["f32", "f16", "bf16"][seed % 3]
    D = int(rng.choice([32, 64, 96, 128, 256] if dtype != "f32" else [32, 64, 128]))
    Hkv = int(rng.integers(1, 5)); G = int(rng.choice([1, 2, 4, 8])); Hq = Hkv * G
    B = int(rng.integers(1, 6)); L = int(rng.integers(1, 700))
    head_map = int(rng.integers(0, 2)); splits = int(rng.choice([0, 1, 2, 5]))
    q, k, v = inputs(oracle, (B, Hq, D), (B, Hkv, L, D), dtype, 9950 + seed)
    lens = rng.integers(1, L + 1, size=B).astype(np.int32) if rng.integers(0, 2) else None
    got = run_decode(lm, hip, q, k, v, dtype, kv_len=lens, head_map=head_map, num_splits=splits)
    want = oracle.decode_attn(q, k, v, kv_len=lens, head_map=head_map, nthreads=NT)
    assert rel_err(got, want) <= TOL[dtype], dict(dtype=dtype, D=D, B=B, Hq=Hq, Hkv=Hkv, L=L, head_map=head_map, splits=splits,
                                                   lens=None if lens is None else lens.tolist())
