"""Pins the CPU oracle (oracle/attn_oracle.c) without running the reference (Julia, not available):
golden vectors from an independent numpy implementation, the reference's own test criterion,
closed forms and invariants chosen so that a dropped term, a wrong sign/index or a transposed
operand fails at least one of them."""
import numpy as np
import pytest

from conftest import rel_err


def test_golden_vectors(oracle, golden):
    for name, c in golden.items():
        q, k, v = c["q"], c["k"], c["v"]
        got = oracle.flash_attn(q, k, v, scale=c["scale"], causal=c["causal"], kv_len=c["kv_len"])
        assert rel_err(got, c["out"]) <= 1e-5, name
        got64 = oracle.naive_attention_f64(q, k, v, scale=c["scale"], causal=c["causal"], kv_len=c["kv_len"])
        assert rel_err(got64, c["out"]) <= 1e-6, name


@pytest.mark.parametrize("causal", [False, True])
def test_flash_equals_naive_on_reference_test_shape(oracle, causal):
    # reference tests/test_flash_attention_verification.jl:24-49 (non-causal, rtol 1e-4) and :54-94
    B, H, S, D = 1, 1, 8, 16
    q, k, v = (oracle.gen_normal((B, H, S, D), s) for s in (1, 2, 3))
    flash = oracle.flash_attn(q, k, v, causal=causal)
    for naive in (oracle.naive_attention_f64(q, k, v, causal=causal), oracle.naive_attention_np(q, k, v, causal=causal)):
        np.testing.assert_allclose(flash, naive, rtol=1e-4, atol=1e-6)
        assert rel_err(flash, naive) <= 1e-5


def test_config1_shape_flash_equals_naive(oracle):
    B, H, S, D = 1, 8, 128, 64
    q, k, v = (oracle.gen_normal((B, H, S, D), s) for s in (11, 12, 13))
    assert rel_err(oracle.flash_attn(q, k, v, causal=True), oracle.naive_attention_np(q, k, v, causal=True)) <= 1e-5


def test_closed_forms(oracle):
    B, H, S, D = 2, 3, 17, 8
    q, k, v = (oracle.gen_normal((B, H, S, D), s) for s in (4, 5, 6))
    out = oracle.flash_attn(q, k, v, causal=True)
    # first causal row sees only key 0 -> exactly V[0]
    np.testing.assert_array_equal(out[:, :, 0, :], v[:, :, 0, :])
    # Q = 0 -> uniform weights -> running mean of V (causal), plain mean (non-causal)
    zero = np.zeros_like(q)
    run_mean = np.cumsum(v.astype(np.float64), axis=2) / np.arange(1, S + 1)[None, None, :, None]
    assert rel_err(oracle.flash_attn(zero, k, v, causal=True), run_mean) <= 1e-6
    assert rel_err(oracle.flash_attn(zero, k, v, causal=False),
                   np.broadcast_to(v.astype(np.float64).mean(axis=2, keepdims=True), v.shape)) <= 1e-6
    # V = 1 -> output 1 (weights sum to one)
    np.testing.assert_allclose(oracle.flash_attn(q, k, np.ones_like(v), causal=True), 1.0, rtol=0, atol=1e-6)
    # a single key -> that V row, whatever the score
    o1 = oracle.flash_attn(q, k[:, :, :1], v[:, :, :1], causal=False)
    np.testing.assert_array_equal(o1, np.broadcast_to(v[:, :, :1], o1.shape))
    # one dominant key -> that key's V row
    kd = k.copy()
    kd[:, :, 5, :] = 50.0 * q[:, :, 9, :] / np.linalg.norm(q[:, :, 9, :], axis=-1, keepdims=True)
    od = oracle.flash_attn(q[:, :, 9:10], kd, v, causal=False, scale=10.0)
    assert rel_err(od[:, :, 0], v[:, :, 5]) <= 1e-5


def test_operand_roles_are_not_interchangeable(oracle):
    # transposed / swapped operands must change the answer (guards the checks above from being vacuous)
    B, H, S, D = 1, 2, 6, 4
    q, k, v = (oracle.gen_normal((B, H, S, D), s) for s in (7, 8, 9))
    base = oracle.naive_attention_np(q, k, v, causal=True)
    assert rel_err(oracle.flash_attn(q, k, v, causal=True), base) <= 1e-5
    assert rel_err(oracle.flash_attn(q, v, k, causal=True), base) > 1e-2
    assert rel_err(oracle.flash_attn(k, q, v, causal=True), base) > 1e-2
    assert rel_err(oracle.flash_attn(q, k, v, causal=False), base) > 1e-2
    assert rel_err(oracle.flash_attn(q, k, v, causal=True, scale=-0.5), base) > 1e-2


def test_logit_shift_and_key_permutation_invariance(oracle):
    B, H, Sq, Sk, D = 1, 2, 5, 33, 16
    q = oracle.gen_normal((B, H, Sq, D), 10)
    k = oracle.gen_normal((B, H, Sk, D), 11)
    v = oracle.gen_normal((B, H, Sk, D), 12)
    base = oracle.flash_attn(q, k, v)
    # permuting keys together with values leaves non-causal attention unchanged
    perm = np.random.default_rng(0).permutation(Sk)
    assert rel_err(oracle.flash_attn(q, k[:, :, perm], v[:, :, perm]), base) <= 1e-5
    # adding the same vector c to every key shifts all logits of a row by q.c -> softmax unchanged
    c = oracle.gen_normal((1, 1, 1, D), 13)
    assert rel_err(oracle.flash_attn(q, k + c, v), base) <= 2e-5
    # huge logits: the online max keeps exp() in range (no inf/nan)
    big = oracle.flash_attn(q * 100, k * 100, v)
    assert np.all(np.isfinite(big))
    assert rel_err(big, oracle.naive_attention_np(q * 100, k * 100, v)) <= 1e-5


def test_gqa_head_map_is_column_major_repeat_kv(oracle):
    # brute force on a tiny input: literal Expand + column-major Reshape vs the hq % Hkv shortcut
    B, Hq, Hkv, S, D = 1, 4, 2, 3, 2
    q = oracle.gen_normal((B, Hq, S, D), 20)
    k = oracle.gen_normal((B, Hkv, S, D), 21)
    v = oracle.gen_normal((B, Hkv, S, D), 22)
    G = Hq // Hkv
    k_rep = oracle.repeat_kv_column_major(k, G)
    v_rep = oracle.repeat_kv_column_major(v, G)
    for hq in range(Hq):
        np.testing.assert_array_equal(k_rep[:, hq], k[:, hq % Hkv])
    want = oracle.flash_attn(q, k_rep, v_rep, causal=True)  # MHA on the materialised repeat
    got = oracle.flash_attn(q, k, v, causal=True, head_map=oracle.HEADMAP_INTERLEAVED)
    np.testing.assert_array_equal(got, want)
    # the blocked map is np.repeat along heads, and differs
    want_b = oracle.flash_attn(q, np.repeat(k, G, axis=1), np.repeat(v, G, axis=1), causal=True)
    got_b = oracle.flash_attn(q, k, v, causal=True, head_map=oracle.HEADMAP_BLOCKED)
    np.testing.assert_array_equal(got_b, want_b)
    assert rel_err(got_b, want) > 1e-3
    # numpy twin agrees on both maps
    for hm in (oracle.HEADMAP_INTERLEAVED, oracle.HEADMAP_BLOCKED):
        assert rel_err(oracle.flash_attn(q, k, v, causal=True, head_map=hm),
                       oracle.naive_attention_np(q, k, v, causal=True, head_map=hm)) <= 1e-5


def test_decode_equals_last_row_of_causal_prefill(oracle):
    B, Hq, Hkv, L, D = 2, 4, 2, 29, 16
    q = oracle.gen_normal((B, Hq, L, D), 30)
    k = oracle.gen_normal((B, Hkv, L, D), 31)
    v = oracle.gen_normal((B, Hkv, L, D), 32)
    full = oracle.flash_attn(q, k, v, causal=True)
    dec = oracle.decode_attn(q[:, :, L - 1], k, v, kv_len=np.full(B, L, np.int32))
    np.testing.assert_array_equal(dec, full[:, :, L - 1])


def test_ragged_kv_len_ignores_tail(oracle):
    B, Hq, Hkv, Lmax, D = 3, 4, 2, 40, 8
    q = oracle.gen_normal((B, Hq, D), 40)
    k = oracle.gen_normal((B, Hkv, Lmax, D), 41)
    v = oracle.gen_normal((B, Hkv, Lmax, D), 42)
    lens = np.array([40, 13, 1], np.int32)
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):  # poison the tail: it must not be read into the result
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.inf
    got = oracle.decode_attn(q, kp, vp, kv_len=lens)
    for b, n in enumerate(lens):
        want = oracle.decode_attn(q[b:b + 1], k[b:b + 1, :, :n], v[b:b + 1, :, :n])
        np.testing.assert_array_equal(got[b:b + 1], want)
    assert rel_err(got, oracle.naive_attention_np(q[:, :, None], k, v, kv_len=lens)[:, :, 0]) <= 1e-5


def test_threads_do_not_change_bits(oracle):
    q, k, v = (oracle.gen_normal((2, 4, 50, 32), s) for s in (50, 51, 52))
    np.testing.assert_array_equal(oracle.flash_attn(q, k, v, causal=True, nthreads=1),
                                  oracle.flash_attn(q, k, v, causal=True, nthreads=4))


def test_generator_twins_and_rounding(oracle):
    a = oracle.gen_normal((1000,), 123, 0.5)
    b = oracle.gen_normal_np((1000,), 123, 0.5)
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-6)
    big = oracle.gen_normal((200000,), 7)
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1) < 0.01
    # prefix property: a shorter stream is a prefix of a longer one
    np.testing.assert_array_equal(oracle.gen_normal((10,), 9), oracle.gen_normal((20,), 9)[:10])
    x = (oracle.gen_normal((100000,), 5) * np.exp(oracle.gen_normal((100000,), 6) * 4)).astype(np.float32)
    with np.errstate(over="ignore"):
        np.testing.assert_array_equal(oracle.round_to(x, "f16"), x.astype(np.float16).astype(np.float32))
    r = oracle.round_to(x, "bf16")
    assert np.all((r.view(np.uint32) & 0xFFFF) == 0)
    assert np.all(np.abs(r - x) <= np.abs(x) * 2.0 ** -8)
    lens = oracle.gen_uniform_int(1000, 3, 8192, 32768)
    assert lens.min() >= 8192 and lens.max() <= 32768 and len(set(lens.tolist())) > 900


# ---------------------------------------------------------------------------------------------
# rotary embedding and KV-cache append (the operators in front of decode attention)
# ---------------------------------------------------------------------------------------------
def test_rope_matches_column_major_replay_of_the_reference_graph(oracle):
    for (shape, prev) in [((1, 2, 5, 8), 0), ((2, 3, 9, 64), 17), ((1, 1, 1, 128), 4095)]:
        x = oracle.gen_normal(shape, 60 + prev)
        want = oracle.rope_column_major_replay(x, prev_seq=prev)
        # the oracle works in fp32 like the reference; the angle pos * inv_freq then carries a rounding
        # error of ~pos * 2^-24 rad, which is what separates it from the float64 replay
        assert rel_err(oracle.rope(x, prev_seq=prev), want) <= 1e-5 + prev * 4e-8
    # the pairing is (j, j + D/2): rotating a tensor that is non-zero only at d = 0 moves weight to d = D/2
    x = np.zeros((1, 1, 2, 8), np.float32)
    x[..., 0] = 1.0
    y = oracle.rope(x, prev_seq=1)
    assert abs(y[0, 0, 0, 4] - np.sin(1.0)) < 1e-6 and abs(y[0, 0, 0, 0] - np.cos(1.0)) < 1e-6
    assert np.all(y[0, 0, 0, [1, 2, 3, 5, 6, 7]] == 0)
    # the interleaved variant pairs (2j, 2j+1) instead
    yi = oracle.rope(x, prev_seq=1, interleaved=True)
    assert abs(yi[0, 0, 0, 1] - np.sin(1.0)) < 1e-6 and yi[0, 0, 0, 4] == 0


def test_rope_properties(oracle):
    B, H, S, D = 2, 2, 6, 32
    x = oracle.gen_normal((B, H, S, D), 70)
    y = oracle.rope(x, prev_seq=3)
    # rotations preserve the norm of every pair, hence of every row
    np.testing.assert_allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)
    # position 0 is the identity
    np.testing.assert_allclose(oracle.rope(x[:, :, :1], prev_seq=0), x[:, :, :1], rtol=0, atol=1e-7)
    # rotating by a then by b is rotating by a + b (single-row tensors so that every row sits at s = 0)
    row = x[:, :, :1]
    np.testing.assert_allclose(oracle.rope(oracle.rope(row, prev_seq=5), prev_seq=9), oracle.rope(row, prev_seq=14),
                               rtol=0, atol=2e-5)
    # q.k after the embedding depends on the position difference only
    q, k = oracle.gen_normal((1, 1, 1, D), 71), oracle.gen_normal((1, 1, 1, D), 72)
    d1 = float(np.sum(oracle.rope(q, prev_seq=10) * oracle.rope(k, prev_seq=4)))
    d2 = float(np.sum(oracle.rope(q, prev_seq=106) * oracle.rope(k, prev_seq=100)))
    assert abs(d1 - d2) < 1e-3
    # per-sequence start positions equal separate calls with scalar prev_seq
    pos0 = np.array([4, 9], np.int32)
    yp = oracle.rope(x, pos0=pos0)
    for b in range(B):
        np.testing.assert_array_equal(yp[b:b + 1], oracle.rope(x[b:b + 1], prev_seq=int(pos0[b])))


def test_kv_append_equals_slice_and_concat_scatter(oracle):
    B, H, Lmax, D = 1, 2, 6, 4
    past = oracle.gen_normal((B, H, Lmax, D), 80)
    new = oracle.gen_normal((B, H, 1, D), 81)
    for step_pos in range(Lmax):  # includes the two special cases of the reference (first and last row)
        got = oracle.kv_append(past, new, np.array([step_pos], np.int32))
        np.testing.assert_array_equal(got, oracle.kv_scatter_replay(past, new, step_pos))
    # several tokens, per-sequence positions, rows past the end are dropped
    past = oracle.gen_normal((2, 2, 5, 4), 82)
    new = oracle.gen_normal((2, 2, 3, 4), 83)
    got = oracle.kv_append(past, new, np.array([1, 3], np.int32))
    want = past.copy()
    want[0, :, 1:4] = new[0]
    want[1, :, 3:5] = new[1, :, :2]
    np.testing.assert_array_equal(got, want)


def test_decode_entry_is_the_one_row_prefill(oracle):
    # lmo_decode_attn (what oracle.decode_attn calls) is the restated recurrence on one query row over the first
    # kv_len[b] cache rows: bit for bit the Sq = 1 non-causal call, and the float64 softmax over exactly those rows
    B, Hq, Hkv, L, D = 3, 8, 2, 77, 32
    q = oracle.gen_normal((B, Hq, D), 40)
    k = oracle.gen_normal((B, Hkv, L, D), 41)
    v = oracle.gen_normal((B, Hkv, L, D), 42)
    lens = np.array([77, 1, 30], np.int32)
    for head_map in (0, 1):
        got = oracle.decode_attn(q, k, v, kv_len=lens, head_map=head_map)
        same = oracle.flash_attn(q[:, :, None], k, v, kv_len=lens, head_map=head_map)[:, :, 0]
        np.testing.assert_array_equal(got, same)
        for b, n in enumerate(lens):
            ref = oracle.naive_attention_np(q[b:b + 1, :, None], k[b:b + 1, :, :n], v[b:b + 1, :, :n], head_map=head_map)[:, :, 0]
            np.testing.assert_allclose(got[b:b + 1], ref, rtol=1e-5, atol=1e-6)
