"""bf16 launches of prefill_mfma_kernel hand V to the matrix cores as fp16: every tile is rewritten on its way into LDS,
relative to the largest finite |v| the workgroup has met so far, and the accumulators carry the power of two. fp16 has
five exponent bits, bf16 eight, so these cases move that largest value around: magnitudes that grow or shrink along the
keys by 80 powers of two, values far outside fp16's range, a jump in the middle of a tile, heads of very different scale,
zeros, infinities and NaNs. The check is per query row (max error over the head dim against the row's own largest output),
which a rewrite relative to one launch-wide maximum would fail."""
import numpy as np
import pytest

from conftest import TOL, rel_err
from test_parity_gpu import inputs, run_flash
from test_random_shapes_gpu import poison_tail

pytestmark = pytest.mark.gpu

NT = 16
ROW_TOL = 3e-3  # per row; the contract's 2e-3 is over the whole tensor

# (B, H, S, D, causal): launches of one-tile workgroups whose waves own their rows alone (the plan query confirms it)
SHAPES = [
    (1, 24, 3072, 64, True),    # 128-row workgroups, 64-key tiles
    (1, 32, 4096, 96, True),    # 256-row workgroups alone on a CU, 128-key tiles
    (1, 40, 2048, 128, False),  # head dim 128, no mask
]
IDS = ["D64-causal", "D96-causal", "D128-full"]


def row_errors(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = np.abs(want).max(axis=-1)
    err = np.abs(got - want).max(axis=-1)
    return np.where(scale > 0, err / np.where(scale > 0, scale, 1.0), err)


def setup(lm, oracle, shape, seed):
    B, H, S, D, causal = shape
    plan = lm.flash_attention_plan((B, H, S, D), (B, H, S, D), "bf16", causal)
    print(plan, flush=True)
    assert "prefill_mfma_kernel<bf16" in plan and "key groups=1" in plan and plan.endswith("V as fp16"), plan
    q, k, v = inputs(oracle, (B, H, S, D), (B, H, S, D), "bf16", seed, 0.8)
    heads = np.array([0, H // 2, H - 1])
    return q, k, v, heads


def power_of_two(e):
    return np.ldexp(np.float32(1.0), np.asarray(e, np.int32)).astype(np.float32)


@pytest.mark.parametrize("shape", SHAPES, ids=IDS)
@pytest.mark.parametrize("profile", ["grows", "shrinks", "huge", "tiny", "heads"])
def test_value_magnitudes_along_keys_and_heads(lm, hip, oracle, shape, profile):
    B, H, S, D, causal = shape
    q, k, v, heads = setup(lm, oracle, shape, 99000 + D)
    if profile == "grows":      # 2^-40 at key 0 ... 2^40 at the last key
        v = v * power_of_two(np.linspace(-40, 40, S).round())[None, None, :, None]
    elif profile == "shrinks":
        v = v * power_of_two(np.linspace(40, -40, S).round())[None, None, :, None]
    elif profile == "huge":     # every value beyond fp16's largest
        v = v * power_of_two(100)
    elif profile == "tiny":     # every value below fp16's smallest subnormal
        v = v * power_of_two(-80)
    else:                       # 2^-50 ... 2^50 from the first head to the last
        v = v * power_of_two(np.linspace(-50, 50, H).round())[None, :, None, None]
    assert np.array_equal(oracle.round_to(v, "bf16"), v)  # powers of two keep bf16 values bf16
    got = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
    assert np.isfinite(got).all()
    want = oracle.flash_attn(q[:, heads], k[:, heads], v[:, heads], causal=causal, nthreads=NT)
    rows = row_errors(got[:, heads], want)
    print("%s: worst row %.3g, median row %.3g" % (profile, rows.max(), np.median(rows)), flush=True)
    assert rows.max() <= ROW_TOL
    if profile != "heads":
        assert rel_err(got[:, heads], want) <= TOL["bf16"]


@pytest.mark.parametrize("shape", SHAPES[:2], ids=IDS[:2])
def test_jump_inside_a_tile(lm, hip, oracle, shape):
    """From key J on the values are 2^60 times larger. Rows that end before J's 256-row tile never meet the large values
    and keep their own scale; rows from J on are dominated by them. Rows between the start of that tile and J share a
    workgroup with the large values: they are held to the contract's tensor-wide tolerance only."""
    B, H, S, D, causal = shape
    q, k, v, heads = setup(lm, oracle, shape, 99100 + D)
    J = S // 2 + 77
    v[:, :, J:] *= power_of_two(60)
    got = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
    assert np.isfinite(got).all()
    want = oracle.flash_attn(q[:, heads], k[:, heads], v[:, heads], causal=True, nthreads=NT)
    rows = row_errors(got[:, heads], want)
    first = J // 256 * 256
    print("rows before the tile %.3g, rows from J on %.3g" % (rows[..., :first].max(), rows[..., J:].max()), flush=True)
    assert rows[..., :first].max() <= ROW_TOL
    assert rows[..., J:].max() <= ROW_TOL
    assert rel_err(got[:, heads], want) <= TOL["bf16"]


@pytest.mark.parametrize("shape", SHAPES[:2], ids=IDS[:2])
@pytest.mark.parametrize("special", [np.inf, -np.inf, np.nan])
def test_an_infinity_or_nan_among_the_values(lm, hip, oracle, shape, special):
    """One element of V (key J, head dim 5) is not finite. It is not taken for the largest value (the finite ones keep their
    precision), it reaches the matrix cores as what it is, and it only shows in its own column: every other head dim is
    untouched, and so is column 5 for the rows that end before J's tile."""
    B, H, S, D, causal = shape
    q, k, v, heads = setup(lm, oracle, shape, 99200 + D)
    J = S // 2 + 41
    v[:, :, J, 5] = special
    got = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
    vf = v.copy()
    vf[:, :, J, 5] = 0.0
    want = oracle.flash_attn(q[:, heads], k[:, heads], vf[:, heads], causal=True, nthreads=NT)
    g = got[:, heads]
    others = np.arange(D) != 5
    assert np.isfinite(g[..., others]).all()
    assert row_errors(g[..., others], want[..., others]).max() <= ROW_TOL
    first = J // 256 * 256
    assert np.isfinite(g[..., :first, 5]).all()
    assert np.abs(g[..., :first, 5] - want[..., :first, 5]).max() <= TOL["bf16"] * np.abs(want).max()
    assert not np.isfinite(g[..., J:, 5]).any()  # every row from J on attends key J with a positive weight
    if special == np.inf:
        assert np.all(g[..., J:, 5] == np.inf)
    elif special == -np.inf:
        assert np.all(g[..., J:, 5] == -np.inf)


@pytest.mark.parametrize("shape", SHAPES, ids=IDS)
def test_zero_values_give_zeros(lm, hip, oracle, shape):
    B, H, S, D, causal = shape
    q, k, v, heads = setup(lm, oracle, shape, 99300 + D)
    v[:] = 0.0
    v[:, 1] = -0.0
    got = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
    assert np.all(got == 0.0)
    # one head with values, its neighbours all zero: nothing leaks between heads
    q, k, v, heads = setup(lm, oracle, shape, 99310 + D)
    v[:, 1:] = 0.0
    got = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
    assert np.all(got[:, 1:] == 0.0)
    want = oracle.flash_attn(q[:, :1], k[:, :1], v[:, :1], causal=causal, nthreads=NT)
    assert rel_err(got[:, :1], want) <= TOL["bf16"]


def test_long_row_random_shapes(lm, hip, oracle):
    """Shapes drawn until at least 16 of them reach the fp16-V form (the plan query says which do) and all three tilings
    have been seen with and without the mask: head dims on all three tilings,
    GQA groups and head maps, ragged key counts with a NaN tail, with and without the mask, V scaled by a random power of
    two per (batch, KV head), bf16 and fp32 outputs."""
    rng = np.random.default_rng(99500)
    done, tried, reached = 0, 0, set()
    while (done < 16 or len(reached) < 6) and done < 40 and tried < 4000:
        tried += 1
        D = int(rng.choice([16, 40, 64, 72, 80, 96, 96, 104, 128]))
        G = int(rng.choice([1, 1, 2, 4]))
        Hkv = int(rng.integers(1, 17))
        Hq = Hkv * G
        B = int(rng.integers(1, 5))
        causal = bool(rng.integers(2))
        Sq = int(rng.integers(129, 3001))
        Sk = Sq if causal and rng.integers(2) else int(rng.integers(600, 3001))
        if B * Hq * Sq * Sk * D > 4e11:
            continue
        plan = lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), "bf16", causal)
        if not plan.endswith("V as fp16"):
            continue
        head_map = int(rng.integers(2))
        lens = None if rng.integers(2) == 0 else rng.integers(0, Sk + 1, size=B).astype(np.int32)
        out_f32 = bool(rng.integers(2))
        what = "case %d: B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d causal=%s head_map=%d kv_len=%s out_f32=%s -> %s" % (
            done, B, Hq, Hkv, Sq, Sk, D, causal, head_map, None if lens is None else lens.tolist(), out_f32, plan)
        print(what, flush=True)
        q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), "bf16", 99600 + 3 * done, float(rng.choice([0.5, 1.0, 1.5])))
        v = v * power_of_two(rng.integers(-60, 61, size=(B, Hkv)))[:, :, None, None]
        kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
        got = run_flash(lm, hip, q, kp, vp, "bf16", causal, head_map=head_map, kv_len=lens, out_dtype="f32" if out_f32 else None)
        hq = np.unique(rng.integers(0, Hq, size=min(Hq, 3)))
        kv_of = hq if Hq == Hkv else (hq // G if head_map == 1 else hq % Hkv)
        want_len = None if lens is None else np.maximum(lens, 1)
        want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=causal, kv_len=want_len, nthreads=NT)
        keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
        assert np.isfinite(got).all(), what
        # every (batch, head) against its own scale: the heads' values differ by up to 2^120
        tol = TOL["bf16"] if out_f32 else 2.0 ** -8 + TOL["bf16"]  # (a bf16 result is rounded once more)
        for b in keep:
            for i, h in enumerate(hq):
                err = rel_err(got[b, h], want[b, i])
                assert err <= tol, "%s: batch %d head %d rel err %.3g" % (what, b, h, err)
        if lens is not None:
            for b in np.nonzero(lens == 0)[0]:
                assert np.all(got[b] == 0), what
        reached.add((plan.split("<")[1].split(",")[1].strip(), causal))
        done += 1
    print("cases:", done, "tilings and masks covered:", sorted(reached), flush=True)
    assert len(reached) == 6, reached


@pytest.mark.parametrize("shape", SHAPES, ids=IDS)
def test_repeated_launches_give_the_same_bits(lm, hip, oracle, shape):
    """The workgroup agrees on the largest value of a tile through two LDS words and a barrier. With a random power of
    two per key (threads post new maxima in most tiles) ten launches must return the same bits, and the right values."""
    B, H, S, D, causal = shape
    q, k, v, heads = setup(lm, oracle, shape, 99400 + D)
    v = v * power_of_two(np.random.default_rng(99401).integers(-30, 31, size=(B, H, S)))[..., None]
    first = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
    for _ in range(9):
        again = run_flash(lm, hip, q, k, v, "bf16", causal, out_dtype="f32")
        np.testing.assert_array_equal(first.view(np.uint32), again.view(np.uint32))
    # (neighbouring keys differ by up to 2^60 here, more than the 2^29 a tile holds: the contract's tensor-wide metric, not the rows')
    want = oracle.flash_attn(q[:, heads], k[:, heads], v[:, heads], causal=causal, nthreads=NT)
    assert rel_err(first[:, heads], want) <= TOL["bf16"]
