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
