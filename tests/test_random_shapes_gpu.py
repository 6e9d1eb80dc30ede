"""Seeded sweeps over shapes nobody picked by hand: every case is drawn from a fixed generator, run through the C ABI and
compared with the CPU oracle to the contract's tolerance. The sweeps report which kernels the cases reached."""
import numpy as np
import pytest

from conftest import TOL, rel_err
from test_parity_gpu import inputs, run_decode, run_flash

pytestmark = pytest.mark.gpu

NT = 16
HEADS = [(1, 1), (4, 4), (8, 2), (6, 3), (12, 4), (5, 1)]


def poison_tail(k, v, lens):
    kp, vp = k.copy(), v.copy()
    for b, n in enumerate(lens):
        kp[b, :, n:] = np.nan
        vp[b, :, n:] = np.nan
    return kp, vp


def test_prefill_random_shapes(lm, hip, oracle):
    reached = {}
    for case in range(56):
        rng = np.random.default_rng(91000 + case)
        dtype = ["f32", "f16", "bf16"][case % 3]
        D = int(rng.choice([8, 16, 24, 40, 64, 72, 80, 96, 104, 128, 136, 192]))
        Hq, Hkv = HEADS[int(rng.integers(len(HEADS)))]
        B = int(rng.integers(1, 4))
        causal = bool(rng.integers(2))
        Sq = int(rng.integers(1, 301))
        Sk = Sq if causal else int(rng.integers(1, 701))
        head_map = int(rng.integers(2))
        lens = None if rng.integers(3) == 0 else rng.integers(1, Sk + 1, size=B).astype(np.int32)
        plan = lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, causal)
        what = "case %d: %s B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d causal=%s head_map=%d kv_len=%s -> %s" % (
            case, dtype, B, Hq, Hkv, Sq, Sk, D, causal, head_map, None if lens is None else lens.tolist(), plan)
        print(what, flush=True)
        q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 92000 + 3 * case, float(rng.choice([0.5, 1.0, 2.0])))
        kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
        got = run_flash(lm, hip, q, kp, vp, dtype, causal, head_map=head_map, kv_len=lens)
        want = oracle.flash_attn(q, k, v, causal=causal, head_map=head_map, kv_len=lens, nthreads=NT)
        err = rel_err(got, want)
        assert err <= TOL[dtype], "%s: rel err %.3g" % (what, err)
        reached[plan.split("<")[0]] = reached.get(plan.split("<")[0], 0) + 1
    print("kernels reached:", reached, flush=True)
    assert {"prefill_f32_kernel", "prefill_mfma_kernel", "prefill_valu_kernel"} <= set(reached)


def test_decode_random_shapes(lm, hip, oracle):
    for case in range(48):
        rng = np.random.default_rng(93000 + case)
        dtype = ["f32", "f16", "bf16"][case % 3]
        D = int(rng.choice([8, 40, 64, 96, 128, 256]))
        Hq, Hkv = HEADS[int(rng.integers(len(HEADS)))]
        B = int(rng.integers(1, 6))
        Lmax = int(rng.integers(1, 3001))
        splits = int(rng.choice([0, 0, 1, 2, 5]))
        head_map = int(rng.integers(2))
        lens = None if rng.integers(4) == 0 else rng.integers(0, Lmax + 1, size=B).astype(np.int32)
        what = "case %d: %s B=%d Hq=%d Hkv=%d Lmax=%d D=%d splits=%d head_map=%d kv_len=%s" % (
            case, dtype, B, Hq, Hkv, Lmax, D, splits, head_map, None if lens is None else lens.tolist())
        print(what, flush=True)
        q = oracle.round_to(oracle.gen_normal((B, Hq, D), 94000 + 3 * case), dtype)
        k = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 94001 + 3 * case), dtype)
        v = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 94002 + 3 * case), dtype)
        kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
        got = run_decode(lm, hip, q, kp, vp, dtype, kv_len=lens, head_map=head_map, num_splits=splits)
        want_len = None if lens is None else np.maximum(lens, 1)
        want = oracle.decode_attn(q, k, v, kv_len=want_len, head_map=head_map, nthreads=NT)
        keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
        assert np.isfinite(got).all(), what
        if len(keep):
            err = rel_err(got[keep], want[keep])
            assert err <= TOL[dtype], "%s: rel err %.3g" % (what, err)
        if lens is not None:
            for b in np.nonzero(lens == 0)[0]:
                assert np.all(got[b] == 0), what  # a sequence without keys is written as zeros


def test_wide_workgroup_random_shapes(lm, hip, oracle):
    """Shapes drawn until 24 of them reach the one-workgroup-per-CU kernel (the plan query says which do): row-block
    counts, key-group counts, ragged lengths and head dims nobody picked by hand."""
    rng = np.random.default_rng(95000)
    done, tried = 0, 0
    seen = set()
    while done < 24 and tried < 4000:
        tried += 1
        dtype = ["f16", "bf16"][int(rng.integers(2))]
        D = int(rng.choice([16, 32, 40, 64, 72, 88, 96]))
        G = int(rng.choice([1, 1, 2, 4]))
        Hkv = int(rng.integers(1, 33))
        B = int(rng.integers(1, 9))
        Hq = Hkv * G
        Sq = int(rng.integers(64, 601))
        Sk = int(rng.integers(640, 2501))
        if B * Hq > 256 or B * Hq * Sq * Sk * D > 6e9:
            continue
        plan = lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, False)
        if "prefill_mfma_wide_kernel" not in plan:
            continue
        key = plan.split("workgroups per head")[1]
        if key in seen and rng.integers(3) != 0:  # favour plans not seen yet
            continue
        seen.add(key)
        head_map = int(rng.integers(2))
        lens = None if rng.integers(2) == 0 else rng.integers(0, Sk + 1, size=B).astype(np.int32)
        what = "case %d: %s B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d head_map=%d kv_len=%s -> %s" % (
            done, dtype, B, Hq, Hkv, Sq, Sk, D, head_map, None if lens is None else lens.tolist(), plan)
        print(what, flush=True)
        q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 96000 + 3 * done, float(rng.choice([0.5, 1.0, 1.5])))
        kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
        got = run_flash(lm, hip, q, kp, vp, dtype, False, head_map=head_map, kv_len=lens)
        hq = np.unique(rng.integers(0, Hq, size=min(Hq, 6)))
        kv_of = hq if Hq == Hkv else (hq // G if head_map == 1 else hq % Hkv)
        want_len = None if lens is None else np.maximum(lens, 1)
        want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=False, kv_len=want_len, nthreads=NT)
        keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
        assert np.isfinite(got).all(), what
        if len(keep):
            err = rel_err(got[keep][:, hq], want[keep])
            assert err <= TOL[dtype], "%s: rel err %.3g" % (what, err)
        if lens is not None:
            for b in np.nonzero(lens == 0)[0]:
                assert np.all(got[b] == 0), what
        done += 1
    assert done == 24, "only %d shapes reached the wide kernel" % done
    print("plans covered:", sorted(seen), flush=True)


# (B, Hq, Hkv, Sq, Sk, D, kv_len or None, head_map, causal, what is special)
PAIRED_TILE_CASES = [
    (1, 64, 16, 2048, 2048, 64, None, 0, True, "GQA 4:1, 8 tiles"),
    (1, 64, 16, 2048, 2048, 64, None, 1, True, "the same with the blocked head map"),
    (2, 64, 64, 1024, 1024, 96, [700, 1024], 0, True, "ragged keys, 4 tiles"),
    (2, 64, 64, 1024, 1024, 96, [0, 300], 0, True, "a sequence without keys, one with fewer keys than a tile"),
    (1, 32, 8, 3700, 3700, 80, None, 0, True, "15 tiles (the middle one alone), a partial last tile, head dim padded to 96"),
    (4, 64, 64, 512, 512, 64, None, 0, True, "two tiles: one pair per head"),
    (1, 30, 30, 4000, 4000, 96, None, 0, True, "30 heads on 32 head slots"),
    (1, 32, 32, 4096, 5000, 96, None, 0, True, "more keys than queries"),
    (1, 32, 32, 4096, 3000, 96, None, 0, True, "fewer keys than queries"),
    (1, 32, 32, 4096, 4096, 40, [2500], 0, True, "head dim 40 on the 64 tiling, keys end inside the late tiles"),
    # without a mask: two neighbouring tiles per workgroup, whole rounds only
    (1, 32, 8, 4000, 1500, 64, None, 0, False, "no mask: GQA, a partial last tile, keys not a multiple of the tile"),
    (2, 64, 64, 1000, 700, 80, [1, 699], 1, False, "no mask: one key; ragged; head dim padded to 96"),
    (1, 32, 32, 3600, 2000, 96, None, 0, False, "no mask: 15 tiles, the last workgroup of a head has one tile"),
    (1, 30, 10, 3900, 4500, 96, [0], 0, False, "no mask: a sequence without keys"),
    (1, 32, 32, 8192, 1100, 96, None, 0, False, "no mask: two rounds"),
]


PAIRED_TILE_CASES_BF16 = [
    (1, 64, 16, 2048, 2048, 64, None, 0, True, "bf16: GQA 4:1, 8 tiles"),
    (1, 32, 32, 3800, 3800, 40, [2500], 0, True, "bf16: head dim 40 on the 64 tiling, 15 tiles, keys end inside the late tiles"),
    (4, 64, 64, 512, 512, 64, [512, 0, 77, 300], 1, True, "bf16: two tiles, ragged"),
]


@pytest.mark.parametrize("case", PAIRED_TILE_CASES_BF16, ids=lambda c: "B%d-H%d:%d-S%dx%d-D%d" % c[:6])
def test_bf16_on_paired_tile_launch_shapes(lm, hip, oracle, case):
    """bf16 launches of the shapes that take the paired-tile kernel in fp16: they stay on the one-tile workgroups, which
    rewrite V as fp16 on its way into LDS."""
    B, Hq, Hkv, Sq, Sk, D, lens, head_map, causal, what = case
    plan = lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), "bf16", causal)
    print(what, "->", plan, flush=True)
    assert "prefill_mfma_kernel<bf16" in plan and "key groups=1" in plan, plan
    lens = None if lens is None else np.asarray(lens, np.int32)
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), "bf16", 97500 + Sq + D, 0.7)
    kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
    got = run_flash(lm, hip, q, kp, vp, "bf16", causal, head_map=head_map, kv_len=lens)
    hq = np.unique(np.concatenate([[0, Hq - 1], np.random.default_rng(97501).integers(0, Hq, size=4)]))
    G = Hq // Hkv
    kv_of = hq if Hq == Hkv else (hq // G if head_map == 1 else hq % Hkv)
    want_len = None if lens is None else np.maximum(lens, 1)
    want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=causal, kv_len=want_len, nthreads=NT)
    keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
    assert np.isfinite(got).all(), what
    err = rel_err(got[keep][:, hq], want[keep])
    assert err <= TOL["bf16"], "%s: rel err %.3g" % (what, err)
    if lens is not None:
        for b in np.nonzero(lens == 0)[0]:
            assert np.all(got[b] == 0), what


@pytest.mark.parametrize("case", PAIRED_TILE_CASES, ids=lambda c: "B%d-H%d:%d-S%dx%d-D%d-%s" % (c[:6] + ("causal" if c[8] else "full",)))
@pytest.mark.parametrize("out_f32", [False, True])
def test_paired_tile_kernel(lm, hip, oracle, case, out_f32):
    """fp16 launches that are whole rounds of paired 256-row query tiles (causal: tile p with tile n - 1 - p in one
    workgroup, the early tile stored half way; no mask: two neighbouring tiles) against the oracle; the plan query
    confirms the kernel."""
    B, Hq, Hkv, Sq, Sk, D, lens, head_map, causal, what = case
    plan = lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), "f16", causal)
    print(what, "->", plan, flush=True)
    assert "prefill_mfma_pair_kernel" in plan and ("causal" if causal else "full") in plan, plan
    lens = None if lens is None else np.asarray(lens, np.int32)
    q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), "f16", 97000 + Sq + D, 0.7)
    kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
    got = run_flash(lm, hip, q, kp, vp, "f16", causal, head_map=head_map, kv_len=lens, out_dtype="f32" if out_f32 else None)
    rng = np.random.default_rng(97001)
    hq = np.unique(np.concatenate([[0, Hq - 1], rng.integers(0, Hq, size=4)]))
    G = Hq // Hkv
    kv_of = hq if Hq == Hkv else (hq // G if head_map == 1 else hq % Hkv)
    want_len = None if lens is None else np.maximum(lens, 1)
    want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=causal, kv_len=want_len, nthreads=NT)
    keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
    assert np.isfinite(got).all(), what
    if len(keep):
        err = rel_err(got[keep][:, hq], want[keep])
        assert err <= TOL["f16"], "%s: rel err %.3g" % (what, err)
    if lens is not None:
        for b in np.nonzero(lens == 0)[0]:
            assert np.all(got[b] == 0), what


def test_paired_tile_random_shapes(lm, hip, oracle):
    """Shapes drawn so that the launch is exactly one round of paired tiles (heads x pairs = 256 on a 256-CU device):
    tile counts from 2 to 32 (odd ones included), partial last tiles, head dims, GQA groups, head maps, ragged keys,
    with and without the mask (fp16: bf16 launches never take this kernel)."""
    rng = np.random.default_rng(98000)
    done, tried, reached = 0, 0, set()
    while done < 16 and tried < 2000:
        tried += 1
        pairs = int(rng.choice([1, 2, 4, 8, 16, 32]))
        heads = 256 // pairs
        n_tiles = 2 * pairs - int(rng.integers(2))
        if n_tiles < 2:
            continue
        Sq = int(rng.integers((n_tiles - 1) * 256 + 1, n_tiles * 256 + 1))
        causal = bool(rng.integers(2))
        dtype = "f16"
        D = int(rng.choice([16, 32, 40, 64, 72, 88, 96]))
        G = int(rng.choice([1, 1, 2, 4]))
        B = int(rng.choice([b for b in (1, 2, 4) if heads % b == 0 and (heads // b) % G == 0]))
        Hq = heads // B - int(rng.integers(0, 2)) * G  # (sometimes fewer heads than head slots)
        if Hq < G or (B * Hq + 7) // 8 * 8 != heads:
            continue
        Hkv = Hq // G
        Sk = int(rng.integers(max(1, Sq // 3), Sq + 600))
        if B * Hq * Sq * Sk * D > 3e11:
            continue
        plan = lm.flash_attention_plan((B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, causal)
        if "prefill_mfma_pair_kernel" not in plan:
            continue
        head_map = int(rng.integers(2))
        lens = None if rng.integers(2) == 0 else rng.integers(0, Sk + 1, size=B).astype(np.int32)
        what = "case %d: %s B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d causal=%s head_map=%d kv_len=%s -> %s" % (
            done, dtype, B, Hq, Hkv, Sq, Sk, D, causal, head_map, None if lens is None else lens.tolist(), plan)
        print(what, flush=True)
        q, k, v = inputs(oracle, (B, Hq, Sq, D), (B, Hkv, Sk, D), dtype, 98100 + 3 * done, float(rng.choice([0.5, 1.0, 1.5])))
        kp, vp = (k, v) if lens is None else poison_tail(k, v, lens)
        got = run_flash(lm, hip, q, kp, vp, dtype, causal, head_map=head_map, kv_len=lens)
        hq = np.unique(rng.integers(0, Hq, size=min(Hq, 3)))
        kv_of = hq if Hq == Hkv else (hq // G if head_map == 1 else hq % Hkv)
        want_len = None if lens is None else np.maximum(lens, 1)
        want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=causal, kv_len=want_len, nthreads=NT)
        keep = np.arange(B) if lens is None else np.nonzero(lens > 0)[0]
        assert np.isfinite(got).all(), what
        if len(keep):
            err = rel_err(got[keep][:, hq], want[keep])
            assert err <= TOL[dtype], "%s: rel err %.3g" % (what, err)
        if lens is not None:
            for b in np.nonzero(lens == 0)[0]:
                assert np.all(got[b] == 0), what
        reached.add((dtype, causal))
        done += 1
    assert done == 16, "only %d shapes reached the paired-tile kernel" % done
    assert {("f16", True), ("f16", False)} <= reached
