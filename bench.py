#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only all|prefill|decode|other|c1|nomask|bf16|c3|c4|ops|step|copy|ceiling|grid|shapes]

A step is one pass of the hot path over one batch of synthetic input, inputs resident in HBM:
  prefill leg (the headline `value`): causal flash attention, Phi-3-mini shape
      B=1, Hq=Hkv=32, S=4096, D=96, fp16 in/out, fp32 accumulate        -> TFLOP/s, MFMA roofline
  decode leg (reported under "decode"): split-KV GQA decode, long ragged batch
      B=64, Hq=32, Hkv=8, D=128, bf16, kv_len ~ U[8192, 32768]          -> GB/s, HBM roofline
Other configurations of the contract (fp32 S=128, Whisper cross attention, B=16 L=4096 decode) are
timed briefly and listed under "other_configs".

Algorithmic work: prefill FLOPs = 4*B*Hq*D*S*(S+1)/2 (2 flops per MAC, QK^T and PV, unmasked pairs
only); decode bytes = 2 * sum_b kv_len[b] * Hkv * D * 2 (K and V once per KV head) + q + out.

Kernel time is measured with HIP events on the launch stream around the timed steps; the CPU
baseline is the oracle (a C restatement of the reference's flash_attn_cpu) on a bounded sample of
the same workload, whose output also serves as a parity check of the GPU result.
Inputs come from the package's seeded generator (SplitMix64 -> Box-Muller, luminal.jl_amd/synth.py) with the
seeds the parity tests use for the same configurations; they are generated before any timed region.
One JSON line on stdout; progress on stderr.
"""
import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_TFLOPS = 157.3  # dense fp32 MFMA
PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16/bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# HBM-side bytes per launch (`roofline.traffic`) come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# script, each scaled by what the same counter reads for the calibration copy kernel (--only copy). Counters
# cannot be read from inside a timed run, so the figures live in profiles/traffic.json next to the summaries they
# were taken from, each with the hash of the kernel source it was measured on; a figure whose kernel source has
# changed since is reported as null rather than as a stale number.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def source_hash(*names):
    h = hashlib.sha256()
    for n in names:
        with open(os.path.join(ROOT, "luminal.jl_amd", "csrc", n), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(key):
    """HBM bytes per launch recorded for `key`, or None when there is no record for the current kernel source."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)[key]
        if rec["source_sha16"] != source_hash(*rec["sources"]):
            log("[bench] %s: %s changed since the counters were read; traffic reported as null" % (key, rec["sources"]))
            return None
        return float(rec["fetch_bytes"]) + float(rec["write_bytes"])
    except (OSError, KeyError, ValueError):
        return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# The GPU raises its clocks over the first tens of milliseconds of load: from idle, C2 measured 141 us per launch
# over the first 20 launches and 118 us from the 100th on. Every timed region is therefore preceded by this much
# untimed work of the same kind (on top of the --warmup steps), so that what is timed is the steady state.
CLOCK_SETTLE_MS = 100.0


def settle_clocks(fn, binding, ms=CLOCK_SETTLE_MS):
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            fn()
        binding.sync()


def time_steps(fn, steps, warmup, binding, settle_ms=CLOCK_SETTLE_MS):
    """Clock settling, `warmup` untimed calls, then `steps` timed calls bracketed by a device sync on both
    sides. Returns (wall ms per step, HIP-event ms per step)."""
    if settle_ms > 0:
        settle_clocks(fn, binding, settle_ms)
    for _ in range(warmup):
        fn()
    binding.sync()
    e0, e1 = binding.Event(), binding.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    binding.sync()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e1.elapsed_ms_since(e0) / steps


def per_launch_us(fn, n, binding):
    """Median and minimum of n launches timed one by one with HIP events (after the main timed region)."""
    evs = [(binding.Event(), binding.Event()) for _ in range(n)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    binding.sync()
    us = sorted(b.elapsed_ms_since(a) * 1e3 for a, b in evs)
    return {"median": us[len(us) // 2], "min": us[0], "n": n}


def attn_params(lm, out, q, k, v, dtype, causal, scale, head_map=0, kv_len=None):
    p = lm.binding.AttnParams()
    p.out, p.q, p.k, p.v = out.ptr, q.ptr, k.ptr, v.ptr
    p.kv_len = kv_len.ptr if kv_len is not None else None
    p.B, p.Hq, p.Sq, p.D = q.shape
    p.Hkv, p.Sk = k.shape[1], k.shape[2]
    p.dtype = lm.binding.DTYPE_CODES[dtype]
    p.scale, p.causal, p.head_map = scale, int(causal), head_map
    p.out_f32 = int(out.dtype == "f32")
    return p


def decode_params(lm, out, q, kc, vc, kv_len, dtype, scale, ws, head_map=0, num_splits=0):
    b = lm.binding
    p = b.DecodeParams()
    p.out, p.q, p.k_cache, p.v_cache = out.ptr, q.ptr, kc.ptr, vc.ptr
    p.kv_len = kv_len.ptr if kv_len is not None else None
    p.B, p.Hq, p.D = q.shape
    p.Hkv, p.Lmax = kc.shape[1], kc.shape[2]
    p.dtype = b.DTYPE_CODES[dtype]
    p.scale, p.head_map = scale, head_map
    p.out_f32 = int(out.dtype == "f32")
    p.num_splits = num_splits or b.decode_auto_splits(p.B, p.Hkv, p.Lmax)
    p.workspace, p.workspace_bytes = ws.ptr, ws.nbytes
    return p


def rel_err(got, want):
    return float(np.abs(np.asarray(got, np.float64) - want).max() / np.abs(want).max())


# -------------------------------------------------------------------------------------------------
def prefill_leg(lm, dev, steps, warmup, cpu_seconds, zero_operands=True):
    B, H, S, D = 1, 32, 4096, 96
    host = [lm.synth.normal((B, H, S, D), 2000 + i, 0.5).astype(np.float16) for i in range(3)]  # seeds of the C2 parity test
    dq, dk, dv = (lm.HipArray((B, H, S, D), "f16", dev).copy_from_host(x) for x in host)
    out = lm.HipArray((B, H, S, D), "f16", dev)
    scale = lm.default_scale(D)
    p = attn_params(lm, out, dq, dk, dv, "f16", True, scale)
    fn = lambda: lm.binding.flash_attn_fwd(p)
    wall_ms, ev_ms = time_steps(fn, steps, warmup, lm.binding)
    flops = 4.0 * B * H * D * S * (S + 1) / 2
    tflops = flops / (wall_ms * 1e-3) / 1e12
    kern_tflops = flops / (ev_ms * 1e-3) / 1e12
    log("[prefill] C2 causal fp16 B=1 H=32 S=4096 D=96: %.1f us/step wall, %.1f us/launch events, %.1f TFLOP/s (%.1f%% of %g)"
        % (wall_ms * 1e3, ev_ms * 1e3, kern_tflops, 100 * kern_tflops / PEAK_FP16_TFLOPS, PEAK_FP16_TFLOPS))
    each = per_launch_us(fn, 20, lm.binding)
    sustained = mfma_sustained(lm, dev, dq)
    on_zeros = zero_operand_launch_us(lm, dev, p, (B, H, S, D), "f16", steps, warmup) if zero_operands else None
    if zero_operands:
        log("[prefill] the same launch on all-zero Q, K, V (same instruction stream, no switching in the data paths): %.1f us" % on_zeros)
    res = {
        "ms_per_step": wall_ms, "value": tflops,
        "roofline": {"bound": "mfma", "achieved": kern_tflops, "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": kern_tflops / PEAK_FP16_TFLOPS, "traffic": measured_traffic("prefill_C2"),
                     "kernel": lm.binding.flash_attn_plan(p), "launch_us": ev_ms * 1e3,
                     "algorithmic_flops_per_launch": flops, "launch_us_one_by_one": each,
                     # what a bare MFMA loop sustains on this GPU right now (clock management under load):
                     # on all-zero operands and on the Q tensor of this workload
                     "mfma_sustained_tflops": sustained,
                     "frac_of_sustained": kern_tflops / sustained["workload_operands"],
                     # the same launch (same kernel, grid and instruction stream) on all-zero Q, K and V: what is left
                     # of the difference to launch_us once the handful of rescales is discounted is the clock the
                     # chip grants under the data's switching activity
                     "launch_us_on_zero_operands": on_zeros},
    }
    if cpu_seconds > 0:
        # CPU baseline = the oracle on a head subset of the same workload, all host threads; the same
        # output is the parity check of the GPU result for those heads.
        import oracle
        nthreads = oracle.max_threads()
        got = out.to_host()
        q32, k32, v32 = (x.astype(np.float32) for x in host)
        heads, t_cpu, worst = 0, 0.0, 0.0
        step_heads = 2
        while heads < H and (heads == 0 or t_cpu * (heads + step_heads) / heads < cpu_seconds):
            sl = slice(heads, heads + step_heads)
            t0 = time.perf_counter()
            want = oracle.flash_attn(q32[:, sl], k32[:, sl], v32[:, sl], scale=scale, causal=True, nthreads=nthreads)
            t_cpu += time.perf_counter() - t0
            worst = max(worst, rel_err(got[:, sl], want))
            heads += step_heads
        cpu_tflops = flops * heads / H / t_cpu / 1e12
        log("[prefill] CPU oracle: %d of %d heads in %.1f s on %d threads = %.4f TFLOP/s; GPU vs oracle rel err %.2e"
            % (heads, H, t_cpu, nthreads, cpu_tflops, worst))
        res["cpu_baseline"] = {"value": cpu_tflops, "unit": "TFLOP/s", "cores": nthreads, "kind": "port",
                               "sample": "heads 0..%d of %d, all %d query rows, %.1f s" % (heads - 1, H, S, t_cpu)}
        res["parity"] = {"max_rel_err": worst, "tolerance": 2e-3, "checked": "heads 0..%d vs CPU oracle" % (heads - 1)}
        if worst > 2e-3:
            raise SystemExit("prefill parity check failed: rel err %.3g > 2e-3" % worst)
        # the reference's own execution model is one scalar thread: same oracle, one thread, one head
        t0 = time.perf_counter()
        oracle.flash_attn(q32[:, :1], k32[:, :1], v32[:, :1], scale=scale, causal=True, nthreads=1)
        t1 = time.perf_counter() - t0
        res["cpu_baseline_single_thread"] = {"value": flops / H / t1 / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
                                             "sample": "head 0 of %d, all %d query rows, %.1f s" % (H, S, t1)}
        log("[prefill] CPU oracle, 1 thread: head 0 in %.1f s = %.5f TFLOP/s" % (t1, flops / H / t1 / 1e12))
    return res


def zero_operand_launch_us(lm, dev, p, shape, dtype, steps, warmup):
    """HIP-event time per launch of the attention launch `p` with its Q, K and V replaced by all-zero tensors."""
    zq, zk, zv = (lm.HipArray(shape, dtype, dev).fill_bytes(0) for _ in range(3))
    zo = lm.HipArray(shape, "f32" if p.out_f32 else dtype, dev)  # (the launch's own output stays as it is)
    pz = lm.binding.AttnParams.from_buffer_copy(p)
    pz.q, pz.k, pz.v, pz.out = zq.ptr, zk.ptr, zv.ptr, zo.ptr
    _, ev = time_steps(lambda: lm.binding.flash_attn_fwd(pz), steps, warmup, lm.binding)
    return ev * 1e3


def mfma_sustained(lm, dev, operands):
    """TFLOP/s of lmh_calib_mfma (a bare v_mfma_f32_32x32x16_f16 loop on the whole chip) on zeros and on `operands`."""
    sink = lm.HipArray((512 * 256,), "f32", dev)
    zeros = lm.HipArray((1 << 16,), "f16", dev).fill_bytes(0)
    out = {}
    for name, buf, nbytes in (("zero_operands", zeros, 1 << 17), ("workload_operands", operands, 1 << 17)):
        flops = [0.0]
        def fn():
            flops[0] = lm.binding.calib_mfma(sink.ptr, buf.ptr, nbytes, 40000)
        _, ev = time_steps(fn, 3, 1, lm.binding)
        out[name] = flops[0] / (ev * 1e-3) / 1e12
    log("[prefill] bare MFMA loop sustains %.0f TFLOP/s on zero operands, %.0f TFLOP/s on the workload's Q values (published peak %g)"
        % (out["zero_operands"], out["workload_operands"], PEAK_FP16_TFLOPS))
    return out


def fill_cache_from_pool(lm, cache, pool, lens, Hkv, Lmax, D, rng):
    """cache[b, h, 0:lens[b]] <- a row-aligned window of `pool` (device-to-device); returns the windows."""
    row_bytes = D * 2
    pool_rows = pool.shape[0]
    starts = np.zeros((len(lens), Hkv), np.int64)
    for b, n in enumerate(lens):
        for h in range(Hkv):
            s = int(rng.integers(0, pool_rows - int(n)))
            starts[b, h] = s
            lm.binding.memcpy_d2d(cache.ptr + ((b * Hkv + h) * Lmax) * row_bytes, pool.ptr + s * row_bytes, int(n) * row_bytes)
    return starts


def decode_leg(lm, dev, steps, warmup, cpu_seconds, num_splits=0):
    B, Hq, Hkv, Lmax, D = 64, 32, 8, 32768, 128
    rng = np.random.default_rng(5)  # only picks where in the pools each (sequence, head) slice is taken from
    lens = lm.synth.uniform_int(B, 5000, 8192, 32768)  # the lengths of the C5 parity test
    pool_rows = 1 << 18  # 256 Ki rows of 128 bf16 = 64 MiB per pool
    pools_host = [lm.f32_to_bf16_bits(lm.synth.normal((pool_rows, D), 6000 + i)) for i in range(2)]
    kpool, vpool = (lm.HipArray((pool_rows, D), "bf16", dev).copy_from_host(x) for x in pools_host)
    kc = lm.HipArray((B, Hkv, Lmax, D), "bf16", dev).fill_bytes(0xFF)  # tail past kv_len is NaN
    vc = lm.HipArray((B, Hkv, Lmax, D), "bf16", dev).fill_bytes(0xFF)
    kstart = fill_cache_from_pool(lm, kc, kpool, lens, Hkv, Lmax, D, rng)
    vstart = fill_cache_from_pool(lm, vc, vpool, lens, Hkv, Lmax, D, rng)
    q_host = lm.f32_to_bf16_bits(lm.synth.normal((B, Hq, D), 5001))
    dq = lm.HipArray((B, Hq, D), "bf16", dev).copy_from_host(q_host)
    dl = lm.HipArray((B,), "i32", dev).copy_from_host(lens)
    out = lm.HipArray((B, Hq, D), "f32", dev)
    ws = lm.HipArray((max(lm.binding.decode_workspace_bytes(B, Hq, Hkv, Lmax, D, num_splits) // 4, 4),), "f32", dev)
    scale = lm.default_scale(D)
    p = decode_params(lm, out, dq, kc, vc, dl, "bf16", scale, ws, num_splits=num_splits)
    fn = lambda: lm.binding.decode_attn(p)
    wall_ms, ev_ms = time_steps(fn, steps, warmup, lm.binding)
    algo_bytes = 2.0 * float(lens.sum()) * Hkv * D * 2 + B * Hq * D * 2 + B * Hq * D * 4
    gbs = algo_bytes / (wall_ms * 1e-3) / 1e9
    kern_gbs = algo_bytes / (ev_ms * 1e-3) / 1e9
    log("[decode] C5 bf16 B=64 Hq=32 Hkv=8 D=128 sum(kv_len)=%d (%.2f GB): %.1f us/step wall, %.1f us events, %.0f GB/s (%.1f%% of %g); %d splits"
        % (int(lens.sum()), algo_bytes / 1e9, wall_ms * 1e3, ev_ms * 1e3, kern_gbs, 100 * kern_gbs / PEAK_HBM_GBS, PEAK_HBM_GBS, p.num_splits))
    res = {
        "workload": "C5 long ragged GQA decode: B=64 Hq=32 Hkv=8 D=128 bf16, kv_len~U[8192,32768], sum=%d" % int(lens.sum()),
        "value": gbs, "unit": "GB/s", "ms_per_step": wall_ms, "num_splits": int(p.num_splits),
        "roofline": {"bound": "hbm", "achieved": kern_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": kern_gbs / PEAK_HBM_GBS,
                     "traffic": measured_traffic("decode_C5") if num_splits == 0 else None,
                     "kernel": "decode_mfma_kernel<Mfma16BF16,128> + decode_merge_kernel",
                     "launch_us": ev_ms * 1e3, "algorithmic_bytes_per_launch": algo_bytes,
                     "launch_us_one_by_one": per_launch_us(fn, 20, lm.binding)},
    }
    if cpu_seconds > 0:
        import oracle
        nthreads = oracle.max_threads()
        got = out.to_host()
        qf = lm.bf16_bits_to_f32(q_host)
        kp32, vp32 = (lm.bf16_bits_to_f32(x) for x in pools_host)
        done, t_cpu, worst, bytes_done = 0, 0.0, 0.0, 0.0
        while done < B and (done == 0 or t_cpu * (done + 1) / done < cpu_seconds):
            b, n = done, int(lens[done])
            kb = np.stack([kp32[kstart[b, h]:kstart[b, h] + n] for h in range(Hkv)])[None]
            vb = np.stack([vp32[vstart[b, h]:vstart[b, h] + n] for h in range(Hkv)])[None]
            t0 = time.perf_counter()
            want = oracle.decode_attn(qf[b:b + 1], kb, vb, scale=scale, nthreads=nthreads)
            t_cpu += time.perf_counter() - t0
            worst = max(worst, rel_err(got[b:b + 1], want))
            bytes_done += 2.0 * n * Hkv * D * 2
            done += 1
        cpu_gbs = bytes_done / t_cpu / 1e9
        log("[decode] CPU oracle: %d of %d sequences in %.2f s on %d threads = %.2f GB/s (bf16-equivalent bytes); rel err %.2e"
            % (done, B, t_cpu, nthreads, cpu_gbs, worst))
        res["cpu_baseline"] = {"value": cpu_gbs, "unit": "GB/s", "cores": nthreads, "kind": "port",
                               "sample": "sequences 0..%d of %d at their full kv_len, %.2f s" % (done - 1, B, t_cpu)}
        res["parity"] = {"max_rel_err": worst, "tolerance": 2e-3, "checked": "sequences 0..%d vs CPU oracle" % (done - 1)}
        if worst > 2e-3:
            raise SystemExit("decode parity check failed: rel err %.3g > 2e-3" % worst)
    for a in (kc, vc, kpool, vpool, ws):
        a.free()
    return res


def flash_config(lm, dev, res, name, B, Hq, Hkv, Sq, Sk, D, dtype, causal, flops, seed, mul=1.0, tol=None, steps=20,
                 peak=None):
    """One flash-attention configuration: 20 timed launches; with `tol`, the whole output against the CPU oracle."""
    hq, hk, hv = (lm.synth.normal(shp, seed + i, mul) for i, shp in enumerate(((B, Hq, Sq, D), (B, Hkv, Sk, D), (B, Hkv, Sk, D))))
    q, k, v = (lm.HipArray(x.shape, dtype, dev).copy_from_host(x) for x in (hq, hk, hv))
    o = lm.HipArray((B, Hq, Sq, D), dtype, dev)
    p = attn_params(lm, o, q, k, v, dtype, causal, lm.default_scale(D))
    fn = lambda: lm.binding.flash_attn_fwd(p)
    _, ev = time_steps(fn, steps, 5, lm.binding)
    res[name] = {"launch_us": ev * 1e3, "TFLOP/s": flops / (ev * 1e-3) / 1e12,
                 "launch_us_one_by_one": per_launch_us(fn, 20, lm.binding), "kernel": lm.binding.flash_attn_plan(p)}
    if peak:
        res[name]["frac_of_mfma_peak"] = res[name]["TFLOP/s"] / peak
    log("[other] %s: %.1f us, %.2f TFLOP/s" % (name, ev * 1e3, res[name]["TFLOP/s"]))
    if tol is not None:
        import oracle
        qh, kh, vh = (np.asarray(x.to_host(), np.float32) for x in (q, k, v))  # the element-type-rounded inputs
        want = oracle.flash_attn(qh, kh, vh, scale=lm.default_scale(D), causal=causal, nthreads=oracle.max_threads())
        err = float(np.max(np.abs(np.asarray(o.to_host(), np.float32) - want)) / np.max(np.abs(want)))
        res[name]["parity"] = {"max_rel_err": err, "tolerance": tol, "checked": "whole output vs CPU oracle"}
        log("[other] %s: GPU vs oracle rel err %.2e (tolerance %g)" % (name, err, tol))


def c1_leg(lm, dev, res, check):
    flash_config(lm, dev, res, "C1 causal fp32 B=1 H=8 S=128 D=64", 1, 8, 8, 128, 128, 64, "f32", True,
                 4.0 * 8 * 64 * 128 * 129 / 2, 1000, tol=1e-5 if check else None)
    # the reference's element type on the C2 shape (an extra line, not one of the five configurations)
    name = "C2 shape in fp32 (causal B=1 H=32 S=4096 D=96)"
    flash_config(lm, dev, res, name, 1, 32, 32, 4096, 4096, 96, "f32", True, 4.0 * 32 * 96 * 4096 * 4097 / 2, 2000, mul=0.5)
    res[name]["frac_of_fp32_mfma_peak"] = res[name]["TFLOP/s"] / PEAK_FP32_TFLOPS


def nomask_leg(lm, dev, res, check, zero_operands=True):
    """The C2 shape without the causal mask (an extra line, not one of the five configurations): every workgroup walks
    all 4096 keys, so the launch is 32 equal tiles per CU and shows the loop's steady state without the diagonal."""
    name = "C2 shape without the mask (fp16 B=1 H=32 S=4096 D=96)"
    B, H, S, D = 1, 32, 4096, 96
    hq, hk, hv = (lm.synth.normal((B, H, S, D), 2000 + i, 0.5) for i in range(3))
    q, k, v = (lm.HipArray(x.shape, "f16", dev).copy_from_host(x) for x in (hq, hk, hv))
    o = lm.HipArray((B, H, S, D), "f16", dev)
    p = attn_params(lm, o, q, k, v, "f16", False, lm.default_scale(D))
    fn = lambda: lm.binding.flash_attn_fwd(p)
    flops = 4.0 * B * H * D * S * S
    _, ev = time_steps(fn, 40, 5, lm.binding)
    res[name] = {"launch_us": ev * 1e3, "TFLOP/s": flops / (ev * 1e-3) / 1e12, "frac_of_mfma_peak": flops / (ev * 1e-3) / 1e12 / PEAK_FP16_TFLOPS,
                 "kernel": lm.binding.flash_attn_plan(p),
                 "launch_us_on_zero_operands": zero_operand_launch_us(lm, dev, p, (B, H, S, D), "f16", 40, 5) if zero_operands else None}
    log("[other] %s: %.1f us, %.1f TFLOP/s; on zero operands %s us; %s" % (name, ev * 1e3, res[name]["TFLOP/s"],
                                                                         res[name]["launch_us_on_zero_operands"], res[name]["kernel"]))
    if check:
        import oracle
        heads = slice(0, 4)
        qh, kh, vh = (np.asarray(x.to_host(), np.float32)[:, heads] for x in (q, k, v))
        want = oracle.flash_attn(qh, kh, vh, scale=lm.default_scale(D), causal=False, nthreads=oracle.max_threads())
        err = rel_err(np.asarray(o.to_host(), np.float32)[:, heads], want)
        res[name]["parity"] = {"max_rel_err": err, "tolerance": 2e-3, "checked": "heads 0..3 vs CPU oracle"}
        log("[other] %s: GPU vs oracle rel err %.2e" % (name, err))
        if err > 2e-3:
            raise SystemExit("parity check failed on %s: rel err %.3g > 2e-3" % (name, err))


def bf16_leg(lm, dev, res, check):
    """The C2 shape in bf16 (an extra line, not one of the five configurations): the element type of most models' prompts.
    The kernel rewrites V as fp16 on its way into LDS and rounds the weights to fp16; parity against the oracle's bf16
    inputs on four heads."""
    name = "C2 shape in bf16 (causal B=1 H=32 S=4096 D=96)"
    B, H, S, D = 1, 32, 4096, 96
    hq, hk, hv = (lm.synth.normal((B, H, S, D), 2000 + i, 0.5) for i in range(3))
    q, k, v = (lm.HipArray(x.shape, "bf16", dev).copy_from_host(x) for x in (hq, hk, hv))
    o = lm.HipArray((B, H, S, D), "bf16", dev)
    p = attn_params(lm, o, q, k, v, "bf16", True, lm.default_scale(D))
    flops = 4.0 * B * H * D * S * (S + 1) / 2
    _, ev = time_steps(lambda: lm.binding.flash_attn_fwd(p), 40, 5, lm.binding)
    res[name] = {"launch_us": ev * 1e3, "TFLOP/s": flops / (ev * 1e-3) / 1e12, "frac_of_mfma_peak": flops / (ev * 1e-3) / 1e12 / PEAK_FP16_TFLOPS,
                 "kernel": lm.binding.flash_attn_plan(p)}
    log("[other] %s: %.1f us, %.1f TFLOP/s; %s" % (name, ev * 1e3, res[name]["TFLOP/s"], res[name]["kernel"]))
    if check:
        import oracle
        heads = slice(0, 4)
        qh, kh, vh = (np.asarray(x.to_host(), np.float32)[:, heads] for x in (q, k, v))
        want = oracle.flash_attn(qh, kh, vh, scale=lm.default_scale(D), causal=True, nthreads=oracle.max_threads())
        err = rel_err(np.asarray(o.to_host(), np.float32)[:, heads], want)
        res[name]["parity"] = {"max_rel_err": err, "tolerance": 2e-3, "checked": "heads 0..3 vs CPU oracle"}
        log("[other] %s: GPU vs oracle rel err %.2e" % (name, err))
        if err > 2e-3:
            raise SystemExit("parity check failed on %s: rel err %.3g > 2e-3" % (name, err))


def shapes_leg(lm, dev, spec):
    """Any flash-attention launches by shape (--only shapes --shapes B,Hq,Hkv,Sq,Sk,D,dtype,causal|full[;...]): µs per
    launch, TFLOP/s and the kernel reached, for comparing two builds of the library (the measurement switches of the
    kernels) on shapes that are not contract configurations."""
    res = {}
    for item in spec.split(";"):
        f = item.split(",")
        B, Hq, Hkv, Sq, Sk, D = (int(x) for x in f[:6])
        dtype, causal = f[6], f[7] == "causal"
        flops = 4.0 * B * Hq * D * (Sq * (Sq + 1) / 2 if causal and Sq == Sk else Sq * Sk)
        steps = 40 if flops < 4e11 else 12
        flash_config(lm, dev, res, item, B, Hq, Hkv, Sq, Sk, D, dtype, causal, flops, 7000, mul=0.5, steps=steps, peak=PEAK_FP16_TFLOPS)
        res[item].pop("launch_us_one_by_one", None)
    return res


def c3_leg(lm, dev, res, check):
    flash_config(lm, dev, res, "C3 cross fp16 B=4 H=20 Sq=448 Sk=1500 D=64", 4, 20, 20, 448, 1500, 64, "f16", False,
                 4.0 * 4 * 20 * 448 * 1500 * 64, 3000, tol=2e-3 if check else None, steps=40, peak=PEAK_FP16_TFLOPS)


def c4_caches(lm, dev):
    """C4's caches, four times over: 268 MB would sit in the 256 MB last-level cache, so launches rotate over 4 copies
    (each a different roll of the same seeded pool)."""
    B, Hkv, L, D = 16, 8, 4096, 128
    pool = lm.f32_to_bf16_bits(lm.synth.normal((B * Hkv * L, D), 4001))
    caches = []
    for i in range(4):
        kc = lm.HipArray((B, Hkv, L, D), "bf16", dev).copy_from_host(np.roll(pool, 977 * i, axis=0))
        vc = lm.HipArray((B, Hkv, L, D), "bf16", dev).copy_from_host(np.roll(pool, 977 * i + 401, axis=0))
        caches.append((kc, vc))
    return caches


def c4_leg(lm, dev, res, check, caches=None):
    B, Hq, Hkv, L, D = 16, 32, 8, 4096, 128
    caches = caches or c4_caches(lm, dev)
    q = lm.HipArray((B, Hq, D), "bf16", dev).copy_from_host(lm.synth.normal((B, Hq, D), 4000))
    o = lm.HipArray((B, Hq, D), "f32", dev)
    ws = lm.HipArray((max(lm.binding.decode_workspace_bytes(B, Hq, Hkv, L, D, 0) // 4, 4),), "f32", dev)
    ps = [decode_params(lm, o, q, kc, vc, None, "bf16", lm.default_scale(D), ws) for kc, vc in caches]
    state = {"i": 0}

    def step():
        lm.binding.decode_attn(ps[state["i"] % 4])
        state["i"] += 1

    _, ev = time_steps(step, 40, 8, lm.binding)
    nbytes = 2.0 * B * L * Hkv * D * 2 + B * Hq * D * 6
    name = "C4 decode bf16 B=16 Hq=32 Hkv=8 L=4096 D=128 (4 caches rotated)"
    res[name] = {"launch_us": ev * 1e3, "GB/s": nbytes / (ev * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ev * 1e-3) / 1e9 / PEAK_HBM_GBS,
                 "num_splits": int(ps[0].num_splits), "launch_us_one_by_one": per_launch_us(step, 20, lm.binding)}
    log("[other] C4 decode: %.1f us, %.0f GB/s, %d splits" % (ev * 1e3, nbytes / (ev * 1e-3) / 1e9, ps[0].num_splits))
    # what a kernel that only reads 268 MB takes, launch included (four buffers in rotation, like the caches): the
    # ceiling of any decode kernel at this size
    sink = lm.HipArray((4,), "f32", dev)
    total = 2 * B * Hkv * L * D * 2
    probes = [lm.HipArray((total // 4,), "f32", dev).fill_bytes(1) for _ in range(4)]

    def read_step():
        lm.binding.calib_read(probes[state["i"] % 4].ptr, total, sink.ptr)
        state["i"] += 1

    _, evr = time_steps(read_step, 40, 8, lm.binding)
    res[name]["plain_read_of_the_same_bytes_us"] = evr * 1e3
    res[name]["frac_of_plain_read_rate"] = evr / ev
    for pb in probes:
        pb.free()
    log("[other] plain read of 268 MB in one launch: %.1f us, %.0f GB/s" % (evr * 1e3, total / (evr * 1e-3) / 1e9))
    if check:
        import oracle
        lm.binding.decode_attn(ps[0])
        qh = np.asarray(q.to_host(), np.float32)
        kh, vh = (np.asarray(x.to_host(), np.float32) for x in caches[0])
        want = oracle.decode_attn(qh, kh, vh, scale=lm.default_scale(D), nthreads=oracle.max_threads())
        err = float(np.max(np.abs(np.asarray(o.to_host(), np.float32) - want)) / np.max(np.abs(want)))
        res[name]["parity"] = {"max_rel_err": err, "tolerance": 2e-3, "checked": "whole output vs CPU oracle"}
        log("[other] C4 decode: GPU vs oracle rel err %.2e (tolerance 2e-3)" % err)
    return caches


def ops_leg(lm, dev, res, caches=None):
    """The two operators in front of attention: rotary embedding of a prompt's Q, and the cache append (K rotated on
    the way in) for a whole prompt and for one decode step. Algorithmic bytes = every element read once, written once."""
    def hbm_line(name, fn, nbytes, n=20):
        _, ev = time_steps(fn, n, 5, lm.binding)
        res[name] = {"launch_us": ev * 1e3, "GB/s": nbytes / (ev * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (ev * 1e-3) / 1e9 / PEAK_HBM_GBS}
        log("[other] %s: %.1f us, %.0f GB/s" % (name, ev * 1e3, res[name]["GB/s"]))

    B, H, S, D = 1, 32, 4096, 96
    # 12 inputs of 25 MB in rotation, more than the 256 MB last-level cache holds: every launch reads from HBM
    x0 = lm.synth.normal((B, H, S, D), 2000, 0.5)
    xs = [lm.HipArray((B, H, S, D), "f16", dev).copy_from_host(np.roll(x0, 131 * i, axis=2)) for i in range(12)]
    y = lm.HipArray((B, H, S, D), "f16", dev)
    rps = []
    for x in xs:
        rp = lm.binding.RopeParams()
        rp.out, rp.x, rp.pos0, rp.prev_seq = y.ptr, x.ptr, None, 0
        rp.B, rp.H, rp.S, rp.D = B, H, S, D
        rp.dtype, rp.base, rp.pairing, rp.stream = lm.binding.DTYPE_CODES["f16"], 10000.0, lm.binding.ROPE_HALF_SPLIT, None
        rps.append(rp)
    rstate = {"i": 0}

    def rope_step():
        lm.binding.rope(rps[rstate["i"] % len(rps)])
        rstate["i"] += 1

    hbm_line("rotary embedding fp16 B=1 H=32 S=4096 D=96 (C2's Q, 12 inputs rotated)", rope_step, 2.0 * B * H * S * D * 2, n=36)

    def copy_step():  # the same bytes through the plain copy kernel: what this size allows (ramp-up is a third of it)
        lm.binding.calib_copy(y.ptr, xs[rstate["i"] % len(xs)].ptr, B * H * S * D * 2)
        rstate["i"] += 1

    hbm_line("plain copy of the same 25 MB (reference for the line above)", copy_step, 2.0 * B * H * S * D * 2, n=36)

    # The prompt path of an attention layer on the C2 shape (reference src/NN.jl:357-382: rotary embedding of q and k,
    # then attention): three launches, against two with the queries rotated inside the attention kernel.
    q, k = xs[0], xs[1]
    v = lm.HipArray((B, H, S, D), "f16", dev).copy_from_host(lm.synth.normal((B, H, S, D), 2001, 0.5))
    qr, kr = lm.HipArray((B, H, S, D), "f16", dev), lm.HipArray((B, H, S, D), "f16", dev)
    o = lm.HipArray((B, H, S, D), "f16", dev)

    def rope_params(dst, src):
        rp = lm.binding.RopeParams()
        rp.out, rp.x, rp.pos0, rp.prev_seq = dst.ptr, src.ptr, None, 0
        rp.B, rp.H, rp.S, rp.D = B, H, S, D
        rp.dtype, rp.base, rp.pairing, rp.stream = lm.binding.DTYPE_CODES["f16"], 10000.0, lm.binding.ROPE_HALF_SPLIT, None
        return rp

    rq, rk = rope_params(qr, q), rope_params(kr, k)
    plain = attn_params(lm, o, qr, kr, v, "f16", True, lm.default_scale(D))
    fused = attn_params(lm, o, q, kr, v, "f16", True, lm.default_scale(D))
    fused.q_rope, fused.q_rope_pairing, fused.q_prev_seq, fused.q_rope_base = 1, lm.binding.ROPE_HALF_SPLIT, 0, 10000.0

    def three_launches():
        lm.binding.rope(rq)
        lm.binding.rope(rk)
        lm.binding.flash_attn_fwd(plain)

    def two_launches():
        lm.binding.rope(rk)
        lm.binding.flash_attn_fwd(fused)

    three_launches()
    lm.binding.sync()
    want = o.to_host()
    two_launches()
    lm.binding.sync()
    same = bool(np.array_equal(o.to_host(), want))
    line = {"same_bits_as_three_launches": same}
    for name, fn in (("attention_alone_us", lambda: lm.binding.flash_attn_fwd(plain)),
                     ("attention_rotating_q_us", lambda: lm.binding.flash_attn_fwd(fused)),
                     ("rope_q_rope_k_attention_3_launches_us", three_launches), ("rope_k_attention_rotating_q_2_launches_us", two_launches)):
        _, ev = time_steps(fn, 20, 5, lm.binding)
        line[name] = ev * 1e3
    res["prompt path fp16 B=1 H=32 S=4096 D=96 causal (rotary embedding of q and k + attention)"] = line
    log("[other] prompt path: %s" % json.dumps(line))
    del xs, q, k, v, qr, kr, o

    caches = caches or c4_caches(lm, dev)
    for T, label in ((4096, "whole prompt T=4096"), (1, "one decode step T=1")):
        B, Hkv, L, D = 16, 8, 4096, 128
        kc, vc = caches[0]
        kn = lm.HipArray((B, Hkv, T, D), "bf16", dev).copy_from_host(lm.synth.normal((B, Hkv, T, D), 4100))
        vn = lm.HipArray((B, Hkv, T, D), "bf16", dev).copy_from_host(lm.synth.normal((B, Hkv, T, D), 4101))
        ap = lm.binding.KvAppendParams()
        ap.k_cache, ap.v_cache, ap.k_new, ap.v_new, ap.pos, ap.pos_all = kc.ptr, vc.ptr, kn.ptr, vn.ptr, None, (0 if T > 1 else L - 1)
        ap.B, ap.Hkv, ap.T, ap.D, ap.Lmax = B, Hkv, T, D, L
        ap.dtype, ap.rope_k, ap.pairing, ap.base, ap.stream = lm.binding.DTYPE_CODES["bf16"], 1, lm.binding.ROPE_HALF_SPLIT, 10000.0, None
        hbm_line("cache append + rotary K bf16 B=16 Hkv=8 D=128, %s" % label, lambda: lm.binding.kv_append(ap), 4.0 * B * Hkv * T * D * 2)


def step_leg(lm, dev, res):
    """One whole decode step of an attention layer, wall clock per step: as append (rotating q and K) + split-KV
    attention + merge (3 kernels) driven from the host and as one recorded HIP graph, and as the fused step
    (lmh_decode_step: the split kernel rotates q as it loads it, the merge launch adds and stores the new row; 2
    kernels). The caches hold L - 1 rows and the step writes row L - 1, so every form reads the same bytes. On the C4
    shape the GPU is the bottleneck either way; a single short sequence is bound by the launches."""
    for B, L in ((16, 4096), (1, 512)):
        Hq, Hkv, D = 32, 8, 128
        timings = {}
        for fused in (False, True):
            g = lm.Graph()
            tq, tkn, tvn = lm.tensor(g, (B, Hq, 1, D), "bf16"), lm.tensor(g, (B, Hkv, 1, D), "bf16"), lm.tensor(g, (B, Hkv, 1, D), "bf16")
            tkc, tvc = lm.tensor(g, (B, Hkv, L, D), "bf16"), lm.tensor(g, (B, Hkv, L, D), "bf16")
            tpos, tlen = lm.tensor(g, (B,), "i32"), lm.tensor(g, (B,), "i32")
            lm.cached_self_attention_core(tq, tkn, tvn, tkc, tvc, tpos, tlen, rope_base=10000.0, out_dtype="f32", fused=fused)
            cg = lm.compile(g, dev)
            assert len(cg.steps) == (1 if fused else 2)
            cg({tpos.id: np.full(B, L - 1, np.int32), tlen.id: np.full(B, L, np.int32)})

            def wall_us(n=200):
                for _ in range(20):
                    cg({})
                lm.binding.sync()
                t0 = time.perf_counter()
                for _ in range(n):
                    cg({})
                lm.binding.sync(cg.cache.get("hip_stream"))
                lm.binding.sync()
                return (time.perf_counter() - t0) / n * 1e6

            timings["fused" if fused else "eager"] = wall_us()
            cg.capture()
            timings["fused_graph" if fused else "graph"] = wall_us()
            cg.release()
        res["decode step of a layer bf16 B=%d Hq=32 Hkv=8 L=%d D=128 (append with rotary q and K + attention), wall clock" % (B, L)] = {
            "us_per_step_3_launches_from_the_host": timings["eager"], "us_per_step_one_hip_graph": timings["graph"],
            "us_per_step_fused_2_launches_from_the_host": timings["fused"], "us_per_step_fused_one_hip_graph": timings["fused_graph"]}
        log("[other] decode step B=%d L=%d, wall clock: %.1f us as 3 host launches, %.1f us as one HIP graph; fused step: %.1f us as "
            "2 host launches, %.1f us as one HIP graph" % (B, L, timings["eager"], timings["graph"], timings["fused"], timings["fused_graph"]))


def ceiling_leg(lm, dev):
    """What the matrix cores sustain, and how it depends on how much of the chip is busy: the bare MFMA loop on the
    workload's own operand values with 1, 2, 4 and 8 XCDs running it (the others idle), and the attention kernel on
    a steady-state shape (B=4, non-causal: 4096 equal workgroups). Rates are scaled to the whole chip (x 8 / active)
    so that they compare; clocks are settled before each timing."""
    res = {"bare_mfma_loop": {}}
    B, H, S, D = 4, 32, 4096, 96
    host = [lm.synth.normal((B, H, S, D), 2100 + i, 0.5).astype(np.float16) for i in range(3)]
    dq, dk, dv = (lm.HipArray((B, H, S, D), "f16", dev).copy_from_host(x) for x in host)
    sink = lm.HipArray((512 * 256,), "f32", dev)
    for active in (1, 2, 4, 8):
        per_wg = [0.0]

        def fn():
            per_wg[0] = lm.binding.calib_mfma_xcds(sink.ptr, dq.ptr, 1 << 17, 40000, active)
        _, ev = time_steps(fn, 3, 1, lm.binding)
        ran = int((sink.to_host().reshape(512, 256)[:, 0] != -1.0).sum())
        tf = per_wg[0] * ran / (ev * 1e-3) / 1e12
        res["bare_mfma_loop"]["%d_xcds" % active] = {
            "workgroups_that_ran": ran, "TFLOP/s": tf, "TFLOP/s_scaled_to_8_xcds": tf * 8 / active,
            "frac_of_peak_scaled": tf * 8 / active / PEAK_FP16_TFLOPS}
        log("[ceiling] bare MFMA loop on %d XCD(s): %d of 512 workgroups ran, %.0f TFLOP/s = %.0f scaled to the chip (%.1f%% of peak)"
            % (active, ran, tf, tf * 8 / active, 100 * tf * 8 / active / PEAK_FP16_TFLOPS))
    # the ceiling of a kernel with attention's instruction mix: synthetic interleaved streams on the whole chip
    mixes = ["MFMA only", "MFMA + 6 vector instr (1 exp)", "MFMA + 6 vector instr (1 exp) + 1 LDS fragment read",
             "MFMA + 6 vector instr (1 exp) + 1 LDS fragment read per 2 MFMAs", "MFMA + 4 vector instr (1 exp) + 1 LDS fragment read",
             "MFMA + 4 vector instr (1 exp) + 1 LDS fragment read per 2 MFMAs",
             "MFMA + 11 vector instr (the exp as a 6-instruction polynomial) + 1 LDS fragment read",
             "MFMA + 6 vector instr (1 exp) + 1 LDS fragment read, accumulators in AGPRs",
             "MFMA + 4 vector instr (1 exp) + 1 LDS fragment read per 2 MFMAs, accumulators in AGPRs"]
    res["instruction_mix_streams"] = {}
    mix_sink = lm.HipArray((512 * 512,), "f32", dev)
    for mix, label in enumerate(mixes):
        row = {}
        for wps in (2, 4):
            fl = [0.0]

            def fn():
                fl[0] = lm.binding.calib_mix(mix_sink.ptr, dq.ptr, 1 << 17, 10000 // (wps // 2), mix, wps)
            _, ev = time_steps(fn, 3, 1, lm.binding)
            row["TFLOP/s at %d waves per SIMD" % wps] = fl[0] / (ev * 1e-3) / 1e12
        res["instruction_mix_streams"][label] = row
        log("[ceiling] synthetic stream, %s: %.0f TFLOP/s at 2 waves per SIMD, %.0f at 4" % ((label,) + tuple(row.values())))
    out = lm.HipArray((B, H, S, D), "f16", dev)
    p = attn_params(lm, out, dq, dk, dv, "f16", False, lm.default_scale(D))
    _, ev = time_steps(lambda: lm.binding.flash_attn_fwd(p), 10, 3, lm.binding)
    active = int(os.environ.get("LMH_BENCH_ACTIVE_XCDS", "8"))  # 8 unless the library was built with -DLMH_ONLY_XCDS=n
    flops = 4.0 * B * H * D * S * S * active / 8
    res["attention_steady_state"] = {"shape": "B=4 H=32 S=4096 D=96 fp16 non-causal", "active_xcds": active, "launch_us": ev * 1e3,
                                     "TFLOP/s_scaled_to_8_xcds": flops / (ev * 1e-3) / 1e12 * 8 / active,
                                     "frac_of_peak_scaled": flops / (ev * 1e-3) / 1e12 * 8 / active / PEAK_FP16_TFLOPS}
    log("[ceiling] attention, steady-state shape, %d XCD(s) working: %.1f us, %.0f TFLOP/s scaled to the chip (%.1f%% of peak)"
        % (active, ev * 1e3, res["attention_steady_state"]["TFLOP/s_scaled_to_8_xcds"],
           100 * res["attention_steady_state"]["frac_of_peak_scaled"]))
    return res


def other_configs(lm, dev, check=False, only="other", zero_operands=True):
    """Short timings of the remaining contract configurations. With `check`, C1, C3 and C4 are also compared with the
    CPU oracle on the whole output (the parity gate of the five configurations: C2 and C5 are checked in their own
    legs). `only` = "other" runs everything, or one of c1 / nomask / bf16 / c3 / c4 / ops / step (a profile of one kernel)."""
    res = {}
    caches = None
    if only in ("other", "c1"):
        c1_leg(lm, dev, res, check)
    if only in ("other", "nomask"):
        nomask_leg(lm, dev, res, check, zero_operands)
    if only in ("other", "bf16"):
        bf16_leg(lm, dev, res, check)
    if only in ("other", "c3"):
        c3_leg(lm, dev, res, check)
    if only in ("other", "c4"):
        caches = c4_leg(lm, dev, res, check)
    if only in ("other", "ops"):
        ops_leg(lm, dev, res, caches)
    if only in ("other", "step"):
        step_leg(lm, dev, res)
    return res


def grid_leg(lm, dev):
    """Flash attention over a grid of square shapes (fp16 and bf16, causal and not, D = 64 / 128): µs per launch, TFLOP/s
    and the kernel each shape reaches. Not one of the contract's configurations: a map of where the launcher's rules put
    which instantiation, and of how far small launches are from the large ones."""
    rows = []
    for dtype in ("f16", "bf16"):
        for causal in (True, False):
            for D in (64, 128):
                for B, H in ((1, 8), (1, 32), (4, 32)):
                    for S in (512, 1024, 2048, 4096, 8192):
                        if B * H * S * S > 2 * 32 * 8192 * 8192:
                            continue
                        hq, hk, hv = (lm.synth.normal((B, H, S, D), 5000 + i, 0.5) for i in range(3))
                        q, k, v = (lm.HipArray(x.shape, dtype, dev).copy_from_host(x) for x in (hq, hk, hv))
                        o = lm.HipArray((B, H, S, D), dtype, dev)
                        p = attn_params(lm, o, q, k, v, dtype, causal, lm.default_scale(D))
                        steps = 30 if B * H * S * S < 2e9 else 8
                        _, ev = time_steps(lambda: lm.binding.flash_attn_fwd(p), steps, 3, lm.binding)
                        flops = 4.0 * B * H * D * (S * (S + 1) / 2 if causal else S * S)
                        row = {"dtype": dtype, "causal": causal, "B": B, "H": H, "S": S, "D": D, "launch_us": ev * 1e3,
                               "TFLOP/s": flops / (ev * 1e-3) / 1e12, "kernel": lm.binding.flash_attn_plan(p)}
                        rows.append(row)
                        log("[grid] %-4s %-6s B=%d H=%-2d S=%-4d D=%-3d %8.1f us %7.1f TFLOP/s (%4.1f%%)  %s" % (
                            dtype, "causal" if causal else "full", B, H, S, D, row["launch_us"], row["TFLOP/s"],
                            100 * row["TFLOP/s"] / PEAK_FP16_TFLOPS, row["kernel"]))
    return rows


def copy_leg(lm, dev, steps, warmup):
    """The calibration copy kernel alone (profile this with --pmc FETCH_SIZE / WRITE_SIZE)."""
    nbytes = 1 << 30
    src = lm.HipArray((nbytes // 4,), "f32", dev).fill_bytes(1)
    dst = lm.HipArray((nbytes // 4,), "f32", dev).fill_bytes(0)
    _, ev = time_steps(lambda: lm.binding.calib_copy(dst.ptr, src.ptr, nbytes), steps, warmup, lm.binding)
    log("[copy] %d bytes read + %d written per launch: %.1f us, %.0f GB/s" % (nbytes, nbytes, ev * 1e3, 2 * nbytes / (ev * 1e-3) / 1e9))
    return {"bytes_read_per_launch": nbytes, "bytes_written_per_launch": nbytes, "launch_us": ev * 1e3}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--only", choices=["all", "prefill", "decode", "other", "c1", "nomask", "bf16", "c3", "c4", "ops", "step", "copy", "ceiling", "grid", "shapes"], default="all")
    ap.add_argument("--decode-splits", type=int, default=0, help="KV splits for the decode leg (0 = library heuristic)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU-baseline budget per leg; 0 disables it")
    ap.add_argument("--shapes", default="1,32,32,4096,4096,96,bf16,causal",
                    help="for --only shapes: B,Hq,Hkv,Sq,Sk,D,dtype,causal|full, several separated by ';'")
    ap.add_argument("--no-zero-operands", action="store_true",
                    help="leave out the second timing of the prefill / nomask launch on all-zero tensors (for counter and "
                         "kernel-trace runs, whose per-kernel averages should cover the workload's launches only)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the attention path shards over (batch, KV head) with no exchange and "
              "nothing here uses a second device; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import __graft_entry__
    lm = __graft_entry__.load_package()
    dev = lm.get_device()
    if not isinstance(dev, lm.HIPDevice):
        raise SystemExit("bench.py needs an MI355X: libluminal_hip.so found no gfx950 device (no CPU fallback exists)")
    log("[bench] device:", lm.binding.device_name())

    line = {
        "metric": "attention TFLOP/s (prefill) + KV-read GB/s (decode), % roofline, 1×MI355X",
        "value": None, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic", "clock_settle_ms": CLOCK_SETTLE_MS,
        "config": {"workload": "C2 Phi-3-mini causal prefill attention: B=1 Hq=Hkv=32 S=4096 D=96, fp16 in/out, fp32 accumulate, scale 1/sqrt(96)"},
    }
    if args.only == "copy":
        line["calibration_copy"] = copy_leg(lm, dev, args.steps, args.warmup)
        print(json.dumps(line))
        return
    if args.only == "ceiling":
        line["ceiling"] = ceiling_leg(lm, dev)
        print(json.dumps(line))
        return
    if args.only == "shapes":
        line["shapes"] = shapes_leg(lm, dev, args.shapes)
        print(json.dumps(line))
        return
    if args.only == "grid":
        line["shape_grid"] = grid_leg(lm, dev)
        print(json.dumps(line))
        return
    if args.only in ("all", "prefill"):
        r = prefill_leg(lm, dev, args.steps, args.warmup, args.cpu_seconds, zero_operands=not args.no_zero_operands)
        line["value"], line["ms_per_step"] = r["value"], r["ms_per_step"]
        line["roofline"] = r["roofline"]
        if "cpu_baseline" in r:
            line["cpu_baseline"], line["parity"] = r["cpu_baseline"], r["parity"]
            line["cpu_baseline_single_thread"] = r["cpu_baseline_single_thread"]
    if args.only in ("all", "decode"):
        line["decode"] = decode_leg(lm, dev, args.steps, args.warmup, args.cpu_seconds, args.decode_splits)
    if args.only in ("all", "other", "c1", "nomask", "bf16", "c3", "c4", "ops", "step"):
        line["other_configs"] = other_configs(lm, dev, check=args.cpu_seconds > 0, only="other" if args.only == "all" else args.only,
                                              zero_operands=not args.no_zero_operands)
    gate = [("C2", line.get("parity"))] + [("C5", line.get("decode", {}).get("parity"))] + \
        [(k.split()[0] if k.split()[1] != "shape" else k.split(" (")[0], v.get("parity"))
         for k, v in line.get("other_configs", {}).items() if isinstance(v, dict) and "parity" in v]
    gate = [(n, p) for n, p in gate if p]
    if gate:
        line["parity_gate"] = {"configs": [n for n, _ in gate], "all_pass": all(p["max_rel_err"] <= p["tolerance"] for _, p in gate)}
        if not line["parity_gate"]["all_pass"]:
            log("PARITY GATE FAILED: " + ", ".join("%s %.2e > %g" % (n, p["max_rel_err"], p["tolerance"]) for n, p in gate if p["max_rel_err"] > p["tolerance"]))
            line["value"] = None  # no throughput is reported for a kernel that disagrees with the oracle
    print(json.dumps(line))


if __name__ == "__main__":
    main()
