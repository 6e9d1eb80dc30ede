"""Prefill launches recorded into one HIP graph: the flash attention entry point allocates nothing and keeps no state, so a
prompt's attention launches can be recorded once and replayed on new data. One recording holds a launch of each matrix-core
form (paired tiles, bf16 with V as fp16, the wide kernel with two and four key groups, wave pairs splitting the keys); it is
replayed three times with fresh inputs, eager work and synchronisations in between, and every replay must return the eager
call's bits; the first replay is also held to the oracle."""
import ctypes

import numpy as np
import pytest

from conftest import TOL, rel_err
from test_parity_gpu import inputs

pytestmark = pytest.mark.gpu

# (dtype, B, Hq, Hkv, Sq, Sk, D, causal, part of the plan the launch must reach)
LAUNCHES = [
    ("f16", 1, 32, 8, 4096, 4096, 96, True, "prefill_mfma_pair_kernel<f16, D=96, causal>"),
    ("bf16", 1, 24, 24, 3072, 3072, 64, True, "V as fp16"),
    ("f16", 4, 20, 20, 448, 704, 64, False, "two and four key groups"),
    ("bf16", 1, 8, 2, 300, 300, 128, True, "key groups=2"),
]


def params(lm, out, q, k, v, dtype, causal, shape_q, shape_kv, stream):
    B, Hq, Sq, D = shape_q
    p = lm.binding.AttnParams()
    p.out, p.q, p.k, p.v = out.ptr, q.ptr, k.ptr, v.ptr
    p.B, p.Hq, p.Sq, p.D = B, Hq, Sq, D
    p.Hkv, p.Sk = shape_kv[1], shape_kv[2]
    p.dtype = lm.binding.DTYPE_CODES[dtype]
    p.scale = lm.default_scale(D)
    p.causal = 1 if causal else 0
    p.out_f32 = 1
    p.stream = stream
    return p


def test_prefill_launches_recorded_as_one_hip_graph(lm, hip, oracle):
    b = lm.binding
    b.init(0)
    stream = b.stream_create()
    bufs = []
    for dtype, B, Hq, Hkv, Sq, Sk, D, causal, want_plan in LAUNCHES:
        sq, skv = (B, Hq, Sq, D), (B, Hkv, Sk, D)
        dq, dk, dv = lm.HipArray(sq, dtype, hip), lm.HipArray(skv, dtype, hip), lm.HipArray(skv, dtype, hip)
        out, eager = lm.HipArray(sq, "f32", hip), lm.HipArray(sq, "f32", hip)
        p = params(lm, out, dq, dk, dv, dtype, causal, sq, skv, stream)
        plan = b.flash_attn_plan(p)
        print(plan, flush=True)
        assert want_plan in plan, plan
        bufs.append((dtype, sq, skv, causal, dq, dk, dv, out, eager, p))
    b.graph_capture_begin(stream)
    try:
        for *_, p in bufs:
            b.flash_attn_fwd(p)
    finally:
        graph = b.graph_capture_end(stream)
    for rep in range(3):
        host = []
        for i, (dtype, sq, skv, causal, dq, dk, dv, out, eager, p) in enumerate(bufs):
            q, k, v = inputs(oracle, sq, skv, dtype, 88000 + 10 * rep + i, 0.7)
            dq.copy_from_host(q), dk.copy_from_host(k), dv.copy_from_host(v)
            out.fill_bytes(0xFF)
            host.append((q, k, v))
        b.graph_launch(graph, stream)
        b.sync(stream)
        for (dtype, sq, skv, causal, dq, dk, dv, out, eager, p), (q, k, v) in zip(bufs, host):
            got = out.to_host()
            pe = params(lm, eager, dq, dk, dv, dtype, causal, sq, skv, None)  # the same launch, eager, on the null stream
            b.flash_attn_fwd(pe)
            b.sync()
            np.testing.assert_array_equal(eager.to_host().view(np.uint32), got.view(np.uint32))
            if rep == 0:
                hq = np.array([0, sq[1] - 1])
                kv_of = hq % skv[1]
                want = oracle.flash_attn(q[:, hq], k[:, kv_of], v[:, kv_of], causal=causal, nthreads=16)
                assert rel_err(got[:, hq], want) <= TOL[dtype]
    b.graph_destroy(graph)
    b.stream_destroy(stream)
