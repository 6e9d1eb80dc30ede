"""lmh_decode_attn_static — the decode entry point that allocates nothing: its split-KV partials live in a
static device array instead of a caller-owned workspace. Called through the C ABI and held to the same
results as lmh_decode_attn (same kernels, same split count: bit for bit) and to the oracle, on calls in a row
that share the array, the later ones with smaller inputs."""
import numpy as np
import pytest

from conftest import TOL, rel_err

pytestmark = pytest.mark.gpu


def _params(lm, out, q, kc, vc, kv_len, dtype, splits, workspace=None):
    p = lm.binding.DecodeParams()
    p.out, p.q, p.k_cache, p.v_cache = out.ptr, q.ptr, kc.ptr, vc.ptr
    p.kv_len = kv_len.ptr
    p.B, p.Hq, p.D = q.shape
    p.Hkv, p.Lmax = kc.shape[1], kc.shape[2]
    p.dtype = lm.binding.DTYPE_CODES[dtype]
    p.scale, p.head_map, p.out_f32 = lm.default_scale(p.D), 0, 1
    p.num_splits = splits
    if workspace is not None:
        p.workspace, p.workspace_bytes = workspace.ptr, workspace.nbytes
    return p


def _case(lm, hip, oracle, B, Hq, Hkv, Lmax, D, dtype, seed, lo):
    """One call through each entry point on the same device buffers; returns (static result, workspace
    result, oracle result, split count used)."""
    b = lm.binding
    q = oracle.round_to(oracle.gen_normal((B, Hq, D), seed), dtype)
    k = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), seed + 1), dtype)
    v = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), seed + 2), dtype)
    lens = oracle.gen_uniform_int(B, seed + 3, lo, Lmax)
    dq, dk, dv = (lm.to_device(x, hip, dtype) for x in (q, k, v))
    dl = lm.to_device(lens, hip)
    splits = b.decode_static_splits(B, Hq, Hkv, Lmax, D)
    assert b.decode_workspace_bytes(B, Hq, Hkv, Lmax, D, splits) <= b.static_scratch_bytes()
    print("static decode case B=%d Hq=%d Hkv=%d Lmax=%d D=%d %s splits=%d" % (B, Hq, Hkv, Lmax, D, dtype, splits),
          flush=True)

    out_static = lm.HipArray((B, Hq, D), "f32", hip).fill_bytes(0xFF)
    b.decode_attn_static(_params(lm, out_static, dq, dk, dv, dl, dtype, 0))  # 0 = the library's own choice
    got_static = out_static.to_host()

    ws = lm.HipArray((max(b.decode_workspace_bytes(B, Hq, Hkv, Lmax, D, splits), 16) // 4,), "f32", hip)
    out_ws = lm.HipArray((B, Hq, D), "f32", hip).fill_bytes(0xFF)
    b.decode_attn(_params(lm, out_ws, dq, dk, dv, dl, dtype, splits, ws))
    got_ws = out_ws.to_host()
    want = oracle.decode_attn(q, k, v, kv_len=lens, nthreads=16)
    return got_static, got_ws, want, splits


def test_static_scratch_decode_matches_workspace_decode_on_consecutive_calls(lm, hip, oracle):
    b = lm.binding
    # 1: partials of the usual split count (32) would need 34.6 MB, more than the array: 16 splits are taken
    B, Hq, Hkv, Lmax, D = 64, 64, 1, 4096, 64
    assert b.decode_workspace_bytes(B, Hq, Hkv, Lmax, D, 0) > b.static_scratch_bytes()
    s1, w1, want1, splits1 = _case(lm, hip, oracle, B, Hq, Hkv, Lmax, D, "f16", 9100, 1000)
    assert splits1 < b.decode_auto_splits(B, Hkv, Lmax)
    np.testing.assert_array_equal(s1, w1)
    assert rel_err(s1, want1) <= TOL["f16"]
    # 2: right after it, a smaller call on the same array (whatever call 1 left there must not matter)
    s2, w2, want2, _ = _case(lm, hip, oracle, 8, 32, 8, 2048, 128, "bf16", 9200, 1)
    np.testing.assert_array_equal(s2, w2)
    assert rel_err(s2, want2) <= TOL["bf16"]
    # 3: smaller again, fp32 caches (the vector kernel with its rectangular grid of splits)
    s3, w3, want3, _ = _case(lm, hip, oracle, 3, 8, 2, 1000, 64, "f32", 9300, 1)
    np.testing.assert_array_equal(s3, w3)
    assert rel_err(s3, want3) <= TOL["f32"]
    # 4: a single split needs no partials at all
    B, Hq, Hkv, Lmax, D = 2, 8, 2, 300, 128
    q = oracle.round_to(oracle.gen_normal((B, Hq, D), 9400), "bf16")
    k = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9401), "bf16")
    v = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9402), "bf16")
    lens = np.array([300, 17], np.int32)
    dq, dk, dv = (lm.to_device(x, hip, "bf16") for x in (q, k, v))
    dl = lm.to_device(lens, hip)
    out = lm.HipArray((B, Hq, D), "f32", hip).fill_bytes(0xFF)
    b.decode_attn_static(_params(lm, out, dq, dk, dv, dl, "bf16", 1))
    assert rel_err(out.to_host(), oracle.decode_attn(q, k, v, kv_len=lens)) <= TOL["bf16"]


def test_static_scratch_decode_rejects_what_does_not_fit(lm, hip):
    b = lm.binding
    B, Hq, Hkv, Lmax, D = 64, 64, 1, 4096, 64
    dq = lm.HipArray((B, Hq, D), "f16", hip)
    dk = lm.HipArray((B, Hkv, Lmax, D), "f16", hip)
    dl = lm.HipArray((B,), "i32", hip)
    out = lm.HipArray((B, Hq, D), "f32", hip)
    with pytest.raises(lm.LuminalHipError) as e:
        b.decode_attn_static(_params(lm, out, dq, dk, dk, dl, "f16", 32))
    assert e.value.code == b.LMH_E_WORKSPACE and "static scratch" in str(e.value)


def test_static_scratch_decode_recorded_into_a_hip_graph(lm, hip, oracle):
    """What the entry point is for: under stream capture nothing can be allocated. One recording of a split-KV call
    (several splits, so the static array is in use) is replayed for two sets of lengths, with eager work and
    synchronisations in between, and every replay is held to the oracle and to the eager call."""
    b = lm.binding
    B, Hq, Hkv, Lmax, D, dtype = 4, 16, 4, 2048, 128, "bf16"
    q = oracle.round_to(oracle.gen_normal((B, Hq, D), 9500), dtype)
    k = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9501), dtype)
    v = oracle.round_to(oracle.gen_normal((B, Hkv, Lmax, D), 9502), dtype)
    dq, dk, dv = (lm.to_device(x, hip, dtype) for x in (q, k, v))
    lens = [np.array([2048, 1500, 700, 33], np.int32), np.array([5, 2048, 1, 1024], np.int32)]
    dl = lm.to_device(lens[0], hip)
    splits = b.decode_static_splits(B, Hq, Hkv, Lmax, D)
    assert splits > 1
    out = lm.HipArray((B, Hq, D), "f32", hip)
    b.init(0)  # resolves the array's address and creates the guard event: set-up stays outside the recording
    stream = b.stream_create()
    p = _params(lm, out, dq, dk, dv, dl, dtype, 0)
    p.stream = stream
    b.graph_capture_begin(stream)
    try:
        b.decode_attn_static(p)
    finally:
        graph = b.graph_capture_end(stream)
    eager_out = lm.HipArray((B, Hq, D), "f32", hip)
    for rep in range(4):
        cur = lens[rep % 2]
        dl.copy_from_host(cur)
        out.fill_bytes(0xFF)
        b.graph_launch(graph, stream)
        b.sync(stream)
        got = out.to_host()
        want = oracle.decode_attn(q, k, v, kv_len=cur, nthreads=16)
        assert rel_err(got, want) <= TOL[dtype], rep
        # an eager call on the null stream in between (it shares the array; ordered by the synchronisations)
        b.decode_attn_static(_params(lm, eager_out, dq, dk, dv, dl, dtype, 0))
        np.testing.assert_array_equal(eager_out.to_host(), got)
    b.graph_destroy(graph)
    b.stream_destroy(stream)


def test_static_scratch_decode_refuses_to_overlap_on_two_streams(lm, hip):
    """Calls that share the array must not overlap: a call on a second stream while the first is still running is
    refused with LMH_E_BUSY; once the first has finished the same call goes through."""
    b = lm.binding
    B, Hq, Hkv, Lmax, D = 8, 32, 8, 32768, 128  # ~1 GB of cache reads: a few hundred microseconds of kernel
    dq = lm.HipArray((B, Hq, D), "bf16", hip).fill_bytes(0)
    dk = lm.HipArray((B, Hkv, Lmax, D), "bf16", hip).fill_bytes(0)
    dl = lm.to_device(np.full(B, Lmax, np.int32), hip)
    out1, out2 = lm.HipArray((B, Hq, D), "f32", hip), lm.HipArray((B, Hq, D), "f32", hip)
    s1, s2 = b.stream_create(), b.stream_create()
    p1, p2 = _params(lm, out1, dq, dk, dk, dl, "bf16", 0), _params(lm, out2, dq, dk, dk, dl, "bf16", 0)
    p1.stream, p2.stream = s1, s2
    b.sync()
    for _ in range(3):
        b.decode_attn_static(p1)  # queued back to back on one stream: ordered, never refused
    with pytest.raises(lm.LuminalHipError) as e:
        b.decode_attn_static(p2)
    assert e.value.code == b.LMH_E_BUSY and "static scratch" in str(e.value)
    b.sync(s1)
    b.decode_attn_static(p2)
    b.sync(s2)
    np.testing.assert_array_equal(out1.to_host(), out2.to_host())
    b.stream_destroy(s1)
    b.stream_destroy(s2)
