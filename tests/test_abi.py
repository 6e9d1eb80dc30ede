"""CPU-side checks of the C ABI: the built library loads, exports every function the header
declares, and validates arguments (returning LMH_E_* with a message) before touching a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions(header="luminal_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lmh_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols(lm):
    assert header_functions() == sorted(lm.binding.EXPORTS)
    assert header_functions("luminal_hip_calib.h") == sorted(lm.binding.CALIB_EXPORTS)


def test_library_exports_every_declared_symbol(lm):
    lib = lm.binding.load()
    for name in header_functions():
        assert hasattr(lib, name), name
    assert lib.lmh_version() == 105
    calib = lm.binding.load_calib()
    for name in header_functions("luminal_hip_calib.h"):
        assert hasattr(calib, name), name


def test_measurement_kernels_are_not_in_the_attention_library(lm):
    """The attention library is the drop-in boundary: it exports nothing but what luminal_hip.h declares for the
    reference's interfaces, and it is a product build (no experiment switches compiled in)."""
    lib = lm.binding.load()
    for name in lm.binding.CALIB_EXPORTS:
        assert not hasattr(lib, name), name
    assert lib.lmh_measurement_build() == 0


def test_experiment_flags_need_the_measurement_marker(lm, monkeypatch):
    import importlib.util
    spec = importlib.util.spec_from_file_location("lmh_build_for_test", os.path.join(ROOT, "luminal.jl_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    monkeypatch.delenv("LMH_EXTRA_FLAGS", raising=False)
    monkeypatch.delenv("LMH_MEASUREMENT_BUILD", raising=False)
    assert build.experiment_flags() == []
    monkeypatch.setenv("LMH_EXTRA_FLAGS", "-DLMH_FOLD_SCALE")
    with pytest.raises(RuntimeError, match="LMH_MEASUREMENT_BUILD"):
        build.experiment_flags()
    monkeypatch.setenv("LMH_MEASUREMENT_BUILD", "1")
    assert build.experiment_flags() == ["-DLMH_FOLD_SCALE", "-DLMH_MEASUREMENT_BUILD"]
    # kernels that only a measurement build contains: not among the product sources, refuse to compile without the marker
    product = {src for sources in build.LIBRARIES.values() for src in sources}
    for switch, (src, _) in build.MEASUREMENT_SOURCES.items():
        assert src not in product
        text = open(os.path.join(ROOT, "luminal.jl_amd", "csrc", src)).read()
        assert "#error" in text and switch[2:] in text and "LMH_MEASUREMENT_BUILD" in text


def test_struct_layout_matches_header(lm):
    # field order/size must match the C struct: compare against sizes computed by hand from the header
    assert ctypes.sizeof(lm.binding.AttnParams) == 5 * 8 + 6 * 4 + 4 * 24 + 5 * 4 + 4 + 8 + 2 * 4 + 8 + 2 * 4
    assert ctypes.sizeof(lm.binding.DecodeStepExtra) == 2 * 8 + 3 * 4 + 4  # (4 bytes of tail padding)
    assert ctypes.sizeof(lm.binding.DecodeParams) == 5 * 8 + 5 * 4 + 4 + 2 * 16 + 2 * 24 + 5 * 4 + 4 + 8 + 8 + 8


def _attn(lm, **kw):
    p = lm.binding.AttnParams()
    p.out, p.q, p.k, p.v = 0x1000, 0x2000, 0x3000, 0x4000  # never dereferenced: validation fails first
    p.B, p.Hq, p.Hkv, p.Sq, p.Sk, p.D = 1, 4, 2, 8, 8, 64
    p.dtype, p.scale, p.causal, p.head_map = 0, 0.125, 1, 0
    for k, v in kw.items():
        setattr(p, k, v)
    return p


@pytest.mark.parametrize("kw,code", [
    (dict(q=None), -1), (dict(out=None), -1), (dict(B=0), -2), (dict(D=-3), -2), (dict(Hq=5), -2),
    (dict(dtype=7), -3), (dict(head_map=9), -3), (dict(D=264), -3), (dict(scale=float("nan")), -2),
])
def test_flash_attn_argument_errors(lm, kw, code):
    with pytest.raises(lm.LuminalHipError) as e:
        lm.binding.flash_attn_fwd(_attn(lm, **kw))
    assert e.value.code == code
    assert "lmh_flash_attn_fwd" in str(e.value)


def test_flash_attn_rejects_overlapping_rows(lm):
    p = _attn(lm)
    p.k_stride[0], p.k_stride[1], p.k_stride[2] = 1024, 512, 32  # row stride < D
    with pytest.raises(lm.LuminalHipError) as e:
        lm.binding.flash_attn_fwd(p)
    assert e.value.code == lm.binding.LMH_E_SHAPE


def _dec(lm, **kw):
    p = lm.binding.DecodeParams()
    p.out, p.q, p.k_cache, p.v_cache = 0x1000, 0x2000, 0x3000, 0x4000
    p.B, p.Hq, p.Hkv, p.Lmax, p.D = 2, 8, 2, 1024, 128
    p.dtype, p.scale, p.head_map, p.num_splits = 2, 0.088, 0, 4
    for k, v in kw.items():
        setattr(p, k, v)
    return p


@pytest.mark.parametrize("kw,code", [
    (dict(k_cache=None), -1), (dict(Lmax=0), -2), (dict(Hkv=3), -2), (dict(dtype=5), -3), (dict(D=100), -3),
    (dict(D=512), -3), (dict(num_splits=-1), -2), (dict(k_cache=0x3004), -2),
    (dict(), -4),                                   # 4 splits but no workspace
    (dict(workspace=0x5000, workspace_bytes=16), -4),  # workspace too small
])
def test_decode_argument_errors(lm, kw, code):
    with pytest.raises(lm.LuminalHipError) as e:
        lm.binding.decode_attn(_dec(lm, **kw))
    assert e.value.code == code
    assert "lmh_decode_attn" in str(e.value)


def test_decode_workspace_and_split_heuristic(lm):
    b = lm.binding
    assert b.decode_workspace_bytes(2, 8, 2, 1024, 128, 1) == 0
    assert b.decode_workspace_bytes(2, 8, 2, 1024, 128, 4) == 2 * 8 * 4 * 130 * 4
    assert b.decode_workspace_bytes(0, 8, 2, 1024, 128, 4) == 0
    for (B, Hkv, L) in [(16, 8, 4096), (64, 8, 32768), (1, 1, 17), (1, 8, 100000)]:
        s = b.decode_auto_splits(B, Hkv, L)
        assert s >= 1
        chunk = -(-L // s)
        assert s == 1 or chunk >= 100  # never shreds the cache into tiny splits
        assert b.decode_workspace_bytes(B, 4 * Hkv, Hkv, L, 128, 0) == b.decode_workspace_bytes(B, 4 * Hkv, Hkv, L, 128, s)


def test_static_scratch_decode_limits_are_checked_on_the_host(lm):
    # the entry point without a workspace: its split count always fits the static array, and an explicit count
    # that does not is refused before anything touches a GPU
    b = lm.binding
    cap = b.static_scratch_bytes()
    assert cap == 32 << 20
    for (B, Hq, Hkv, L, D) in [(16, 32, 8, 4096, 128), (64, 32, 8, 32768, 128), (64, 64, 1, 4096, 64), (1, 8, 8, 17, 64),
                               (512, 128, 8, 65536, 256)]:
        s = b.decode_static_splits(B, Hq, Hkv, L, D)
        assert 1 <= s <= b.decode_auto_splits(B, Hkv, L)
        assert b.decode_workspace_bytes(B, Hq, Hkv, L, D, s) <= cap
    assert b.decode_static_splits(16, 32, 8, 4096, 128) == b.decode_auto_splits(16, 8, 4096)  # fits as it is
    assert b.decode_static_splits(64, 32, 8, 32768, 128) < b.decode_auto_splits(64, 8, 32768)
    p = _dec(lm, B=64, Hq=32, Hkv=8, Lmax=32768, D=128, num_splits=64)
    with pytest.raises(lm.LuminalHipError) as e:
        b.decode_attn_static(p)
    assert e.value.code == b.LMH_E_WORKSPACE and "lmh_decode_attn_static" in str(e.value)
    with pytest.raises(lm.LuminalHipError) as e:
        b.decode_attn_static(_dec(lm, q=None))
    assert e.value.code == b.LMH_E_NULL and "lmh_decode_attn_static" in str(e.value)


def test_no_device_is_reported_not_fatal(lm):
    # Device probing never raises: the host's get_device() relies on it to fall through
    # (reference src/Device.jl:31-74 does the same with try/catch around a tiny allocation).
    n = lm.binding.device_count()
    assert n >= 0
    if n == 0:
        with pytest.raises(lm.LuminalHipError) as e:
            lm.binding.init(0)
        assert e.value.code == lm.binding.LMH_E_NODEVICE
        assert isinstance(lm.get_device(), lm.CPUDevice)


def test_null_and_zero_size_plumbing(lm):
    b = lm.binding
    with pytest.raises(lm.LuminalHipError):
        b.check(b.load().lmh_malloc(None, 16))
    assert b.load().lmh_free(None) == 0
    assert b.load().lmh_memcpy_h2d(None, None, 0, None) == 0
    with pytest.raises(lm.LuminalHipError):
        b.check(b.load().lmh_memcpy_h2d(None, None, 8, None))


def test_rope_and_kv_append_argument_errors(lm):
    b = lm.binding
    r = b.RopeParams()
    r.out, r.x = 0x1000, 0x2000
    r.B, r.H, r.S, r.D = 1, 2, 4, 7  # odd head dim
    r.dtype, r.base, r.pairing = 0, 10000.0, 0
    with pytest.raises(lm.LuminalHipError) as e:
        b.rope(r)
    assert e.value.code == b.LMH_E_SHAPE and "lmh_rope" in str(e.value)
    r.D, r.pairing = 8, 5
    with pytest.raises(lm.LuminalHipError) as e:
        b.rope(r)
    assert e.value.code == b.LMH_E_UNSUPPORTED
    a = b.KvAppendParams()
    a.k_cache, a.v_cache, a.k_new = 0x1000, 0x2000, 0x3000  # v_new missing
    a.B, a.Hkv, a.T, a.D, a.Lmax = 1, 1, 1, 8, 16
    with pytest.raises(lm.LuminalHipError) as e:
        b.kv_append(a)
    assert e.value.code == b.LMH_E_NULL and "lmh_kv_append" in str(e.value)
    a.v_new, a.Lmax = 0x4000, 0
    with pytest.raises(lm.LuminalHipError) as e:
        b.kv_append(a)
    assert e.value.code == b.LMH_E_SHAPE
    # queries to rotate along: a head count is needed, and the rotary arguments are checked although rope_k is off
    a.Lmax, a.q_rope, a.Hq = 16, 0x5000, 0
    with pytest.raises(lm.LuminalHipError) as e:
        b.kv_append(a)
    assert e.value.code == b.LMH_E_SHAPE and "Hq" in str(e.value)
    a.Hq, a.rope_k, a.pairing, a.base = 4, 0, 7, 10000.0
    with pytest.raises(lm.LuminalHipError) as e:
        b.kv_append(a)
    assert e.value.code == b.LMH_E_UNSUPPORTED
    a.pairing, a.D = 0, 7
    with pytest.raises(lm.LuminalHipError) as e:
        b.kv_append(a)
    assert e.value.code == b.LMH_E_SHAPE


def test_graph_recording_argument_errors(lm):
    # the null stream cannot be captured and a null graph cannot be launched; both are refused before any HIP call
    b = lm.binding
    with pytest.raises(lm.LuminalHipError) as e:
        b.graph_capture_begin(None)
    assert e.value.code == b.LMH_E_NULL and "null stream" in str(e.value)
    with pytest.raises(lm.LuminalHipError) as e:
        b.graph_launch(None, None)
    assert e.value.code == b.LMH_E_NULL
    with pytest.raises(lm.LuminalHipError) as e:
        b.check(b.load().lmh_graph_capture_end(None, None))
    assert e.value.code == b.LMH_E_NULL
    assert b.load().lmh_graph_destroy(None) == 0
    assert b.load().lmh_stream_destroy(None) == 0


def test_plain_c_client_builds_against_the_public_header(tmp_path):
    """tests/c_host/abi_client.c uses nothing but include/luminal_hip.h and the C library: it must compile as pedantic
    C99 without a warning, link against the shared library and start. Without a GPU it stops after the device count
    (exit status 77); with one it runs its checks (the GPU suite does that on the in-tree binary)."""
    import importlib.util
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("c_host_build", os.path.join(here, "c_host", "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    # same rpath convention as the in-tree binary: place it two levels below the repository root
    out_dir = os.path.join(here, "c_host")
    binary = mod.build(os.path.join(out_dir, "abi_client"))
    res = subprocess.run([binary], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert "libluminal_hip version" in res.stdout, res.stdout
    assert res.returncode in (0, 77), res.stdout
