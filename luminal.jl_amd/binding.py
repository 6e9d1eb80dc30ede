"""ctypes binding of libluminal_hip.so — one Python function per C-ABI entry point of
include/luminal_hip.h, with LMH_E_* codes turned into LuminalHipError (the Julia glue does the
same with error(unsafe_string(lmh_last_error()))).

There is no CPU fallback: if the shared library is missing, load() raises.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libluminal_hip.so")
CALIB_LIB_PATH = os.path.join(HERE, "lib", "libluminal_hip_calib.so")

LMH_F32, LMH_F16, LMH_BF16 = 0, 1, 2
HEADMAP_INTERLEAVED, HEADMAP_BLOCKED = 0, 1
DTYPE_CODES = {"f32": LMH_F32, "f16": LMH_F16, "bf16": LMH_BF16}
DTYPE_BYTES = {"f32": 4, "f16": 2, "bf16": 2}

LMH_OK = 0
LMH_E_NULL, LMH_E_SHAPE, LMH_E_UNSUPPORTED, LMH_E_WORKSPACE, LMH_E_HIP, LMH_E_NODEVICE, LMH_E_BUSY = -1, -2, -3, -4, -5, -6, -7

# every symbol include/luminal_hip.h declares
EXPORTS = [
    "lmh_version", "lmh_measurement_build", "lmh_last_error", "lmh_device_count", "lmh_init", "lmh_device_name", "lmh_malloc", "lmh_free",
    "lmh_memset", "lmh_memcpy_h2d", "lmh_memcpy_d2h", "lmh_memcpy_d2d", "lmh_sync", "lmh_event_create",
    "lmh_event_destroy", "lmh_event_record", "lmh_event_elapsed_ms", "lmh_flash_attn_fwd",
    "lmh_decode_workspace_bytes", "lmh_decode_auto_splits", "lmh_decode_attn", "lmh_flash_attn_plan", "lmh_rope",
    "lmh_kv_append", "lmh_stream_create", "lmh_stream_destroy", "lmh_graph_capture_begin", "lmh_graph_capture_end",
    "lmh_graph_launch", "lmh_graph_destroy", "lmh_static_scratch_bytes", "lmh_decode_static_splits",
    "lmh_decode_attn_static", "lmh_decode_step_splits", "lmh_decode_step",
]


class LuminalHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libluminal_hip error %d: %s" % (code, message))
        self.code = code


class AttnParams(ctypes.Structure):
    _fields_ = [
        ("out", ctypes.c_void_p), ("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
        ("kv_len", ctypes.c_void_p),
        ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("Sq", ctypes.c_int32),
        ("Sk", ctypes.c_int32), ("D", ctypes.c_int32),
        ("q_stride", ctypes.c_int64 * 3), ("k_stride", ctypes.c_int64 * 3), ("v_stride", ctypes.c_int64 * 3),
        ("o_stride", ctypes.c_int64 * 3),
        ("dtype", ctypes.c_int32), ("scale", ctypes.c_float), ("causal", ctypes.c_int32),
        ("head_map", ctypes.c_int32), ("out_f32", ctypes.c_int32), ("stream", ctypes.c_void_p),
        ("q_rope", ctypes.c_int32), ("q_rope_pairing", ctypes.c_int32), ("q_pos0", ctypes.c_void_p),
        ("q_prev_seq", ctypes.c_int32), ("q_rope_base", ctypes.c_float),
    ]


class DecodeParams(ctypes.Structure):
    _fields_ = [
        ("out", ctypes.c_void_p), ("q", ctypes.c_void_p), ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p),
        ("kv_len", ctypes.c_void_p),
        ("B", ctypes.c_int32), ("Hq", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("Lmax", ctypes.c_int32),
        ("D", ctypes.c_int32),
        ("q_stride", ctypes.c_int64 * 2), ("o_stride", ctypes.c_int64 * 2), ("k_stride", ctypes.c_int64 * 3),
        ("v_stride", ctypes.c_int64 * 3),
        ("dtype", ctypes.c_int32), ("scale", ctypes.c_float), ("head_map", ctypes.c_int32),
        ("out_f32", ctypes.c_int32), ("num_splits", ctypes.c_int32), ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
    ]


class DecodeStepExtra(ctypes.Structure):
    _fields_ = [
        ("k_new", ctypes.c_void_p), ("v_new", ctypes.c_void_p), ("rope", ctypes.c_int32), ("pairing", ctypes.c_int32),
        ("rope_base", ctypes.c_float),
    ]


class RopeParams(ctypes.Structure):
    _fields_ = [
        ("out", ctypes.c_void_p), ("x", ctypes.c_void_p), ("pos0", ctypes.c_void_p), ("prev_seq", ctypes.c_int32),
        ("B", ctypes.c_int32), ("H", ctypes.c_int32), ("S", ctypes.c_int32), ("D", ctypes.c_int32),
        ("x_stride", ctypes.c_int64 * 3), ("o_stride", ctypes.c_int64 * 3),
        ("dtype", ctypes.c_int32), ("base", ctypes.c_float), ("pairing", ctypes.c_int32), ("stream", ctypes.c_void_p),
    ]


class KvAppendParams(ctypes.Structure):
    _fields_ = [
        ("k_cache", ctypes.c_void_p), ("v_cache", ctypes.c_void_p), ("k_new", ctypes.c_void_p),
        ("v_new", ctypes.c_void_p), ("pos", ctypes.c_void_p), ("pos_all", ctypes.c_int32),
        ("B", ctypes.c_int32), ("Hkv", ctypes.c_int32), ("T", ctypes.c_int32), ("D", ctypes.c_int32),
        ("Lmax", ctypes.c_int32),
        ("k_stride", ctypes.c_int64 * 3), ("v_stride", ctypes.c_int64 * 3),
        ("dtype", ctypes.c_int32), ("rope_k", ctypes.c_int32), ("pairing", ctypes.c_int32), ("base", ctypes.c_float),
        ("stream", ctypes.c_void_p),
        ("q_rope", ctypes.c_void_p), ("Hq", ctypes.c_int32),
    ]


# every symbol include/luminal_hip_calib.h declares (libluminal_hip_calib.so: measurement kernels, loaded on demand)
CALIB_EXPORTS = ["lmh_calib_last_error", "lmh_calib_copy", "lmh_calib_read", "lmh_calib_mfma", "lmh_calib_mfma_xcds",
                 "lmh_calib_mix"]

ROPE_HALF_SPLIT, ROPE_INTERLEAVED = 0, 1

_lib = None
_calib = None


def load():
    """Load the shared library (once). Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libluminal_hip.so is not built (%s missing); run `python luminal.jl_amd/build.py`. "
            "This backend has no CPU fallback." % LIB_PATH)
    L = ctypes.CDLL(LIB_PATH)
    vp = ctypes.c_void_p
    L.lmh_version.restype = ctypes.c_int
    L.lmh_measurement_build.restype = ctypes.c_int
    if L.lmh_measurement_build() and os.environ.get("LMH_MEASUREMENT_BUILD") != "1":
        raise RuntimeError(
            "%s was compiled with experiment switches (lmh_measurement_build() == 1): its kernels may compute wrong "
            "results on purpose. Rebuild with `python luminal.jl_amd/build.py`, or set LMH_MEASUREMENT_BUILD=1 to "
            "load it for a measurement." % LIB_PATH)
    L.lmh_last_error.restype = ctypes.c_char_p
    L.lmh_device_count.restype = ctypes.c_int
    L.lmh_init.argtypes = [ctypes.c_int]
    L.lmh_device_name.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    L.lmh_malloc.argtypes = [ctypes.POINTER(vp), ctypes.c_size_t]
    L.lmh_free.argtypes = [vp]
    L.lmh_memset.argtypes = [vp, ctypes.c_int, ctypes.c_size_t, vp]
    L.lmh_memcpy_h2d.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.lmh_memcpy_d2h.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.lmh_memcpy_d2d.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.lmh_sync.argtypes = [vp]
    L.lmh_event_create.argtypes = [ctypes.POINTER(vp)]
    L.lmh_event_destroy.argtypes = [vp]
    L.lmh_event_record.argtypes = [vp, vp]
    L.lmh_event_elapsed_ms.argtypes = [ctypes.POINTER(ctypes.c_float), vp, vp]
    L.lmh_flash_attn_fwd.argtypes = [ctypes.POINTER(AttnParams)]
    L.lmh_decode_attn.argtypes = [ctypes.POINTER(DecodeParams)]
    L.lmh_decode_workspace_bytes.restype = ctypes.c_size_t
    L.lmh_decode_workspace_bytes.argtypes = [ctypes.c_int32] * 6
    L.lmh_decode_auto_splits.restype = ctypes.c_int32
    L.lmh_decode_auto_splits.argtypes = [ctypes.c_int32] * 3
    L.lmh_decode_step_splits.restype = ctypes.c_int32
    L.lmh_decode_step_splits.argtypes = [ctypes.c_int32] * 3
    L.lmh_decode_step.argtypes = [ctypes.POINTER(DecodeParams), ctypes.POINTER(DecodeStepExtra)]
    L.lmh_decode_attn_static.argtypes = [ctypes.POINTER(DecodeParams)]
    L.lmh_decode_attn_static.restype = ctypes.c_int
    L.lmh_static_scratch_bytes.restype = ctypes.c_size_t
    L.lmh_decode_static_splits.restype = ctypes.c_int32
    L.lmh_decode_static_splits.argtypes = [ctypes.c_int32] * 5
    L.lmh_flash_attn_plan.argtypes = [ctypes.POINTER(AttnParams), ctypes.c_char_p, ctypes.c_size_t]
    L.lmh_flash_attn_plan.restype = ctypes.c_int
    L.lmh_rope.argtypes = [ctypes.POINTER(RopeParams)]
    L.lmh_kv_append.argtypes = [ctypes.POINTER(KvAppendParams)]
    L.lmh_stream_create.argtypes = [ctypes.POINTER(vp)]
    L.lmh_stream_destroy.argtypes = [vp]
    L.lmh_graph_capture_begin.argtypes = [vp]
    L.lmh_graph_capture_end.argtypes = [vp, ctypes.POINTER(vp)]
    L.lmh_graph_launch.argtypes = [vp, vp]
    L.lmh_graph_destroy.argtypes = [vp]
    for name in ("lmh_rope", "lmh_kv_append", "lmh_init", "lmh_device_name", "lmh_malloc", "lmh_free", "lmh_memset", "lmh_memcpy_h2d",
                 "lmh_memcpy_d2h", "lmh_memcpy_d2d", "lmh_sync", "lmh_event_create", "lmh_event_destroy",
                 "lmh_event_record", "lmh_event_elapsed_ms", "lmh_flash_attn_fwd", "lmh_decode_attn"):
        getattr(L, name).restype = ctypes.c_int
    _lib = L
    return L


def load_calib():
    """Load libluminal_hip_calib.so, the measurement kernels (once). Raises if it has not been built."""
    global _calib
    if _calib is not None:
        return _calib
    if not os.path.exists(CALIB_LIB_PATH):
        raise RuntimeError("libluminal_hip_calib.so is not built (%s missing); run `python luminal.jl_amd/build.py`." % CALIB_LIB_PATH)
    L = ctypes.CDLL(CALIB_LIB_PATH)
    vp = ctypes.c_void_p
    dp = ctypes.POINTER(ctypes.c_double)
    L.lmh_calib_last_error.restype = ctypes.c_char_p
    L.lmh_calib_copy.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.lmh_calib_read.argtypes = [vp, ctypes.c_size_t, vp, vp]
    L.lmh_calib_mfma.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int, dp, vp]
    L.lmh_calib_mfma_xcds.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, dp, vp]
    L.lmh_calib_mix.argtypes = [vp, vp, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, dp, vp]
    for name in CALIB_EXPORTS[1:]:
        getattr(L, name).restype = ctypes.c_int
    _calib = L
    return L


def check(rc):
    if rc != LMH_OK:
        raise LuminalHipError(rc, load().lmh_last_error().decode("utf-8", "replace"))


def check_calib(rc):
    if rc != LMH_OK:
        raise LuminalHipError(rc, load_calib().lmh_calib_last_error().decode("utf-8", "replace"))


def device_count():
    return int(load().lmh_device_count())


def init(device=0):
    check(load().lmh_init(device))


def device_name():
    buf = ctypes.create_string_buffer(256)
    check(load().lmh_device_name(buf, 256))
    return buf.value.decode()


def malloc(nbytes):
    p = ctypes.c_void_p()
    check(load().lmh_malloc(ctypes.byref(p), nbytes))
    return p.value or 0


def free(ptr):
    check(load().lmh_free(ptr))


def memset(ptr, value, nbytes, stream=None):
    check(load().lmh_memset(ptr, value, nbytes, stream))


def memcpy_h2d(dst, src_host_ptr, nbytes, stream=None):
    check(load().lmh_memcpy_h2d(dst, src_host_ptr, nbytes, stream))


def memcpy_d2h(dst_host_ptr, src, nbytes, stream=None):
    check(load().lmh_memcpy_d2h(dst_host_ptr, src, nbytes, stream))


def memcpy_d2d(dst, src, nbytes, stream=None):
    check(load().lmh_memcpy_d2d(dst, src, nbytes, stream))


def sync(stream=None):
    check(load().lmh_sync(stream))


class Event:
    def __init__(self):
        p = ctypes.c_void_p()
        check(load().lmh_event_create(ctypes.byref(p)))
        self.ptr = p.value

    def record(self, stream=None):
        check(load().lmh_event_record(self.ptr, stream))

    def elapsed_ms_since(self, start):
        ms = ctypes.c_float()
        check(load().lmh_event_elapsed_ms(ctypes.byref(ms), start.ptr, self.ptr))
        return float(ms.value)

    def __del__(self):
        try:
            if self.ptr:
                load().lmh_event_destroy(self.ptr)
        except Exception:
            pass


def flash_attn_fwd(params):
    check(load().lmh_flash_attn_fwd(ctypes.byref(params)))


def decode_attn(params):
    check(load().lmh_decode_attn(ctypes.byref(params)))


def decode_step(params, extra):
    """lmh_decode_step: append this step's K / V rows and attend, in two launches."""
    check(load().lmh_decode_step(ctypes.byref(params), ctypes.byref(extra)))


def decode_step_splits(B, Hkv, Lmax):
    return int(load().lmh_decode_step_splits(B, Hkv, Lmax))


def decode_attn_static(params):
    """lmh_decode_attn without a workspace: partials go to the library's static device scratch."""
    check(load().lmh_decode_attn_static(ctypes.byref(params)))


def static_scratch_bytes():
    return int(load().lmh_static_scratch_bytes())


def decode_static_splits(B, Hq, Hkv, Lmax, D):
    return int(load().lmh_decode_static_splits(B, Hq, Hkv, Lmax, D))


def rope(params):
    check(load().lmh_rope(ctypes.byref(params)))


def kv_append(params):
    check(load().lmh_kv_append(ctypes.byref(params)))


def stream_create():
    s = ctypes.c_void_p()
    check(load().lmh_stream_create(ctypes.byref(s)))
    return s


def stream_destroy(stream):
    check(load().lmh_stream_destroy(stream))


def graph_capture_begin(stream):
    check(load().lmh_graph_capture_begin(stream))


def graph_capture_end(stream):
    g = ctypes.c_void_p()
    check(load().lmh_graph_capture_end(stream, ctypes.byref(g)))
    return g


def graph_launch(graph_exec, stream):
    check(load().lmh_graph_launch(graph_exec, stream))


def graph_destroy(graph_exec):
    check(load().lmh_graph_destroy(graph_exec))


def calib_copy(dst, src, nbytes, stream=None):
    check_calib(load_calib().lmh_calib_copy(dst, src, nbytes, stream))


def calib_read(src, nbytes, sink4, stream=None):
    check_calib(load_calib().lmh_calib_read(src, nbytes, sink4, stream))


def calib_mfma(sink, operands, operand_bytes, iters, stream=None):
    """Launch the bare MFMA loop; returns the flops of the launch."""
    flops = ctypes.c_double(0.0)
    check_calib(load_calib().lmh_calib_mfma(sink, operands, operand_bytes, iters, ctypes.byref(flops), stream))
    return flops.value


def flash_attn_plan(params):
    """Text naming the kernel lmh_flash_attn_fwd would launch for `params`; launches nothing."""
    buf = ctypes.create_string_buffer(256)
    check(load().lmh_flash_attn_plan(ctypes.byref(params), buf, len(buf)))
    return buf.value.decode()


def calib_mix(sink, operands, operand_bytes, iters, mix, waves_per_simd=2, stream=None):
    """Launch the synthetic instruction-mix stream `mix` (0..8) at 2 or 4 waves per SIMD; returns the flops of the launch."""
    flops = ctypes.c_double(0.0)
    check_calib(load_calib().lmh_calib_mix(sink, operands, operand_bytes, iters, mix, waves_per_simd, ctypes.byref(flops), stream))
    return flops.value


def calib_mfma_xcds(sink, operands, operand_bytes, iters, active_xcds, stream=None):
    """The bare MFMA loop on the first `active_xcds` XCDs only; returns the flops of one running workgroup."""
    flops = ctypes.c_double(0.0)
    check_calib(load_calib().lmh_calib_mfma_xcds(sink, operands, operand_bytes, iters, active_xcds, ctypes.byref(flops), stream))
    return flops.value


def decode_workspace_bytes(B, Hq, Hkv, Lmax, D, num_splits=0):
    return int(load().lmh_decode_workspace_bytes(B, Hq, Hkv, Lmax, D, num_splits))


def decode_auto_splits(B, Hkv, Lmax):
    return int(load().lmh_decode_auto_splits(B, Hkv, Lmax))
