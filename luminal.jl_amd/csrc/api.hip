// C-ABI layer of libluminal_hip.so: argument validation, dispatch to the kernel launchers, and
// the small device-runtime surface (allocation, copies, sync, events) that stands in for the
// CuArray()/Array() calls of the reference's device layer (reference src/Device.jl:82-105).
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "common.hpp"

// Split-KV partial storage of lmh_decode_attn_static, for callers that cannot allocate device memory.
// One copy per GPU, held from the moment the code object is loaded on that GPU until the process ends.
static __device__ __align__(256) unsigned char scratch[LMH_STATIC_SCRATCH_BYTES];

namespace lmh {

static thread_local char g_last_error[512] = "";

int device_cu_count() {
  static const int n = [] {  // one device kind per process (gfx950); initialised once, thread-safely
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess || prop.multiProcessorCount < 1) {
      (void)hipGetLastError();
      return 256;
    }
    return prop.multiProcessorCount;
  }();
  return n;
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

static thread_local char *g_plan_buf = nullptr;
static thread_local size_t g_plan_bytes = 0;

bool plan_only(const char *fmt, ...) {
  if (!g_plan_buf) return false;
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_plan_buf, g_plan_bytes, fmt, ap);
  va_end(ap);
  return true;
}

int hip_fail(hipError_t e, const char *what) {
  return fail(LMH_E_HIP, "HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
}

namespace {

bool all_zero(const int64_t *s, int n) {
  for (int i = 0; i < n; i++)
    if (s[i] != 0) return false;
  return true;
}

size_t elem_bytes(int dtype) { return dtype == LMH_F32 ? 4 : 2; }

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kMaxDevices = 64;
// Device address of `scratch` on each GPU. In host code the array's name is only a handle for
// hipGetSymbolAddress, never an address a kernel can use.
void *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;
// Who used the scratch last on each GPU: an event recorded behind that call's kernels and the stream it ran on. The next
// call on another stream asks the event whether the earlier call has finished, and refuses to race with it.
struct ScratchUse {
  hipEvent_t done = nullptr;
  hipStream_t stream = nullptr;
  bool pending = false;
};
ScratchUse g_scratch_use[kMaxDevices];

// Looks the address up once per device, with that device current, and returns it in *out.
int static_scratch_for_current_device(void **out) {
  *out = nullptr;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return fail(LMH_E_NODEVICE, "static scratch: no current HIP device (or its index is >= %d)", kMaxDevices);
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (!ptr) return fail(LMH_E_HIP, "static scratch: hipGetSymbolAddress returned a null address");
    hipEvent_t ev = nullptr;  // part of the same one-time set-up: the entry point itself creates nothing
    const hipError_t ee = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
    if (ee != hipSuccess) return hip_fail(ee, "hipEventCreateWithFlags(static scratch)");
    g_scratch_use[dev].done = ev;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return LMH_OK;
}

// True while `stream` is recording a HIP graph (then nothing may be queried or recorded on its behalf).
bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // cannot tell: behave as under capture (no event calls)
  }
  return st != hipStreamCaptureStatusNone;
}

// Before a call that uses the scratch: refuse when the previous user, on another stream, is still running. Two calls on
// one stream are ordered by the stream; the null stream and the streams of lmh_stream_create order themselves against
// each other, so only two different non-null streams can overlap. Calls recorded into a graph are not seen here.
int static_scratch_claim(hipStream_t stream, const char *fn) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return LMH_OK;
  }
  if (stream_is_capturing(stream)) return LMH_OK;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ScratchUse &u = g_scratch_use[dev];
  if (u.pending && u.stream != stream && u.stream != nullptr && stream != nullptr) {
    const hipError_t q = hipEventQuery(u.done);
    if (q == hipErrorNotReady)
      return fail(LMH_E_BUSY, "%s: the previous call that uses this GPU's static scratch is still running on another stream; "
                              "calls that share the scratch must not overlap (order them, or use lmh_decode_attn with a workspace)", fn);
    if (q != hipSuccess) (void)hipGetLastError();
  }
  return LMH_OK;
}

// After the kernels of such a call were enqueued.
void static_scratch_mark(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return;
  }
  if (stream_is_capturing(stream)) return;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ScratchUse &u = g_scratch_use[dev];
  if (!u.done) return;
  if (hipEventRecord(u.done, stream) != hipSuccess) {
    (void)hipGetLastError();
    u.pending = false;
    return;
  }
  u.stream = stream;
  u.pending = true;
}

}  // namespace
}  // namespace lmh

using namespace lmh;

extern "C" {

int lmh_version(void) { return LMH_VERSION; }

int lmh_measurement_build(void) {
#ifdef LMH_MEASUREMENT_BUILD
  return 1;
#else
  return 0;
#endif
}

const char *lmh_last_error(void) { return g_last_error; }

int lmh_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  int usable = 0;
  for (int i = 0; i < n; i++) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, i) == hipSuccess && strncmp(prop.gcnArchName, "gfx950", 6) == 0) usable++;
  }
  return usable;
}

int lmh_init(int device) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    return fail(LMH_E_NODEVICE, "no HIP device visible");
  }
  if (device < 0 || device >= n) return fail(LMH_E_NODEVICE, "device %d out of range (have %d)", device, n);
  hipDeviceProp_t prop;
  LMH_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(LMH_E_NODEVICE, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
  LMH_HIP_TRY(hipSetDevice(device));
  void *probe = nullptr;  // same health check as get_device(): a tiny allocation
  LMH_HIP_TRY(hipMalloc(&probe, 4));
  LMH_HIP_TRY(hipFree(probe));
  // set-up for lmh_decode_attn_static: resolve this device's copy of the static scratch now, so that the
  // entry point itself never has to (a failure here is reported by that entry point, not by init)
  void *unused = nullptr;
  if (static_scratch_for_current_device(&unused) != LMH_OK) g_last_error[0] = 0;  // init succeeded: leave no stale message
  return LMH_OK;
}

int lmh_device_name(char *buf, size_t buf_bytes) {
  if (!buf || buf_bytes == 0) return fail(LMH_E_NULL, "lmh_device_name: null buffer");
  int dev = 0;
  LMH_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  LMH_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  snprintf(buf, buf_bytes, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  return LMH_OK;
}

int lmh_malloc(void **dev_ptr, size_t bytes) {
  if (!dev_ptr) return fail(LMH_E_NULL, "lmh_malloc: null result pointer");
  *dev_ptr = nullptr;
  if (bytes == 0) return LMH_OK;
  LMH_HIP_TRY(hipMalloc(dev_ptr, bytes));
  return LMH_OK;
}

int lmh_free(void *dev_ptr) {
  if (!dev_ptr) return LMH_OK;
  LMH_HIP_TRY(hipFree(dev_ptr));
  return LMH_OK;
}

int lmh_memset(void *dev_ptr, int byte_value, size_t bytes, void *stream) {
  if (bytes == 0) return LMH_OK;
  if (!dev_ptr) return fail(LMH_E_NULL, "lmh_memset: null pointer");
  LMH_HIP_TRY(hipMemsetAsync(dev_ptr, byte_value, bytes, (hipStream_t)stream));
  return LMH_OK;
}

int lmh_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, void *stream) {
  if (bytes == 0) return LMH_OK;
  if (!dst_dev || !src_host) return fail(LMH_E_NULL, "lmh_memcpy_h2d: null pointer");
  LMH_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, (hipStream_t)stream));
  LMH_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));  // the host buffer may be reused at once
  return LMH_OK;
}

int lmh_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, void *stream) {
  if (bytes == 0) return LMH_OK;
  if (!dst_host || !src_dev) return fail(LMH_E_NULL, "lmh_memcpy_d2h: null pointer");
  LMH_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
  LMH_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  return LMH_OK;
}

int lmh_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes, void *stream) {
  if (bytes == 0) return LMH_OK;
  if (!dst_dev || !src_dev) return fail(LMH_E_NULL, "lmh_memcpy_d2d: null pointer");
  LMH_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return LMH_OK;
}

int lmh_sync(void *stream) {
  LMH_HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
  return LMH_OK;
}

int lmh_stream_create(void **stream) {
  if (!stream) return fail(LMH_E_NULL, "lmh_stream_create: null result pointer");
  hipStream_t s;
  LMH_HIP_TRY(hipStreamCreate(&s));  // default flags and priority
  *stream = s;
  return LMH_OK;
}

int lmh_stream_destroy(void *stream) {
  if (!stream) return LMH_OK;
  LMH_HIP_TRY(hipStreamDestroy((hipStream_t)stream));
  return LMH_OK;
}

int lmh_graph_capture_begin(void *stream) {
  if (!stream) return fail(LMH_E_NULL, "lmh_graph_capture_begin: the null stream cannot be captured");
  // thread-local: API calls of other host threads (a finalizer freeing memory) do not break the capture
  LMH_HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return LMH_OK;
}

int lmh_graph_capture_end(void *stream, void **graph_exec) {
  if (!stream || !graph_exec) return fail(LMH_E_NULL, "lmh_graph_capture_end: null stream or result pointer");
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  LMH_HIP_TRY(hipStreamEndCapture((hipStream_t)stream, &graph));
  if (!graph) return fail(LMH_E_HIP, "lmh_graph_capture_end: the capture was invalidated");
  hipGraphExec_t exec = nullptr;
  const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  LMH_HIP_TRY(e);
  *graph_exec = exec;
  return LMH_OK;
}

int lmh_graph_launch(void *graph_exec, void *stream) {
  if (!graph_exec) return fail(LMH_E_NULL, "lmh_graph_launch: null graph");
  LMH_HIP_TRY(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream));
  return LMH_OK;
}

int lmh_graph_destroy(void *graph_exec) {
  if (!graph_exec) return LMH_OK;
  LMH_HIP_TRY(hipGraphExecDestroy((hipGraphExec_t)graph_exec));
  return LMH_OK;
}

int lmh_event_create(void **event) {
  if (!event) return fail(LMH_E_NULL, "lmh_event_create: null result pointer");
  hipEvent_t e;
  LMH_HIP_TRY(hipEventCreate(&e));
  *event = e;
  return LMH_OK;
}

int lmh_event_destroy(void *event) {
  if (!event) return LMH_OK;
  LMH_HIP_TRY(hipEventDestroy((hipEvent_t)event));
  return LMH_OK;
}

int lmh_event_record(void *event, void *stream) {
  if (!event) return fail(LMH_E_NULL, "lmh_event_record: null event");
  LMH_HIP_TRY(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
  return LMH_OK;
}

int lmh_event_elapsed_ms(float *ms, void *start, void *stop) {
  if (!ms || !start || !stop) return fail(LMH_E_NULL, "lmh_event_elapsed_ms: null argument");
  LMH_HIP_TRY(hipEventSynchronize((hipEvent_t)stop));
  LMH_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return LMH_OK;
}

// --------------------------------------------------------------------------------------------
// flash attention forward
// --------------------------------------------------------------------------------------------
int lmh_flash_attn_fwd(const lmh_attn_params *p) {
  if (!p) return fail(LMH_E_NULL, "lmh_flash_attn_fwd: null params");
  if (!p->out || !p->q || !p->k || !p->v) return fail(LMH_E_NULL, "lmh_flash_attn_fwd: null tensor pointer");
  if (p->B <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->Sq <= 0 || p->Sk <= 0 || p->D <= 0)
    return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: non-positive dimension (B=%d Hq=%d Hkv=%d Sq=%d Sk=%d D=%d)", p->B,
                p->Hq, p->Hkv, p->Sq, p->Sk, p->D);
  if (p->Hq % p->Hkv != 0)
    return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: Hq=%d is not a multiple of Hkv=%d", p->Hq, p->Hkv);
  if (p->dtype != LMH_F32 && p->dtype != LMH_F16 && p->dtype != LMH_BF16)
    return fail(LMH_E_UNSUPPORTED, "lmh_flash_attn_fwd: unknown dtype %d", p->dtype);
  if (p->head_map != LMH_HEADMAP_INTERLEAVED && p->head_map != LMH_HEADMAP_BLOCKED)
    return fail(LMH_E_UNSUPPORTED, "lmh_flash_attn_fwd: unknown head_map %d", p->head_map);
  if (p->D > 256) return fail(LMH_E_UNSUPPORTED, "lmh_flash_attn_fwd: head dim %d > 256 is not supported", p->D);
  if (!(p->scale == p->scale)) return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: scale is NaN");
  if (p->q_rope) {
    if (p->D % 2 != 0) return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: head dim %d must be even for the rotary embedding", p->D);
    if (p->q_rope_pairing != LMH_ROPE_HALF_SPLIT && p->q_rope_pairing != LMH_ROPE_INTERLEAVED)
      return fail(LMH_E_UNSUPPORTED, "lmh_flash_attn_fwd: unknown q_rope_pairing %d", p->q_rope_pairing);
    if (!(p->q_rope_base > 0.f)) return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: q_rope_base must be positive");
  }

  PrefillArgs a;
  a.out = p->out; a.q = p->q; a.k = p->k; a.v = p->v; a.kv_len = p->kv_len;
  a.B = p->B; a.Hq = p->Hq; a.Hkv = p->Hkv; a.Sq = p->Sq; a.Sk = p->Sk; a.D = p->D;
  a.scale = p->scale; a.causal = p->causal ? 1 : 0; a.head_map = p->head_map;
  a.out_f32 = (p->out_f32 != 0 || p->dtype == LMH_F32) ? 1 : 0;
  a.q_rope = p->q_rope ? 1 : 0;
  a.q_interleaved = p->q_rope_pairing == LMH_ROPE_INTERLEAVED;
  a.q_pos0 = p->q_rope ? p->q_pos0 : nullptr;
  a.q_prev_seq = p->q_prev_seq;
  a.q_log2_base = p->q_rope ? log2f(p->q_rope_base) : 0.f;
  auto fill = [&](int64_t *dst, const int64_t *src, int64_t H, int64_t S) {
    if (all_zero(src, 3)) {
      dst[0] = H * S * p->D; dst[1] = S * p->D; dst[2] = p->D;
    } else {
      dst[0] = src[0]; dst[1] = src[1]; dst[2] = src[2];
    }
  };
  fill(a.qs, p->q_stride, p->Hq, p->Sq);
  fill(a.os, p->o_stride, p->Hq, p->Sq);
  fill(a.ks, p->k_stride, p->Hkv, p->Sk);
  fill(a.vs, p->v_stride, p->Hkv, p->Sk);
  for (int i = 0; i < 3; i++)
    if (a.qs[i] < 0 || a.os[i] < 0 || a.ks[i] < 0 || a.vs[i] < 0)
      return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: negative stride");
  if (a.qs[2] < p->D || a.os[2] < p->D || a.ks[2] < p->D || a.vs[2] < p->D)
    return fail(LMH_E_SHAPE, "lmh_flash_attn_fwd: row stride smaller than head dim (rows overlap)");

  // The matrix-core kernels do 128-bit accesses, track the max on raw scores (needs scale > 0) and fetch
  // K/V tiles with 32-bit buffer offsets inside one (b, kv head) slice.
  const int64_t esz = (int64_t)elem_bytes(p->dtype), vec = 16 / esz;
  bool mfma_ok = (prefill_mfma_supported(p->dtype, p->D) || prefill_f32_mfma_supported(p->dtype, p->D)) && p->scale > 0.f &&
                 aligned16(p->q) && aligned16(p->k) && aligned16(p->v) && aligned16(p->out);
  // (offsets from 0x7ffffff0 up are what the half-precision kernel uses as "out of range")
  constexpr int64_t kMaxSliceBytes = 0x7ffffff0;
  mfma_ok = mfma_ok && (int64_t)p->Sk * a.ks[2] * esz < kMaxSliceBytes && (int64_t)p->Sk * a.vs[2] * esz < kMaxSliceBytes;
  mfma_ok = mfma_ok && (!p->q_rope || prefill_mfma_rope_ok(p->D));  // the rotation in registers needs a head dim that fills its tiling
  for (int i = 0; i < 3 && mfma_ok; i++)
    mfma_ok = (a.qs[i] % vec == 0) && (a.ks[i] % vec == 0) && (a.vs[i] % vec == 0) && (a.os[i] % vec == 0);
  if (mfma_ok && p->dtype == LMH_F32) return launch_prefill_f32_mfma(a, (hipStream_t)p->stream);
  if (mfma_ok) return launch_prefill_mfma(a, p->dtype, (hipStream_t)p->stream);
  return launch_prefill_valu(a, p->dtype, (hipStream_t)p->stream);
}

int lmh_flash_attn_plan(const lmh_attn_params *p, char *plan, size_t plan_bytes) {
  if (!plan || plan_bytes < 2) return fail(LMH_E_NULL, "lmh_flash_attn_plan: no room for the description");
  plan[0] = 0;
  g_plan_buf = plan;
  g_plan_bytes = plan_bytes;
  const int rc = lmh_flash_attn_fwd(p);
  g_plan_buf = nullptr;
  return rc;
}

// --------------------------------------------------------------------------------------------
// decode attention
// --------------------------------------------------------------------------------------------
int32_t lmh_decode_auto_splits(int32_t B, int32_t Hkv, int32_t Lmax) {
  if (B <= 0 || Hkv <= 0 || Lmax <= 0) return 0;
  // The chunk (keys per split) is the unit the persistent decode kernel balances its workgroups
  // with: aim for >= 2048 units (4 per resident workgroup) with 128..512 keys each. Shorter chunks
  // only add partial-result slots; longer ones leave the last workgroups of a ragged batch idle.
  const int64_t pairs = (int64_t)B * Hkv;
  int64_t want = (2048 + pairs - 1) / pairs;
  int64_t chunk = (Lmax + want - 1) / want;
  if (chunk < 128) chunk = 128;
  if (chunk > 512) chunk = 512;
  chunk = (chunk + 63) / 64 * 64;
  int64_t splits = (Lmax + chunk - 1) / chunk;
  return (int32_t)(splits < 1 ? 1 : splits);
}

size_t lmh_decode_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t Lmax, int32_t D, int32_t num_splits) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Lmax <= 0 || D <= 0 || num_splits < 0) return 0;
  if (num_splits == 0) num_splits = lmh_decode_auto_splits(B, Hkv, Lmax);
  if (num_splits == 1) return 0;
  return (size_t)B * Hq * num_splits * (size_t)(D + 2) * sizeof(float);
}

// Validation and launch shared by lmh_decode_attn (caller-owned workspace) and lmh_decode_attn_static (the
// library's static scratch): `ws` / `ws_bytes` is the split-KV partial storage, `num_splits` already resolved.
static int decode_launch(const lmh_decode_params *p, const char *fn, int32_t num_splits, void *ws, size_t ws_bytes,
                         const lmh_decode_step_extra *step = nullptr) {
  DecodeArgs a;
  a.step = step ? 1 : 0;
  a.q_rope = (step && step->rope) ? 1 : 0;
  a.rope_interleaved = (step && step->pairing == LMH_ROPE_INTERLEAVED) ? 1 : 0;
  a.rope_log2_base = step ? log2f(step->rope_base) : 0.f;
  a.k_new = step ? step->k_new : nullptr;
  a.v_new = step ? step->v_new : nullptr;
  a.out = p->out; a.q = p->q; a.k = p->k_cache; a.v = p->v_cache; a.kv_len = p->kv_len;
  a.B = p->B; a.Hq = p->Hq; a.Hkv = p->Hkv; a.Lmax = p->Lmax; a.D = p->D;
  a.scale = p->scale; a.head_map = p->head_map;
  a.out_f32 = (p->out_f32 != 0 || p->dtype == LMH_F32) ? 1 : 0;
  if (all_zero(p->q_stride, 2)) { a.qs[0] = (int64_t)p->Hq * p->D; a.qs[1] = p->D; }
  else { a.qs[0] = p->q_stride[0]; a.qs[1] = p->q_stride[1]; }
  if (all_zero(p->o_stride, 2)) { a.os[0] = (int64_t)p->Hq * p->D; a.os[1] = p->D; }
  else { a.os[0] = p->o_stride[0]; a.os[1] = p->o_stride[1]; }
  auto fill3 = [&](int64_t *dst, const int64_t *src) {
    if (all_zero(src, 3)) {
      dst[0] = (int64_t)p->Hkv * p->Lmax * p->D; dst[1] = (int64_t)p->Lmax * p->D; dst[2] = p->D;
    } else {
      dst[0] = src[0]; dst[1] = src[1]; dst[2] = src[2];
    }
  };
  fill3(a.ks, p->k_stride);
  fill3(a.vs, p->v_stride);
  // 128-bit loads: every row start must be 16-byte aligned
  const int64_t align_elems = 16 / (int64_t)elem_bytes(p->dtype);
  if (!aligned16(p->k_cache) || !aligned16(p->v_cache))
    return fail(LMH_E_SHAPE, "%s: cache pointers must be 16-byte aligned", fn);
  for (int i = 0; i < 3; i++)
    if (a.ks[i] < 0 || a.vs[i] < 0 || a.ks[i] % align_elems != 0 || a.vs[i] % align_elems != 0)
      return fail(LMH_E_SHAPE, "%s: cache strides must be non-negative multiples of %lld elements", fn,
                  (long long)align_elems);
  if (a.ks[2] < p->D || a.vs[2] < p->D) return fail(LMH_E_SHAPE, "%s: cache row stride smaller than head dim", fn);
  if (a.qs[0] < 0 || a.qs[1] < 0 || a.os[0] < 0 || a.os[1] < 0) return fail(LMH_E_SHAPE, "%s: negative stride", fn);

  // the matrix-core kernel addresses a (b, kv head) slice with 32-bit buffer offsets
  // (a block of 32 rows is addressed even when Lmax is smaller, so bound that too)
  const int64_t rows = p->Lmax > 32 ? p->Lmax : 32;
  const bool slice_fits = rows * a.ks[2] * 2 < 0x7ffffff0 && rows * a.vs[2] * 2 < 0x7ffffff0;
  a.mfma_ok = (p->scale > 0.f && aligned16(p->q) && a.qs[0] % 8 == 0 && a.qs[1] % 8 == 0 && slice_fits) ? 1 : 0;
  a.num_splits = num_splits;
  a.chunk = decode_chunk_for(p->Lmax, a.num_splits);
  a.ws_o = nullptr;
  a.ws_ml = nullptr;
  if (a.num_splits > 1) {
    const size_t need = lmh_decode_workspace_bytes(p->B, p->Hq, p->Hkv, p->Lmax, p->D, a.num_splits);
    if (!ws || ws_bytes < need)
      return fail(LMH_E_WORKSPACE, "%s: workspace of %zu bytes needed for %d splits, got %zu", fn, need,
                  a.num_splits, ws ? ws_bytes : (size_t)0);
    if (!aligned16(ws)) return fail(LMH_E_WORKSPACE, "%s: workspace must be 16-byte aligned", fn);
    a.ws_o = reinterpret_cast<float *>(ws);
    a.ws_ml = a.ws_o + (size_t)p->B * p->Hq * a.num_splits * p->D;
  }
  if (step) {
    // two launches only where the split kernel can rotate q in registers and the slice fits its addressing
    if (!a.mfma_ok || !decode_mfma_supported(p->dtype, p->D, p->B))
      return fail(LMH_E_UNSUPPORTED, "%s: needs the matrix-core decode kernel (fp16 / bf16, head dim 64, 96, 128 or 256, aligned q, "
                  "batch <= 1024); use lmh_kv_append + lmh_decode_attn", fn);
    if (a.q_rope && !decode_mfma_rope_ok(p->D, a.rope_interleaved))
      return fail(LMH_E_UNSUPPORTED, "%s: head dim %d with the half-split pairing cannot be rotated in registers; use lmh_kv_append + "
                  "lmh_decode_attn", fn, p->D);
  }
  return launch_decode(a, p->dtype, (hipStream_t)p->stream);
}

static int decode_check(const lmh_decode_params *p, const char *fn) {
  if (!p) return fail(LMH_E_NULL, "%s: null params", fn);
  if (!p->out || !p->q || !p->k_cache || !p->v_cache) return fail(LMH_E_NULL, "%s: null tensor pointer", fn);
  if (p->B <= 0 || p->Hq <= 0 || p->Hkv <= 0 || p->Lmax <= 0 || p->D <= 0)
    return fail(LMH_E_SHAPE, "%s: non-positive dimension (B=%d Hq=%d Hkv=%d Lmax=%d D=%d)", fn, p->B, p->Hq,
                p->Hkv, p->Lmax, p->D);
  if (p->Hq % p->Hkv != 0) return fail(LMH_E_SHAPE, "%s: Hq=%d is not a multiple of Hkv=%d", fn, p->Hq, p->Hkv);
  if (p->dtype != LMH_F32 && p->dtype != LMH_F16 && p->dtype != LMH_BF16)
    return fail(LMH_E_UNSUPPORTED, "%s: unknown dtype %d", fn, p->dtype);
  if (p->head_map != LMH_HEADMAP_INTERLEAVED && p->head_map != LMH_HEADMAP_BLOCKED)
    return fail(LMH_E_UNSUPPORTED, "%s: unknown head_map %d", fn, p->head_map);
  const int vec = p->dtype == LMH_F32 ? 4 : 8;
  if (p->D % vec != 0 || p->D > 256)
    return fail(LMH_E_UNSUPPORTED, "%s: head dim %d must be a multiple of %d and <= 256", fn, p->D, vec);
  if (p->num_splits < 0) return fail(LMH_E_SHAPE, "%s: negative num_splits", fn);
  if (!(p->scale == p->scale)) return fail(LMH_E_SHAPE, "%s: scale is NaN", fn);
  return LMH_OK;
}

int lmh_decode_attn(const lmh_decode_params *p) {
  const int rc = decode_check(p, "lmh_decode_attn");
  if (rc != LMH_OK) return rc;
  const int32_t splits = p->num_splits == 0 ? lmh_decode_auto_splits(p->B, p->Hkv, p->Lmax) : p->num_splits;
  return decode_launch(p, "lmh_decode_attn", splits, p->workspace, p->workspace_bytes);
}

int32_t lmh_decode_step_splits(int32_t B, int32_t Hkv, int32_t Lmax) {
  const int32_t s = lmh_decode_auto_splits(B, Hkv, Lmax);
  return s == 0 ? 0 : (s < 2 ? 2 : s);  // the merge launch always runs: it is what adds the new row
}

int lmh_decode_step(const lmh_decode_params *p, const lmh_decode_step_extra *x) {
  const char *fn = "lmh_decode_step";
  const int rc = decode_check(p, fn);
  if (rc != LMH_OK) return rc;
  if (!x || !x->k_new || !x->v_new) return fail(LMH_E_NULL, "%s: null k_new / v_new", fn);
  if (!p->kv_len) return fail(LMH_E_NULL, "%s: kv_len (the rows already in the caches) is required", fn);
  if (p->dtype == LMH_F32) return fail(LMH_E_UNSUPPORTED, "%s: fp16 / bf16 only; use lmh_kv_append + lmh_decode_attn", fn);
  if (x->pairing != LMH_ROPE_HALF_SPLIT && x->pairing != LMH_ROPE_INTERLEAVED)
    return fail(LMH_E_UNSUPPORTED, "%s: unknown rope pairing %d", fn, x->pairing);
  if (x->rope && !(x->rope_base > 1.f)) return fail(LMH_E_SHAPE, "%s: rope base must be > 1", fn);
  if (p->num_splits == 1) return fail(LMH_E_SHAPE, "%s: num_splits must be 0 or >= 2", fn);
  const int32_t splits = p->num_splits == 0 ? lmh_decode_step_splits(p->B, p->Hkv, p->Lmax) : p->num_splits;
  return decode_launch(p, fn, splits, p->workspace, p->workspace_bytes, x);
}

// --------------------------------------------------------------------------------------------
// decode attention for callers that cannot allocate: the split-KV partials live in a static device array
// --------------------------------------------------------------------------------------------
size_t lmh_static_scratch_bytes(void) { return LMH_STATIC_SCRATCH_BYTES; }

int32_t lmh_decode_static_splits(int32_t B, int32_t Hq, int32_t Hkv, int32_t Lmax, int32_t D) {
  int32_t splits = lmh_decode_auto_splits(B, Hkv, Lmax);
  if (splits <= 0 || Hq <= 0 || D <= 0) return 0;
  // halve the split count (double the keys per split) until the partials fit; one split needs none
  while (splits > 1 && lmh_decode_workspace_bytes(B, Hq, Hkv, Lmax, D, splits) > LMH_STATIC_SCRATCH_BYTES)
    splits = (splits + 1) / 2;
  return splits;
}

int lmh_decode_attn_static(const lmh_decode_params *p) {
  const char *fn = "lmh_decode_attn_static";
  const int rc = decode_check(p, fn);
  if (rc != LMH_OK) return rc;
  const int32_t splits = p->num_splits == 0 ? lmh_decode_static_splits(p->B, p->Hq, p->Hkv, p->Lmax, p->D) : p->num_splits;
  const size_t need = lmh_decode_workspace_bytes(p->B, p->Hq, p->Hkv, p->Lmax, p->D, splits);
  if (need > LMH_STATIC_SCRATCH_BYTES)
    return fail(LMH_E_WORKSPACE,
                "%s: %d splits of B=%d Hq=%d D=%d need %zu bytes of partials, the static scratch holds %zu; "
                "pass num_splits = 0 or a smaller count, or use lmh_decode_attn with a workspace",
                fn, splits, p->B, p->Hq, p->D, need, (size_t)LMH_STATIC_SCRATCH_BYTES);
  void *ws = nullptr;
  if (splits > 1) {
    const int rc_ws = static_scratch_for_current_device(&ws);
    if (rc_ws != LMH_OK) return rc_ws;
    const int rc_claim = static_scratch_claim((hipStream_t)p->stream, fn);
    if (rc_claim != LMH_OK) return rc_claim;
  }
  // Nothing in the scratch has to start at zero: every partial slot the merge kernel reads was written by
  // the split kernel of the same call (a result, or the "empty" marker), so no clearing is enqueued.
  const int rc_launch = decode_launch(p, fn, splits, ws, LMH_STATIC_SCRATCH_BYTES);
  if (rc_launch == LMH_OK && splits > 1) static_scratch_mark((hipStream_t)p->stream);
  return rc_launch;
}

// --------------------------------------------------------------------------------------------
// rotary embedding and KV-cache append
// --------------------------------------------------------------------------------------------
int lmh_rope(const lmh_rope_params *p) {
  if (!p) return fail(LMH_E_NULL, "lmh_rope: null params");
  if (!p->out || !p->x) return fail(LMH_E_NULL, "lmh_rope: null tensor pointer");
  if (p->B <= 0 || p->H <= 0 || p->S <= 0 || p->D <= 0)
    return fail(LMH_E_SHAPE, "lmh_rope: non-positive dimension (B=%d H=%d S=%d D=%d)", p->B, p->H, p->S, p->D);
  if (p->D % 2 != 0) return fail(LMH_E_SHAPE, "lmh_rope: head dim %d must be even", p->D);
  if (p->dtype != LMH_F32 && p->dtype != LMH_F16 && p->dtype != LMH_BF16)
    return fail(LMH_E_UNSUPPORTED, "lmh_rope: unknown dtype %d", p->dtype);
  if (p->pairing != LMH_ROPE_HALF_SPLIT && p->pairing != LMH_ROPE_INTERLEAVED)
    return fail(LMH_E_UNSUPPORTED, "lmh_rope: unknown pairing %d", p->pairing);
  if (!(p->base > 0.f)) return fail(LMH_E_SHAPE, "lmh_rope: base must be positive");
  RopeArgs a;
  a.out = p->out; a.x = p->x; a.pos0 = p->pos0; a.prev_seq = p->prev_seq;
  a.B = p->B; a.H = p->H; a.S = p->S; a.D = p->D;
  auto fill = [&](int64_t *dst, const int64_t *src) {
    if (all_zero(src, 3)) { dst[0] = (int64_t)p->H * p->S * p->D; dst[1] = (int64_t)p->S * p->D; dst[2] = p->D; }
    else { dst[0] = src[0]; dst[1] = src[1]; dst[2] = src[2]; }
  };
  fill(a.xs, p->x_stride);
  fill(a.os, p->o_stride);
  for (int i = 0; i < 3; i++)
    if (a.xs[i] < 0 || a.os[i] < 0) return fail(LMH_E_SHAPE, "lmh_rope: negative stride");
  a.log2_base = log2f(p->base);
  a.interleaved = p->pairing == LMH_ROPE_INTERLEAVED;
  return launch_rope(a, p->dtype, (hipStream_t)p->stream);
}

int lmh_kv_append(const lmh_kv_append_params *p) {
  if (!p) return fail(LMH_E_NULL, "lmh_kv_append: null params");
  if (!p->k_cache || !p->v_cache || !p->k_new || !p->v_new) return fail(LMH_E_NULL, "lmh_kv_append: null tensor pointer");
  if (p->B <= 0 || p->Hkv <= 0 || p->T <= 0 || p->D <= 0 || p->Lmax <= 0)
    return fail(LMH_E_SHAPE, "lmh_kv_append: non-positive dimension (B=%d Hkv=%d T=%d D=%d Lmax=%d)", p->B, p->Hkv, p->T,
                p->D, p->Lmax);
  if (p->dtype != LMH_F32 && p->dtype != LMH_F16 && p->dtype != LMH_BF16)
    return fail(LMH_E_UNSUPPORTED, "lmh_kv_append: unknown dtype %d", p->dtype);
  if (p->q_rope && p->Hq <= 0) return fail(LMH_E_SHAPE, "lmh_kv_append: q_rope given with Hq=%d", p->Hq);
  if (p->rope_k || p->q_rope) {
    if (p->D % 2 != 0) return fail(LMH_E_SHAPE, "lmh_kv_append: head dim %d must be even for the rotary embedding", p->D);
    if (p->pairing != LMH_ROPE_HALF_SPLIT && p->pairing != LMH_ROPE_INTERLEAVED)
      return fail(LMH_E_UNSUPPORTED, "lmh_kv_append: unknown pairing %d", p->pairing);
    if (!(p->base > 0.f)) return fail(LMH_E_SHAPE, "lmh_kv_append: base must be positive");
  }
  KvAppendArgs a;
  a.k_cache = p->k_cache; a.v_cache = p->v_cache; a.k_new = p->k_new; a.v_new = p->v_new;
  a.pos = p->pos; a.pos_all = p->pos_all;
  a.B = p->B; a.Hkv = p->Hkv; a.T = p->T; a.D = p->D; a.Lmax = p->Lmax;
  auto fill = [&](int64_t *dst, const int64_t *src) {
    if (all_zero(src, 3)) { dst[0] = (int64_t)p->Hkv * p->Lmax * p->D; dst[1] = (int64_t)p->Lmax * p->D; dst[2] = p->D; }
    else { dst[0] = src[0]; dst[1] = src[1]; dst[2] = src[2]; }
  };
  fill(a.ks, p->k_stride);
  fill(a.vs, p->v_stride);
  for (int i = 0; i < 3; i++)
    if (a.ks[i] < 0 || a.vs[i] < 0) return fail(LMH_E_SHAPE, "lmh_kv_append: negative stride");
  if (a.ks[2] < p->D || a.vs[2] < p->D) return fail(LMH_E_SHAPE, "lmh_kv_append: cache row stride smaller than head dim");
  a.rope_k = p->rope_k ? 1 : 0;
  a.interleaved = p->pairing == LMH_ROPE_INTERLEAVED;
  a.log2_base = (p->rope_k || p->q_rope) ? log2f(p->base) : 0.f;
  a.q = p->q_rope;
  a.Hq = p->q_rope ? p->Hq : 0;
  return launch_kv_append(a, p->dtype, (hipStream_t)p->stream);
}

}  // extern "C"
