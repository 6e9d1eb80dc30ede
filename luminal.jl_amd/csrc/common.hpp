// Shared declarations of libluminal_hip.so: error reporting, launch argument blocks and the
// kernel launchers each .hip file exports to the C-ABI layer in api.hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/luminal_hip.h"

namespace lmh {

// Records a message for lmh_last_error() and returns `code`, so call sites read
// `return fail(LMH_E_SHAPE, "...")`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
// Compute units of the current device (256 on an MI355X in its default partition mode; 256 as well if the query
// fails). The launchers size their workgroups by it; any value gives correct results.
int device_cu_count();
int hip_fail(hipError_t e, const char *what);
// While a plan query (lmh_flash_attn_plan) runs on this thread, a launcher that calls this with the description of
// the kernel it has chosen gets `true` back and must return LMH_OK without launching.
bool plan_only(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

#define LMH_HIP_TRY(expr)                                \
  do {                                                   \
    hipError_t lmh_e_ = (expr);                          \
    if (lmh_e_ != hipSuccess) return ::lmh::hip_fail(lmh_e_, #expr); \
  } while (0)

// Prefill (flash attention forward) launch arguments; strides are in elements.
struct PrefillArgs {
  void *out;
  const void *q, *k, *v;
  const int32_t *kv_len;
  int32_t B, Hq, Hkv, Sq, Sk, D;
  int64_t qs[3], ks[3], vs[3], os[3];
  float scale;
  int32_t causal;
  int32_t head_map;
  int32_t out_f32;  // out is fp32 whatever the input element type
  // Rotary embedding of the query rows on their way into the kernel (q_rope != 0): row i of sequence b is rotated at
  // position (q_pos0 ? q_pos0[b] : q_prev_seq) + i and rounded to the element type, as lmh_rope would have stored it.
  int32_t q_rope;
  int32_t q_interleaved;  // 0: pairs (j, j + D/2) as the reference; 1: pairs (2j, 2j+1)
  const int32_t *q_pos0;
  int32_t q_prev_seq;
  float q_log2_base;
};

// Decode launch arguments.
struct DecodeArgs {
  void *out;
  const void *q, *k, *v;
  const int32_t *kv_len;
  int32_t B, Hq, Hkv, Lmax, D;
  int64_t qs[2], os[2], ks[3], vs[3];
  float scale;
  int32_t head_map;
  int32_t out_f32;  // out is fp32 whatever the input element type
  int32_t num_splits;
  int32_t chunk;  // keys per split
  int32_t mfma_ok;  // q is 16-byte aligned with 8-element strides and scale > 0: the MFMA kernel may run
  float *ws_o;    // [B][Hq][num_splits][D] un-normalised partial outputs
  float *ws_ml;   // [B][Hq][num_splits][2] (running max in log2 units, partial sum)
  // lmh_decode_step: the split kernel attends the kv_len[b] rows already in the cache with q rotated as it is loaded;
  // the merge kernel adds row kv_len[b] from k_new / v_new (K rotated) and writes it into the caches.
  int32_t step;             // 0: plain decode attention
  int32_t q_rope;           // rotate q (and k_new) at position kv_len[b]
  int32_t rope_interleaved;
  float rope_log2_base;
  const void *k_new, *v_new;  // [B][Hkv][D] contiguous
};

// Rotary embedding launch arguments.
struct RopeArgs {
  void *out;
  const void *x;
  const int32_t *pos0;  // per-sequence position of row 0 (device), or null -> prev_seq
  int32_t prev_seq;
  int32_t B, H, S, D;
  int64_t xs[3], os[3];
  float log2_base;
  int32_t interleaved;  // 0: pairs (j, j + D/2) as the reference; 1: pairs (2j, 2j+1)
};

// KV-cache append launch arguments; k_new / v_new are contiguous [B, Hkv, T, D].
struct KvAppendArgs {
  void *k_cache, *v_cache;
  const void *k_new, *v_new;
  const int32_t *pos;  // per-sequence first row (device), or null -> pos_all
  int32_t pos_all;
  int32_t B, Hkv, T, D, Lmax;
  int64_t ks[3], vs[3];
  int32_t rope_k;  // rotate K by its row position while writing it
  int32_t interleaved;
  float log2_base;
  void *q;         // optional [B, Hq, T, D], contiguous: rotated in place at the same positions
  int32_t Hq;
};

// Every field of a launch-argument block, requested from memory in one batch at the kernel's start (a kernel calls this first).
// Left to the compiler, the scalar loads of these 100 to 230 byte blocks are issued where their values are first needed: in the
// attention kernels five and more round trips to memory, one after the other, before a wave has issued its first tile load
// (measured: 0.2 to 0.4 us per launch). The empty asm statements only name the values as scalar-register inputs.
__device__ __forceinline__ void request_arg(int x) { asm volatile("" ::"s"(x)); }
__device__ __forceinline__ void request_args(const PrefillArgs &a) {
  asm volatile("" ::"s"(a.out), "s"(a.q), "s"(a.k), "s"(a.v), "s"(a.kv_len), "s"(a.B), "s"(a.Hq), "s"(a.Hkv), "s"(a.Sq), "s"(a.Sk), "s"(a.D));
  asm volatile("" ::"s"(a.qs[0]), "s"(a.qs[1]), "s"(a.qs[2]), "s"(a.ks[0]), "s"(a.ks[1]), "s"(a.ks[2]), "s"(a.vs[0]), "s"(a.vs[1]), "s"(a.vs[2]), "s"(a.os[0]), "s"(a.os[1]), "s"(a.os[2]));
  asm volatile("" ::"s"(a.scale), "s"(a.causal), "s"(a.head_map), "s"(a.out_f32), "s"(a.q_rope), "s"(a.q_interleaved), "s"(a.q_pos0), "s"(a.q_prev_seq), "s"(a.q_log2_base));
}
__device__ __forceinline__ void request_args(const DecodeArgs &a) {
  asm volatile("" ::"s"(a.out), "s"(a.q), "s"(a.k), "s"(a.v), "s"(a.kv_len), "s"(a.B), "s"(a.Hq), "s"(a.Hkv), "s"(a.Lmax), "s"(a.D));
  asm volatile("" ::"s"(a.qs[0]), "s"(a.qs[1]), "s"(a.os[0]), "s"(a.os[1]), "s"(a.ks[0]), "s"(a.ks[1]), "s"(a.ks[2]), "s"(a.vs[0]), "s"(a.vs[1]), "s"(a.vs[2]));
  asm volatile("" ::"s"(a.scale), "s"(a.head_map), "s"(a.out_f32), "s"(a.num_splits), "s"(a.chunk), "s"(a.ws_o), "s"(a.ws_ml), "s"(a.step), "s"(a.q_rope), "s"(a.rope_interleaved), "s"(a.rope_log2_base), "s"(a.k_new), "s"(a.v_new));
}
__device__ __forceinline__ void request_args(const RopeArgs &a) {
  asm volatile("" ::"s"(a.out), "s"(a.x), "s"(a.pos0), "s"(a.prev_seq), "s"(a.B), "s"(a.H), "s"(a.S), "s"(a.D), "s"(a.xs[0]), "s"(a.xs[1]), "s"(a.xs[2]), "s"(a.os[0]), "s"(a.os[1]), "s"(a.os[2]), "s"(a.log2_base), "s"(a.interleaved));
}
__device__ __forceinline__ void request_args(const KvAppendArgs &a) {
  asm volatile("" ::"s"(a.k_cache), "s"(a.v_cache), "s"(a.k_new), "s"(a.v_new), "s"(a.pos), "s"(a.pos_all), "s"(a.B), "s"(a.Hkv), "s"(a.T), "s"(a.D), "s"(a.Lmax));
  asm volatile("" ::"s"(a.ks[0]), "s"(a.ks[1]), "s"(a.ks[2]), "s"(a.vs[0]), "s"(a.vs[1]), "s"(a.vs[2]), "s"(a.rope_k), "s"(a.interleaved), "s"(a.log2_base), "s"(a.q), "s"(a.Hq));
}

__host__ __device__ inline int kv_head_of(int hq, int Hq, int Hkv, int head_map) {
  if (Hq == Hkv) return hq;
  return head_map == LMH_HEADMAP_BLOCKED ? hq / (Hq / Hkv) : hq % Hkv;
}

// Query head number `g` (0..G-1) of KV head `kvh`.
__host__ __device__ inline int q_head_of(int kvh, int g, int Hq, int Hkv, int head_map) {
  if (Hq == Hkv) return kvh;
  return head_map == LMH_HEADMAP_BLOCKED ? kvh * (Hq / Hkv) + g : kvh + Hkv * g;
}

// Launchers: validate nothing (api.hip already did), pick an instantiation, enqueue on `stream`.
// Return LMH_OK or LMH_E_UNSUPPORTED / LMH_E_HIP.
// The matrix-core kernels rotate Q in registers, which needs the partner of every element in the same lane: head dims
// that fill a tiling exactly (64, 96, 128).
inline bool prefill_mfma_rope_ok(int D) { return D == 64 || D == 96 || D == 128; }
bool prefill_mfma_supported(int dtype, int D);
int launch_prefill_mfma(const PrefillArgs &a, int dtype, hipStream_t stream);
#ifdef LMH_W64_KERNEL
// measurement builds only (prefill_mfma_w64.hip): the hand-pipelined 64-columns-per-wave kernel and the launches it takes
bool prefill_w64_takes(const PrefillArgs &a, int dtype);
int launch_prefill_w64(const PrefillArgs &a, hipStream_t stream);
#endif
bool prefill_f32_mfma_supported(int dtype, int D);
int launch_prefill_f32_mfma(const PrefillArgs &a, hipStream_t stream);
int launch_prefill_valu(const PrefillArgs &a, int dtype, hipStream_t stream);
int launch_decode(const DecodeArgs &a, int dtype, hipStream_t stream);
int launch_rope(const RopeArgs &a, int dtype, hipStream_t stream);
int launch_kv_append(const KvAppendArgs &a, int dtype, hipStream_t stream);
bool decode_mfma_supported(int dtype, int D, int B);
bool decode_mfma_rope_ok(int D, int interleaved);
int launch_decode_mfma_split(const DecodeArgs &a, int dtype, hipStream_t stream);

// Keys per split used for a given (Lmax, num_splits); always a multiple of 64.
int decode_chunk_for(int Lmax, int num_splits);

}  // namespace lmh
