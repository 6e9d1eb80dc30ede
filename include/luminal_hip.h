/*
 * luminal_hip.h — C ABI of libluminal_hip.so, the MI355X (gfx950) backend for the
 * attention hot path of Luminal.jl.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, never throws, never
 * aborts, and returns LMH_OK (0) or a negative LMH_E_* code; lmh_last_error() then holds a
 * human-readable message (thread-local). The library keeps no pointer past a call and
 * allocates nothing inside the attention entry points: outputs and the decode workspace are
 * caller-owned, exactly like the pre-allocated node buffers the reference's compiled graph
 * hands to execute_op! (reference src/Compiler.jl:218-255).
 *
 * Tensor layout: row-major [B, H, S, D] addressed through element strides for (b, h, s);
 * the innermost (D) stride must be 1. A Julia (B,H,S,D) array is column-major, so the Julia
 * glue uploads permutedims(x, (4,3,2,1)).
 */
#ifndef LUMINAL_HIP_H
#define LUMINAL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LMH_VERSION 105 /* major*10000 + minor*100 + patch */

/* status codes */
#define LMH_OK 0
#define LMH_E_NULL (-1)        /* a required pointer is null */
#define LMH_E_SHAPE (-2)       /* non-positive or inconsistent dimension / stride */
#define LMH_E_UNSUPPORTED (-3) /* head dim / dtype / head map not implemented */
#define LMH_E_WORKSPACE (-4)   /* decode workspace missing, too small or not 16-byte aligned */
#define LMH_E_HIP (-5)         /* a HIP runtime call failed */
#define LMH_E_NODEVICE (-6)    /* no usable gfx950 device */
#define LMH_E_BUSY (-7)        /* the static scratch is still in use by a call on another stream */

/* element type of q/k/v/out; accumulation is always fp32 */
#define LMH_F32 0
#define LMH_F16 1
#define LMH_BF16 2
/* out_f32 (a field of both parameter blocks): 0 writes the result in the input element type,
 * 1 writes fp32. A bf16 result carries a rounding error of up to 2^-8 of its magnitude on its
 * own, more than the 2e-3 parity budget of the half-precision configurations, so bf16 callers
 * that need that budget ask for fp32.
 * The softmax weights reach the matrix cores with 11 (fp16) or 16 (bf16, head + remainder) significant bits.
 * bf16 flash attention with long rows (from about 512 keys per query row on; lmh_flash_attn_plan ends in
 * "V as fp16") rounds the weights to 11 bits and hands V over as fp16, rewritten exactly tile by tile relative to
 * the largest finite |v| staged so far by the row's workgroup (128 or 256 query rows; the keys the causal mask hides from
 * the row but not from the workgroup's last row included):
 * values more than 2^29 below it count as zero; infinities and NaNs stay what they are. */

/* which KV head a query head reads.
 * INTERLEAVED: hq % Hkv — what the reference's repeat_kv produces, because its
 *   Expand(dim 3) + Reshape run on column-major arrays (reference src/NN.jl:305-317,
 *   src/Execution.jl:238-248, :228).
 * BLOCKED: hq / (Hq/Hkv) — the row-major (HuggingFace) convention. */
#define LMH_HEADMAP_INTERLEAVED 0
#define LMH_HEADMAP_BLOCKED 1

/* which elements of a row the rotary embedding rotates together (lmh_rope, lmh_kv_append, lmh_attn_params.q_rope).
 * HALF_SPLIT: (j, j + D/2), what the reference's column-major reshape to (D/2, 2) produces
 *   (reference src/NN.jl:253-303). INTERLEAVED: (2j, 2j+1). */
#define LMH_ROPE_HALF_SPLIT 0
#define LMH_ROPE_INTERLEAVED 1

/* ---- runtime plumbing: replaces CUDA.functional()/CuArray()/Array() in the reference's
 * device layer (reference src/Device.jl:31-74 get_device, :82-96 to_device, :103-105
 * from_device). ---- */
int lmh_version(void);
/* 1 when the library was compiled with experiment switches (a measurement build, whose kernels may compute
 * wrong results on purpose), 0 for the product. Hosts refuse a library that answers 1. */
int lmh_measurement_build(void);
const char *lmh_last_error(void);
/* number of visible gfx950 devices; 0 when there is none (never an error) */
int lmh_device_count(void);
/* select the device and run the health check get_device() does (a 4-byte alloc+free) */
int lmh_init(int device);
int lmh_device_name(char *buf, size_t buf_bytes);
int lmh_malloc(void **dev_ptr, size_t bytes);
int lmh_free(void *dev_ptr);
int lmh_memset(void *dev_ptr, int byte_value, size_t bytes, void *stream);
int lmh_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, void *stream);
/* copies and then synchronises the stream, like Array(::CuArray) */
int lmh_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, void *stream);
int lmh_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes, void *stream);
int lmh_sync(void *stream);
/* HIP-event timing on a stream (for benchmarks) */
int lmh_event_create(void **event);
int lmh_event_destroy(void *event);
int lmh_event_record(void *event, void *stream);
int lmh_event_elapsed_ms(float *ms, void *start, void *stop);

/* ---- a compiled step list as one launch: what execute_with_capture(device, f, cache) is meant to do
 * in the reference (reference src/Device.jl:108-121, called from the compiled step closure at
 * src/Compiler.jl:98; stubbed out there because freed transient workspaces invalidated the recording).
 * Every entry point above enqueues on the stream it is given and allocates nothing, so a sequence of
 * them on persistent buffers can be recorded once into a HIP graph and replayed; per-step values
 * (positions, lengths) live in device memory, so one recording serves every decode position.
 *   lmh_stream_create      a stream that can be captured (the null stream cannot); default priority,
 *                          blocking with respect to the null stream
 *   lmh_graph_capture_begin / _end   record what is enqueued on `stream` in between; _end returns an
 *                          executable graph (and must be called even after a failed call in between)
 *   lmh_graph_launch       replay on `stream`
 * Nothing may be allocated, freed, copied to the host or synchronised on the capturing stream between
 * begin and end, and lmh_memset stays outside (it would record a memset node; clear buffers before the
 * capture or with a kernel). ---- */
int lmh_stream_create(void **stream);
int lmh_stream_destroy(void *stream);
int lmh_graph_capture_begin(void *stream);
int lmh_graph_capture_end(void *stream, void **graph_exec);
int lmh_graph_launch(void *graph_exec, void *stream);
int lmh_graph_destroy(void *graph_exec);

/* ---- flash attention forward: replaces
 *   execute_op!(out, op::FlashAttentionOp, q, k, v)   reference src/Execution.jl:565-578
 *   flash_attn_cpu(q, k, v, scale, causal)            reference src/Execution.jl:453-479
 * generalised to Sq != Sk (cross attention, reference src/Whisper.jl:299-316) and to
 * Hkv < Hq (GQA, reference src/NN.jl:305-317, :362-382).
 *
 * out[b,hq,i,:] = sum_j softmax_j(scale * q[b,hq,i,:] . k[b,kvh,j,:]) v[b,kvh,j,:]
 * with j restricted to j <= i when causal != 0 (the reference skips j > i,
 * src/Execution.jl:462), and to j < kv_len[b] when kv_len is non-null.
 * Head dims up to 256, like decode. The matrix-core kernels take multiples of 8 up to 128 (with 16-byte
 * aligned pointers and strides, scale > 0); everything else runs on a vector-ALU kernel with the same
 * results at a fraction of the speed. ---- */
typedef struct lmh_attn_params {
  void *out;          /* [B,Hq,Sq,D] device */
  const void *q;      /* [B,Hq,Sq,D] device */
  const void *k;      /* [B,Hkv,Sk,D] device */
  const void *v;      /* [B,Hkv,Sk,D] device */
  const int32_t *kv_len; /* optional device int32[B]: valid keys per sequence (0..Sk; 0 writes zeros); null = Sk */
  int32_t B, Hq, Hkv, Sq, Sk, D;
  int64_t q_stride[3]; /* element strides for (b, h, s); all-zero = contiguous */
  int64_t k_stride[3];
  int64_t v_stride[3];
  int64_t o_stride[3];
  int32_t dtype;    /* element type of q, k, v: LMH_F32 / LMH_F16 / LMH_BF16 */
  float scale;      /* FlashAttentionOp.scale, reference src/Ops.jl:104-107 */
  int32_t causal;   /* FlashAttentionOp.causal */
  int32_t head_map; /* LMH_HEADMAP_* */
  int32_t out_f32;  /* 0: out has element type `dtype`; 1: out is fp32 */
  void *stream;     /* hipStream_t, null = default stream */
  /* Optional: the rotary embedding of the queries, which the reference applies directly in front of attention
   * (reference src/NN.jl:357, apply_rotary_embeddings :253-303), done on the rows as the kernel loads them instead of
   * by a launch of lmh_rope on q: row i of sequence b is rotated at position (q_pos0 ? q_pos0[b] : q_prev_seq) + i and
   * rounded to `dtype`, exactly what lmh_rope would have stored; q itself is not modified. K is not rotated here
   * (lmh_kv_append rotates it on its way into a cache, lmh_rope anywhere else). D must be even; head dims 64, 96 and
   * 128 keep the matrix-core kernels, any other runs on the vector-ALU kernel. Last in the struct so that
   * zero-initialised params of earlier callers keep their meaning. */
  int32_t q_rope;         /* 0 / 1 */
  int32_t q_rope_pairing; /* LMH_ROPE_* */
  const int32_t *q_pos0;  /* optional device int32[B]: position of row 0 per sequence; null = q_prev_seq */
  int32_t q_prev_seq;
  float q_rope_base;      /* 10000 in the reference */
} lmh_attn_params;

int lmh_flash_attn_fwd(const lmh_attn_params *p);

/* Which kernel lmh_flash_attn_fwd would launch for `p` (instantiation, workgroup count), as text in `plan`; nothing
 * is launched and no tensor is touched. Same validation and return codes as lmh_flash_attn_fwd. No counterpart in the
 * reference: a test and bench aid (which shapes reach which kernel). */
int lmh_flash_attn_plan(const lmh_attn_params *p, char *plan, size_t plan_bytes);

/* ---- single-token decode attention over a KV cache: replaces the un-fused subgraph
 *   whisper_self_attn_cached  reference src/Whisper.jl:584-620 (slice 0:step_pos+1, matmul,
 *   softmax, matmul) and whisper_cross_attn_cached :628-645, over a cache laid out like
 *   KVCacheState :519-540, i.e. (B, H, max_seq, D); with GQA per reference src/NN.jl:305-317.
 *
 * out[b,hq,:] = sum_{j < kv_len[b]} softmax_j(scale * q[b,hq,:] . K[b,kvh,j,:]) V[b,kvh,j,:]
 * Rows j >= kv_len[b] of the cache are never read into the result. ---- */
typedef struct lmh_decode_params {
  void *out;             /* [B,Hq,D] device */
  const void *q;         /* [B,Hq,D] device */
  const void *k_cache;   /* [B,Hkv,Lmax,D] device */
  const void *v_cache;   /* [B,Hkv,Lmax,D] device */
  const int32_t *kv_len; /* device int32[B], each in 1..Lmax; null = Lmax for every b */
  int32_t B, Hq, Hkv, Lmax, D;
  int64_t q_stride[2];   /* (b, h); all-zero = contiguous */
  int64_t o_stride[2];
  int64_t k_stride[3];   /* (b, h, s); all-zero = contiguous */
  int64_t v_stride[3];
  int32_t dtype;         /* element type of q and the caches */
  float scale;
  int32_t head_map;
  int32_t out_f32;       /* 0: out has element type `dtype`; 1: out is fp32 */
  int32_t num_splits;    /* KV splits per (b, kv head); 0 = choose */
  void *workspace;       /* device, 16-byte aligned, >= lmh_decode_workspace_bytes(...) */
  size_t workspace_bytes;
  void *stream;
} lmh_decode_params;

/* bytes of split-KV partial storage lmh_decode_attn needs for these sizes (0 on bad input) */
size_t lmh_decode_workspace_bytes(int32_t B, int32_t Hq, int32_t Hkv, int32_t Lmax, int32_t D,
                                  int32_t num_splits);
/* the split count lmh_decode_attn uses when num_splits == 0 */
int32_t lmh_decode_auto_splits(int32_t B, int32_t Hkv, int32_t Lmax);
int lmh_decode_attn(const lmh_decode_params *p);

/* ---- one decode step of a cached attention layer in two launches: append + attend.
 * Replaces, for one layer, what decode_step! does with the self-attention caches (reference
 * src/Whisper.jl:761-801: feed the caches in, run whisper_self_attn_cached :584-620, take the rebuilt caches
 * out) and the rotary embedding of this step's q and k in front of it (src/NN.jl:356-358).
 * `p` is the parameter block of lmh_decode_attn with these differences:
 *   - kv_len is required: kv_len[b] = rows already in the caches = the row this step writes, 0 <= kv_len[b] < Lmax
 *     (a sequence whose cache is full attends its old rows only and writes nothing);
 *   - k_cache / v_cache are written: row kv_len[b] of every KV head receives x->k_new (rotated when x->rope)
 *     and x->v_new; out = attention of q over rows 0 .. kv_len[b] inclusive. q itself is not modified.
 *   - num_splits == 0 takes lmh_decode_step_splits(); an explicit count must be >= 2; the workspace is
 *     lmh_decode_workspace_bytes(..., that count).
 * The first launch is the split kernel of lmh_decode_attn over the old rows, rotating q as it loads it; the second
 * merges the partials, adds the new row from k_new / v_new and stores it into the caches, so the separate append
 * launch (lmh_kv_append) disappears. fp16 / bf16 on the matrix-core decode kernel only (head dims 64, 128, 256;
 * 96 with the interleaved pairing); anything else returns LMH_E_UNSUPPORTED and the caller uses
 * lmh_kv_append + lmh_decode_attn. The caller advances kv_len afterwards. */
typedef struct lmh_decode_step_extra {
  const void *k_new;  /* device [B, Hkv, D], contiguous, element type of the caches: this step's key rows */
  const void *v_new;  /* device [B, Hkv, D]: this step's value rows */
  int32_t rope;       /* 1: rotate q and k_new at position kv_len[b] */
  int32_t pairing;    /* LMH_ROPE_HALF_SPLIT / LMH_ROPE_INTERLEAVED */
  float rope_base;    /* e.g. 10000 */
} lmh_decode_step_extra;
int32_t lmh_decode_step_splits(int32_t B, int32_t Hkv, int32_t Lmax);
int lmh_decode_step(const lmh_decode_params *p, const lmh_decode_step_extra *x);

/* ---- decode attention that allocates nothing and takes no workspace. No counterpart in the reference: it
 * is lmh_decode_attn for callers that cannot call hipMalloc (code under HIP graph capture, tight serving
 * loops, harnesses that forbid allocation). Same parameter block, same kernels, same results; `workspace`
 * and `workspace_bytes` are ignored. The split-KV partials go to a static device array of
 * LMH_STATIC_SCRATCH_BYTES that each GPU the library runs on holds until the process ends.
 *   - num_splits == 0 takes lmh_decode_static_splits(): the split count of lmh_decode_attn, halved until
 *     the partials fit. An explicit num_splits whose partials (lmh_decode_workspace_bytes) exceed the
 *     array is rejected with LMH_E_WORKSPACE.
 *   - Every call on one GPU shares that GPU's array, which keeps the last call's contents. Nothing in it
 *     has to start at zero (each call writes every slot it later reads), so none is cleared; calls that
 *     overlap in time on one GPU race on it and must be ordered by the caller. One stream orders its own
 *     calls. A call on a second (non-null) stream while the previous user is still running is refused with
 *     LMH_E_BUSY (the library records an event behind every eager call and queries it; no allocation). Calls
 *     recorded into a HIP graph cannot be checked this way: a replay must not overlap another user of the array.
 *   - The array is part of the library's code object: every process that loads the library holds
 *     LMH_STATIC_SCRATCH_BYTES of device memory on each GPU it initialises, whether or not this entry point is
 *     ever called.
 *   - lmh_init(device) resolves the array's address on that device; a device that was never passed to
 *     lmh_init resolves it on its first call here, which may load the code object (do that before a capture).
 * No hipMalloc, hipFree or other allocating call is made. ---- */
#define LMH_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
size_t lmh_static_scratch_bytes(void);
int32_t lmh_decode_static_splits(int32_t B, int32_t Hq, int32_t Hkv, int32_t Lmax, int32_t D);
int lmh_decode_attn_static(const lmh_decode_params *p);

/* ---- rotary position embedding: replaces the ~25-node subgraph of
 *   apply_rotary_embeddings(input, prev_seq; base)    reference src/NN.jl:253-303
 * out[b,h,s,:] = rotate(x[b,h,s,:], position = (pos0 ? pos0[b] : prev_seq) + s); out may alias x.
 * pairing: LMH_ROPE_* (above). D must be even. ---- */
typedef struct lmh_rope_params {
  void *out;           /* [B,H,S,D] device */
  const void *x;       /* [B,H,S,D] device */
  const int32_t *pos0; /* optional device int32[B]; null = prev_seq for every sequence */
  int32_t prev_seq;
  int32_t B, H, S, D;
  int64_t x_stride[3]; /* (b, h, s); all-zero = contiguous */
  int64_t o_stride[3];
  int32_t dtype;
  float base;          /* 10000 in the reference */
  int32_t pairing;     /* LMH_ROPE_* */
  void *stream;
} lmh_rope_params;
int lmh_rope(const lmh_rope_params *p);

/* ---- in-place KV-cache append: replaces
 *   _kv_scatter(past, new_slot, step_pos)              reference src/Whisper.jl:552-570
 * (a slice + concat rebuild of the whole (B,H,max_seq,D) cache) and the per-step host round trip of
 * decode_step!, reference src/Whisper.jl:775-797.
 * cache[b,h,pos+t,:] = new[b,h,t,:] for t < T, pos = pos ? pos[b] : pos_all; rows that would fall
 * outside 0..Lmax-1 are dropped. With rope_k != 0, K is rotated by its row position while it is
 * written (V never is). ---- */
typedef struct lmh_kv_append_params {
  void *k_cache;        /* [B,Hkv,Lmax,D] device, updated in place */
  void *v_cache;
  const void *k_new;    /* [B,Hkv,T,D] device, contiguous */
  const void *v_new;
  const int32_t *pos;   /* optional device int32[B]: first row to write per sequence */
  int32_t pos_all;      /* used when pos is null */
  int32_t B, Hkv, T, D, Lmax;
  int64_t k_stride[3];  /* cache strides (b, h, s); all-zero = contiguous */
  int64_t v_stride[3];
  int32_t dtype;
  int32_t rope_k;       /* 0 / 1 */
  int32_t pairing;      /* LMH_ROPE_*, used when rope_k != 0 or q_rope is given */
  float base;
  void *stream;
  /* Optional, for a decode step: this step's queries [B,Hq,T,D] (device, contiguous), rotated in place at the
   * same positions pos + t with `pairing` and `base` (whatever rope_k says) — saves the separate lmh_rope
   * launch of apply_rotary_embeddings on q (reference src/NN.jl:253-303, called on the queries at :356).
   * Null = none. Last in the struct so that zero-initialised params of earlier callers keep their meaning. */
  void *q_rope;
  int32_t Hq;
} lmh_kv_append_params;
int lmh_kv_append(const lmh_kv_append_params *p);

#ifdef __cplusplus
}
#endif
#endif /* LUMINAL_HIP_H */
