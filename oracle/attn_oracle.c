/*
 * attn_oracle.c — CPU restatement of Luminal.jl's attention hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. Only the test-suite, the smoke check and the
 * benchmark's CPU-baseline leg may load this library, and only as the checker. The shipped
 * GPU library never links or calls anything in this file.
 *
 * What it restates (all reference paths are under the Luminal.jl source tree):
 *   lmo_flash_attn      <- flash_attn_cpu, src/Execution.jl:453-479: the same recurrence in the
 *                          same loop order (b, h, i, j), fp32 state (m_i, l_i, o_row), the NaN
 *                          guard on scale_old (:468-469), the causal skip `j > i` (:462) and the
 *                          final o_row ./ l_i (:475). Default scale 1/sqrt(D) is the builder's
 *                          (src/HighLevelOps.jl:377-388) and is applied by the caller.
 *     generalised along the three axes the reference only has as un-fused subgraphs:
 *       Sq != Sk   cross attention, src/Whisper.jl:299-316 and :628-645 (no mask)
 *       Hkv < Hq   GQA, src/NN.jl:305-317 (repeat_kv = Expand(dim 3) then Reshape, both executed
 *                  on column-major arrays: src/Execution.jl:238-248, :228, :287-296), which makes
 *                  query head hq read KV head hq % Hkv (LMO_HEADMAP_INTERLEAVED). The row-major
 *                  convention hq / G is offered as LMO_HEADMAP_BLOCKED.
 *       kv_len[b]  single-token decode over the first step_pos+1 rows of a (B,H,max_seq,D)
 *                  cache, src/Whisper.jl:584-620 (slice at :610-611) and :519-540.
 *   lmo_attn_naive_f64  <- the manual attention the reference's tests compare against
 *                          (tests/test_flash_attention_verification.jl:30-35, :60-70; model code
 *                          src/NN.jl:369-382): softmax(scale * Q K^T + mask) V, evaluated in
 *                          double precision with the max-subtracted softmax of
 *                          src/HighLevelOps.jl:313-319. It shares no code with lmo_flash_attn, so
 *                          an error in either shows up as a disagreement.
 *
 *   lmo_rope            <- apply_rotary_embeddings, src/NN.jl:253-303 (pairs (j, j+D/2) under the
 *                          reference's column-major reshape)
 *   lmo_kv_append       <- _kv_scatter, src/Whisper.jl:552-570, as an in-place row write
 *
 * Pinned by (tests/test_oracle.py): flash == naive-f64 to 1e-5 on the reference's test shape
 * (B=H=1,S=8,D=16; the reference's own criterion is rtol 1e-4,
 * tests/test_flash_attention_verification.jl:48); closed forms (row 0 == V[0], Q=0 -> running
 * mean of V, V=1 -> 1, single key -> that V row, logit-shift invariance); the GQA map against a
 * literal column-major replay of Expand+Reshape; decode == last row of causal prefill; and the
 * committed golden vectors under tests/golden/, which were produced by an independent numpy
 * float64 implementation. lmo_rope is pinned by a literal numpy replay of the reference's graph
 * on column-major arrays (reshape to (D/2,2), slice, rotate, concat, reshape back), by norm
 * preservation, the position-0 identity, additivity of positions and the relative-position
 * property of q.k; lmo_kv_append by a literal replay of the slice + concat of _kv_scatter.
 *
 * Layout: row-major [B, H, S, D] (D contiguous), all tensors fp32. Half-precision configs are
 * evaluated on inputs already rounded to fp16 / bf16 (lmo_round_f16 / lmo_round_bf16).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define LMO_HEADMAP_INTERLEAVED 0
#define LMO_HEADMAP_BLOCKED 1

static inline int kv_head_of(int hq, int Hq, int Hkv, int head_map) {
  if (Hq == Hkv) return hq;
  return head_map == LMO_HEADMAP_BLOCKED ? hq / (Hq / Hkv) : hq % Hkv;
}

int lmo_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* One (b, hq, i) query row of flash_attn_cpu (src/Execution.jl:457-475). */
static void flash_row(float *o_out, const float *q_row, const float *k_base, const float *v_base,
                      int64_t k_row_stride, int64_t v_row_stride, int n_keys, int D, float scale,
                      float *o_row) {
  float m_i = -INFINITY; /* :458 */
  float l_i = 0.0f;      /* :459 */
  for (int d = 0; d < D; d++) o_row[d] = 0.0f; /* :460 */
  for (int j = 0; j < n_keys; j++) {
    const float *k_row = k_base + (int64_t)j * k_row_stride;
    const float *v_row = v_base + (int64_t)j * v_row_stride;
    float dot = 0.0f;
    for (int d = 0; d < D; d++) dot += q_row[d] * k_row[d];
    dot *= scale; /* :464 */
    float m_next = m_i > dot ? m_i : dot; /* :466 */
    float p = expf(dot - m_next);         /* :467 */
    float scale_old = expf(m_i - m_next); /* :468 */
    if (isnan(scale_old)) scale_old = 0.0f; /* :469 */
    for (int d = 0; d < D; d++) o_row[d] = o_row[d] * scale_old + p * v_row[d]; /* :471 */
    l_i = l_i * scale_old + p; /* :472 */
    m_i = m_next;              /* :473 */
  }
  for (int d = 0; d < D; d++) o_out[d] = o_row[d] / l_i; /* :475 */
}

/*
 * out[B,Hq,Sq,D] = attention(q[B,Hq,Sq,D], k[B,Hkv,Sk,D], v[B,Hkv,Sk,D]).
 * kv_len may be NULL (all Sk keys valid) or int32[B] with 1 <= kv_len[b] <= Sk.
 * causal != 0 keeps key j for query i only when j <= i (0-based, as src/Execution.jl:462).
 * nthreads <= 1 runs the reference's single-threaded loop order; > 1 spreads (b, hq, i) rows
 * over OpenMP threads (rows are independent, results are bit-identical).
 * Returns 0, or -1 on bad arguments.
 */
int lmo_flash_attn(float *out, const float *q, const float *k, const float *v,
                   const int32_t *kv_len, int B, int Hq, int Hkv, int Sq, int Sk, int D,
                   float scale, int causal, int head_map, int nthreads) {
  if (!out || !q || !k || !v) return -1;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq <= 0 || Sk <= 0 || D <= 0) return -1;
  if (Hq % Hkv != 0) return -1;
  int64_t rows = (int64_t)B * Hq * Sq;
  if (nthreads < 1) nthreads = 1;
#ifdef _OPENMP
#pragma omp parallel num_threads(nthreads)
#endif
  {
    float *o_row = (float *)malloc(sizeof(float) * (size_t)D);
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 16)
#endif
    for (int64_t r = 0; r < rows; r++) {
      int i = (int)(r % Sq);
      int hq = (int)((r / Sq) % Hq);
      int b = (int)(r / ((int64_t)Sq * Hq));
      int kvh = kv_head_of(hq, Hq, Hkv, head_map);
      int n_keys = kv_len ? kv_len[b] : Sk;
      if (n_keys > Sk) n_keys = Sk;
      if (causal && n_keys > i + 1) n_keys = i + 1;
      const float *q_row = q + (((int64_t)b * Hq + hq) * Sq + i) * D;
      const float *k_base = k + (((int64_t)b * Hkv + kvh) * Sk) * D;
      const float *v_base = v + (((int64_t)b * Hkv + kvh) * Sk) * D;
      float *o_out = out + (((int64_t)b * Hq + hq) * Sq + i) * D;
      flash_row(o_out, q_row, k_base, v_base, D, D, n_keys, D, scale, o_row);
    }
    free(o_row);
  }
  return 0;
}

/*
 * Single-token decode over a cache: q[B,Hq,D], k_cache/v_cache[B,Hkv,Lmax,D], out[B,Hq,D].
 * Equals lmo_flash_attn with Sq = 1, causal = 0 and Sk = Lmax; kept as its own entry so the
 * benchmark can time exactly this case (src/Whisper.jl:610-616).
 */
int lmo_decode_attn(float *out, const float *q, const float *k_cache, const float *v_cache,
                    const int32_t *kv_len, int B, int Hq, int Hkv, int Lmax, int D, float scale,
                    int head_map, int nthreads) {
  return lmo_flash_attn(out, q, k_cache, v_cache, kv_len, B, Hq, Hkv, 1, Lmax, D, scale, 0,
                        head_map, nthreads);
}

/*
 * Independent second oracle: materialise the score row in double precision, add the mask as
 * "excluded", subtract the max, exponentiate, normalise, multiply by V. Output is double.
 */
int lmo_attn_naive_f64(double *out, const float *q, const float *k, const float *v,
                       const int32_t *kv_len, int B, int Hq, int Hkv, int Sq, int Sk, int D,
                       double scale, int causal, int head_map) {
  if (!out || !q || !k || !v) return -1;
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Sq <= 0 || Sk <= 0 || D <= 0 || Hq % Hkv != 0) return -1;
  int64_t rows = (int64_t)B * Hq * Sq;
#ifdef _OPENMP
#pragma omp parallel
#endif
  {
    double *w = (double *)malloc(sizeof(double) * (size_t)Sk);
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 16)
#endif
    for (int64_t r = 0; r < rows; r++) {
      int i = (int)(r % Sq);
      int hq = (int)((r / Sq) % Hq);
      int b = (int)(r / ((int64_t)Sq * Hq));
      int kvh = kv_head_of(hq, Hq, Hkv, head_map);
      int n_valid = kv_len ? kv_len[b] : Sk;
      const float *q_row = q + (((int64_t)b * Hq + hq) * Sq + i) * D;
      const float *k_base = k + (((int64_t)b * Hkv + kvh) * Sk) * D;
      const float *v_base = v + (((int64_t)b * Hkv + kvh) * Sk) * D;
      double *o = out + (((int64_t)b * Hq + hq) * Sq + i) * D;
      double mx = -INFINITY;
      for (int j = 0; j < Sk; j++) {
        int keep = (j < n_valid) && !(causal && j > i);
        if (!keep) { w[j] = -INFINITY; continue; }
        double s = 0.0;
        for (int d = 0; d < D; d++) s += (double)q_row[d] * (double)k_base[(int64_t)j * D + d];
        w[j] = s * scale;
        if (w[j] > mx) mx = w[j];
      }
      double sum = 0.0;
      for (int j = 0; j < Sk; j++) {
        w[j] = isinf(w[j]) && w[j] < 0 ? 0.0 : exp(w[j] - mx);
        sum += w[j];
      }
      for (int d = 0; d < D; d++) o[d] = 0.0;
      for (int j = 0; j < Sk; j++) {
        if (w[j] == 0.0) continue;
        double pj = w[j] / sum;
        for (int d = 0; d < D; d++) o[d] += pj * (double)v_base[(int64_t)j * D + d];
      }
    }
    free(w);
  }
  return 0;
}

/*
 * Rotary embedding, restating apply_rotary_embeddings (src/NN.jl:253-303) on row-major [B,H,S,D]:
 *   freqs = arange(D/2) * 2 / D; inv_freqs = 1 / exp2(freqs * log2(base))     (:261-263)
 *   pos = arange(S) + prev_seq; emb[s][j] = pos[s] * inv_freqs[j]              (:265-270)
 *   the input is reshaped to (B,H,S,D/2,2) in COLUMN-major order and split on the last axis
 *   (:274-276), so x0 = x[.., j] and x1 = x[.., j + D/2];
 *   x0' = x0 cos - x1 sin, x1' = x0 sin + x1 cos                                (:292-293)
 * interleaved != 0 pairs (2j, 2j+1) instead. pos0 (int32[B]) overrides prev_seq per sequence.
 */
int lmo_rope(float *out, const float *x, const int32_t *pos0, int prev_seq, int B, int H, int S, int D,
             float base, int interleaved) {
  if (!out || !x || B <= 0 || H <= 0 || S <= 0 || D <= 0 || D % 2 != 0) return -1;
  const int half = D / 2;
  const float log2_base = log2f(base);
  for (int b = 0; b < B; b++)
    for (int h = 0; h < H; h++)
      for (int s = 0; s < S; s++) {
        const float *xr = x + (((int64_t)b * H + h) * S + s) * D;
        float *orow = out + (((int64_t)b * H + h) * S + s) * D;
        const float pos = (float)((pos0 ? pos0[b] : prev_seq) + s);
        for (int j = 0; j < half; j++) {
          const float freq = (float)j * 2.0f / (float)D;
          const float inv_freq = 1.0f / exp2f(freq * log2_base);
          const float ang = pos * inv_freq;
          const int d0 = interleaved ? 2 * j : j, d1 = interleaved ? 2 * j + 1 : j + half;
          const float x0 = xr[d0], x1 = xr[d1];
          orow[d0] = x0 * cosf(ang) - x1 * sinf(ang);
          orow[d1] = x0 * sinf(ang) + x1 * cosf(ang);
        }
      }
  return 0;
}

/*
 * KV-cache append, the in-place equivalent of _kv_scatter (src/Whisper.jl:552-570):
 * cache[b,h,pos[b]+t,:] = new[b,h,t,:]; every other row unchanged. cache [B,H,Lmax,D], new [B,H,T,D].
 */
int lmo_kv_append(float *cache, const float *new_rows, const int32_t *pos, int B, int H, int T, int D, int Lmax) {
  if (!cache || !new_rows || !pos || B <= 0 || H <= 0 || T <= 0 || D <= 0 || Lmax <= 0) return -1;
  for (int b = 0; b < B; b++)
    for (int h = 0; h < H; h++)
      for (int t = 0; t < T; t++) {
        const int row = pos[b] + t;
        if (row < 0 || row >= Lmax) continue;
        memcpy(cache + (((int64_t)b * H + h) * Lmax + row) * D, new_rows + (((int64_t)b * H + h) * T + t) * D,
               sizeof(float) * (size_t)D);
      }
  return 0;
}

/* ------------------------------------------------------------------------------------------
 * Deterministic input generator shared by the oracle, the tests and the benchmark:
 * SplitMix64 stream -> pairs of uniforms -> Box-Muller normals, computed in double and
 * rounded once to fp32. Element e of a stream with seed s depends only on (s, e / 2), so
 * any sub-range can be generated independently.
 * ---------------------------------------------------------------------------------------- */
static inline uint64_t splitmix64_at(uint64_t seed, uint64_t index) {
  uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

void lmo_gen_normal(float *out, uint64_t n, uint64_t seed, float mul) {
  const double two_pi = 6.283185307179586476925286766559;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int64_t pair = 0; pair < (int64_t)((n + 1) / 2); pair++) {
    uint64_t a = splitmix64_at(seed, 2 * (uint64_t)pair);
    uint64_t b = splitmix64_at(seed, 2 * (uint64_t)pair + 1);
    double u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740992.0); /* (0, 1] */
    double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);         /* [0, 1) */
    double r = sqrt(-2.0 * log(u1));
    out[2 * pair] = (float)(r * cos(two_pi * u2)) * mul;
    if ((uint64_t)(2 * pair + 1) < n) out[2 * pair + 1] = (float)(r * sin(two_pi * u2)) * mul;
  }
}

/* uniform integers in [lo, hi] from the same stream (ragged kv lengths) */
void lmo_gen_uniform_int(int32_t *out, uint64_t n, uint64_t seed, int32_t lo, int32_t hi) {
  uint64_t span = (uint64_t)(hi - lo) + 1;
  for (uint64_t i = 0; i < n; i++) out[i] = lo + (int32_t)(splitmix64_at(seed, i) % span);
}

/* round-to-nearest-even to bf16 / fp16 precision, result kept as fp32 */
void lmo_round_bf16(float *x, uint64_t n) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int64_t i = 0; i < (int64_t)n; i++) {
    uint32_t u;
    memcpy(&u, &x[i], 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) { u |= 0x00400000u; u &= 0xffff0000u; }
    else { u += 0x7fffu + ((u >> 16) & 1u); u &= 0xffff0000u; }
    memcpy(&x[i], &u, 4);
  }
}

/* fp32 -> nearest fp16 (ties to even, subnormals and overflow to inf handled) -> fp32 */
static float round_one_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t sign = u & 0x80000000u;
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return f; /* inf / nan unchanged */
  float af;
  memcpy(&af, &a, 4);
  if (af >= 65520.0f) { /* rounds to infinity */
    uint32_t inf = sign | 0x7f800000u;
    memcpy(&f, &inf, 4);
    return f;
  }
  if (af < 6.103515625e-05f) { /* below the smallest normal fp16: spacing 2^-24 */
    float r = nearbyintf(af * 16777216.0f) * (1.0f / 16777216.0f); /* default mode: ties to even */
    uint32_t ru;
    memcpy(&ru, &r, 4);
    ru |= sign;
    memcpy(&f, &ru, 4);
    return f;
  }
  a += 0x0fffu + ((a >> 13) & 1u); /* keep 10 mantissa bits, ties to even */
  a &= 0xffffe000u;
  a |= sign;
  memcpy(&f, &a, 4);
  return f;
}

void lmo_round_f16(float *x, uint64_t n) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (int64_t i = 0; i < (int64_t)n; i++) x[i] = round_one_f16(x[i]);
}
