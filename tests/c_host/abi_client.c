/* A consumer of libluminal_hip.so that is not Python: plain C99 against include/luminal_hip.h only, the way a host written in
 * a compiled language (or Julia's ccall) binds it. Runs one non-causal cross attention, one causal GQA attention and one
 * split-KV decode in fp32 and checks them against a float64 softmax(scale QK^T + mask) V computed here.
 * Exit status: 0 = all within 1e-5 of the output range, 1 = mismatch or library error, 77 = no device to run on. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "luminal_hip.h"

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float next_uniform(void) { /* xorshift64*, [-1, 1) */
  rng_state ^= rng_state >> 12;
  rng_state ^= rng_state << 25;
  rng_state ^= rng_state >> 27;
  return (float)((double)((rng_state * 0x2545F4914F6CDD1Dull) >> 11) / 4503599627370496.0 - 1.0);
}
static float *random_tensor(size_t n) {
  float *p = (float *)malloc(n * sizeof(float));
  size_t i;
  for (i = 0; i < n; i++) p[i] = next_uniform();
  return p;
}

#define CHECK(call)                                                              \
  do {                                                                           \
    int rc_ = (call);                                                            \
    if (rc_ != LMH_OK) {                                                         \
      fprintf(stderr, "%s -> %d: %s\n", #call, rc_, lmh_last_error());           \
      return 1;                                                                  \
    }                                                                            \
  } while (0)

/* reference: q [B,Hq,Sq,D], k/v [B,Hkv,Sk,D], KV head of hq = hq % Hkv, keys limited to len[b] (and to j <= i if causal) */
static void reference(double *out, const float *q, const float *k, const float *v, const int32_t *len, int B, int Hq, int Hkv,
                      int Sq, int Sk, int D, double scale, int causal) {
  int b, h, i, j, d;
  double *w = (double *)malloc((size_t)Sk * sizeof(double));
  for (b = 0; b < B; b++)
    for (h = 0; h < Hq; h++)
      for (i = 0; i < Sq; i++) {
        const float *qr = q + (((size_t)b * Hq + h) * Sq + i) * D;
        const float *kb = k + ((size_t)b * Hkv + h % Hkv) * Sk * D, *vb = v + ((size_t)b * Hkv + h % Hkv) * Sk * D;
        int n = len ? len[b] : Sk;
        double m = -INFINITY, l = 0.0;
        double *o = out + (((size_t)b * Hq + h) * Sq + i) * D;
        if (causal && n > i + 1) n = i + 1;
        for (j = 0; j < n; j++) {
          double s = 0.0;
          for (d = 0; d < D; d++) s += (double)qr[d] * kb[(size_t)j * D + d];
          w[j] = s * scale;
          if (w[j] > m) m = w[j];
        }
        for (j = 0; j < n; j++) l += (w[j] = exp(w[j] - m));
        for (d = 0; d < D; d++) o[d] = 0.0;
        for (j = 0; j < n; j++)
          for (d = 0; d < D; d++) o[d] += w[j] / l * vb[(size_t)j * D + d];
      }
  free(w);
}

static double max_rel_err(const float *got, const double *want, size_t n) {
  double err = 0.0, top = 0.0;
  size_t i;
  for (i = 0; i < n; i++) {
    if (fabs(got[i] - want[i]) > err) err = fabs(got[i] - want[i]);
    if (fabs(want[i]) > top) top = fabs(want[i]);
  }
  return err / top;
}

static int to_device(void **dev, const void *host, size_t bytes) {
  CHECK(lmh_malloc(dev, bytes));
  CHECK(lmh_memcpy_h2d(*dev, host, bytes, NULL));
  return 0;
}

static int prefill_case(const char *name, int B, int Hq, int Hkv, int Sq, int Sk, int D, int causal) {
  const size_t nq = (size_t)B * Hq * Sq * D, nk = (size_t)B * Hkv * Sk * D;
  float *q = random_tensor(nq), *k = random_tensor(nk), *v = random_tensor(nk), *got = (float *)malloc(nq * sizeof(float));
  double *want = (double *)malloc(nq * sizeof(double));
  void *dq, *dk, *dv, *dout;
  lmh_attn_params p;
  double err;
  if (to_device(&dq, q, nq * 4) || to_device(&dk, k, nk * 4) || to_device(&dv, v, nk * 4)) return 1;
  CHECK(lmh_malloc(&dout, nq * 4));
  memset(&p, 0, sizeof(p)); /* zero strides = contiguous, stream 0, no kv_len */
  p.out = dout; p.q = dq; p.k = dk; p.v = dv;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Sq = Sq; p.Sk = Sk; p.D = D;
  p.dtype = LMH_F32; p.scale = (float)(1.0 / sqrt((double)D)); p.causal = causal; p.head_map = LMH_HEADMAP_INTERLEAVED;
  CHECK(lmh_flash_attn_fwd(&p));
  CHECK(lmh_memcpy_d2h(got, dout, nq * 4, NULL));
  reference(want, q, k, v, NULL, B, Hq, Hkv, Sq, Sk, D, (double)p.scale, causal);
  err = max_rel_err(got, want, nq);
  printf("%s: max err / max|out| = %.3g\n", name, err);
  CHECK(lmh_free(dq)); CHECK(lmh_free(dk)); CHECK(lmh_free(dv)); CHECK(lmh_free(dout));
  free(q); free(k); free(v); free(got); free(want);
  return err <= 1e-5 ? 0 : 1;
}

static int decode_case(int B, int Hq, int Hkv, int Lmax, int D, int num_splits) {
  const size_t nq = (size_t)B * Hq * D, nk = (size_t)B * Hkv * Lmax * D;
  float *q = random_tensor(nq), *k = random_tensor(nk), *v = random_tensor(nk), *got = (float *)malloc(nq * sizeof(float));
  double *want = (double *)malloc(nq * sizeof(double));
  int32_t *len = (int32_t *)malloc((size_t)B * sizeof(int32_t));
  void *dq, *dk, *dv, *dout, *dlen, *ws = NULL;
  size_t ws_bytes;
  lmh_decode_params p;
  double err;
  int b;
  for (b = 0; b < B; b++) len[b] = 1 + (int32_t)((b * 977 + 313) % Lmax);
  if (to_device(&dq, q, nq * 4) || to_device(&dk, k, nk * 4) || to_device(&dv, v, nk * 4) || to_device(&dlen, len, (size_t)B * 4)) return 1;
  CHECK(lmh_malloc(&dout, nq * 4));
  ws_bytes = lmh_decode_workspace_bytes(B, Hq, Hkv, Lmax, D, num_splits);
  if (ws_bytes) CHECK(lmh_malloc(&ws, ws_bytes));
  memset(&p, 0, sizeof(p));
  p.out = dout; p.q = dq; p.k_cache = dk; p.v_cache = dv; p.kv_len = (const int32_t *)dlen;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.Lmax = Lmax; p.D = D;
  p.dtype = LMH_F32; p.scale = (float)(1.0 / sqrt((double)D)); p.head_map = LMH_HEADMAP_INTERLEAVED;
  p.num_splits = num_splits; p.workspace = ws; p.workspace_bytes = ws_bytes;
  CHECK(lmh_decode_attn(&p));
  CHECK(lmh_memcpy_d2h(got, dout, nq * 4, NULL));
  reference(want, q, k, v, len, B, Hq, Hkv, 1, Lmax, D, (double)p.scale, 0);
  err = max_rel_err(got, want, nq);
  printf("decode B=%d Hq=%d Hkv=%d Lmax=%d D=%d splits=%d: max err / max|out| = %.3g\n", B, Hq, Hkv, Lmax, D, num_splits, err);
  CHECK(lmh_free(dq)); CHECK(lmh_free(dk)); CHECK(lmh_free(dv)); CHECK(lmh_free(dout)); CHECK(lmh_free(dlen));
  if (ws) CHECK(lmh_free(ws));
  free(q); free(k); free(v); free(got); free(want); free(len);
  return err <= 1e-5 ? 0 : 1;
}

int main(void) {
  int bad = 0;
  printf("libluminal_hip version %d, %d device(s)\n", lmh_version(), lmh_device_count());
  if (lmh_device_count() < 1) return 77;
  CHECK(lmh_init(0));
  bad |= prefill_case("cross attention B=2 H=3 Sq=40 Sk=70 D=64", 2, 3, 3, 40, 70, 64, 0);
  bad |= prefill_case("causal GQA B=1 Hq=4 Hkv=2 S=130 D=32", 1, 4, 2, 130, 130, 32, 1);
  bad |= decode_case(3, 8, 2, 700, 64, 0);
  bad |= decode_case(2, 4, 4, 300, 128, 1);
  CHECK(lmh_sync(NULL));
  puts(bad ? "FAILED" : "ok");
  return bad;
}
