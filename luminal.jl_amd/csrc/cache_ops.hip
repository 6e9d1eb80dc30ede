// The two operators that sit directly in front of attention on the decode path:
//
//   rotary embedding   apply_rotary_embeddings, reference src/NN.jl:253-303. The reference reshapes
//     the head dim to (D/2, 2) on a column-major array, so the rotated pairs are (j, j + D/2), the
//     "half-split" convention; inv_freq[j] = base^(-2j/D), angle = (prev_seq + s) * inv_freq[j],
//     x0' = x0 cos - x1 sin, x1' = x0 sin + x1 cos. The interleaved pairing (2j, 2j+1) is offered too.
//   KV-cache append    _kv_scatter, reference src/Whisper.jl:552-570, which rebuilds the whole
//     (B, H, max_seq, D) cache by slice + concat to insert one row at step_pos. Here the new rows
//     are written in place at pos[b] .. pos[b]+T-1 (per-sequence positions, device int32[B]), with
//     the rotary embedding of K optionally fused into the same pass.
//
// Both are a few bytes of traffic per element and purely HBM/latency-bound; one thread handles one
// rotated pair (rope) or one 16-byte chunk (append).
#include "common.hpp"
#include "dtypes.hpp"

namespace lmh {
namespace {

template <typename E>
__device__ inline void rope_pair(float x0, float x1, float pos, int j, int D, float log2_base, float *o0, float *o1) {
  // inv_freq = 1 / exp2((2j/D) * log2(base)), evaluated as the reference does (src/NN.jl:262-263)
  const float freq = (float)j * 2.0f / (float)D;
  const float inv_freq = 1.0f / exp2f(freq * log2_base);
  float sn, cs;
  sincosf(pos * inv_freq, &sn, &cs);
  *o0 = x0 * cs - x1 * sn;
  *o1 = x0 * sn + x1 * cs;
}

template <typename E>
__global__ __launch_bounds__(256) void rope_kernel(RopeArgs a) {
  using raw = typename E::raw;
  const int half = a.D / 2;
  const int64_t total = (int64_t)a.B * a.H * a.S * half;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int j = (int)(idx % half);
    const int s = (int)((idx / half) % a.S);
    const int h = (int)((idx / ((int64_t)half * a.S)) % a.H);
    const int b = (int)(idx / ((int64_t)half * a.S * a.H));
    const int d0 = a.interleaved ? 2 * j : j;
    const int d1 = a.interleaved ? 2 * j + 1 : j + half;
    const float pos = (float)((a.pos0 ? a.pos0[b] : a.prev_seq) + s);
    const raw *xp = reinterpret_cast<const raw *>(a.x) + b * a.xs[0] + h * a.xs[1] + (int64_t)s * a.xs[2];
    raw *op = reinterpret_cast<raw *>(a.out) + b * a.os[0] + h * a.os[1] + (int64_t)s * a.os[2];
    float o0, o1;
    rope_pair<E>(E::ld(xp[d0]), E::ld(xp[d1]), pos, j, a.D, a.log2_base, &o0, &o1);
    op[d0] = E::st(o0);
    op[d1] = E::st(o1);
  }
}

template <typename E>
__global__ __launch_bounds__(256) void kv_append_kernel(KvAppendArgs a) {
  using raw = typename E::raw;
  const int64_t total = (int64_t)a.B * a.Hkv * a.T * a.D;
  const int half = a.D / 2;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int d = (int)(idx % a.D);
    const int t = (int)((idx / a.D) % a.T);
    const int h = (int)((idx / ((int64_t)a.D * a.T)) % a.Hkv);
    const int b = (int)(idx / ((int64_t)a.D * a.T * a.Hkv));
    const int row = (a.pos ? a.pos[b] : a.pos_all) + t;
    if (row < 0 || row >= a.Lmax) continue;  // a full cache drops the row instead of writing out of bounds
    const raw *kn = reinterpret_cast<const raw *>(a.k_new) + ((((int64_t)b * a.Hkv + h) * a.T + t) * a.D);
    const raw *vn = reinterpret_cast<const raw *>(a.v_new) + ((((int64_t)b * a.Hkv + h) * a.T + t) * a.D);
    raw *kc = reinterpret_cast<raw *>(a.k_cache) + b * a.ks[0] + h * a.ks[1] + (int64_t)row * a.ks[2];
    raw *vc = reinterpret_cast<raw *>(a.v_cache) + b * a.vs[0] + h * a.vs[1] + (int64_t)row * a.vs[2];
    vc[d] = vn[d];
    if (!a.rope_k) {
      kc[d] = kn[d];
    } else {
      const bool first = a.interleaved ? (d % 2 == 0) : (d < half);
      const int j = a.interleaved ? d / 2 : (d < half ? d : d - half);
      const int dp = a.interleaved ? (first ? d + 1 : d - 1) : (first ? d + half : d - half);
      const float x0 = E::ld(first ? kn[d] : kn[dp]);
      const float x1 = E::ld(first ? kn[dp] : kn[d]);
      float o0, o1;
      rope_pair<E>(x0, x1, (float)row, j, a.D, a.log2_base, &o0, &o1);
      kc[d] = E::st(first ? o0 : o1);
    }
  }
}

int grid_for(int64_t total) {
  int64_t blocks = (total + 255) / 256;
  return (int)(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

}  // namespace

int launch_rope(const RopeArgs &a, int dtype, hipStream_t stream) {
  const int64_t total = (int64_t)a.B * a.H * a.S * (a.D / 2);
  dim3 grid(grid_for(total)), block(256);
  switch (dtype) {
    case LMH_F32: hipLaunchKernelGGL(rope_kernel<F32>, grid, block, 0, stream, a); break;
    case LMH_F16: hipLaunchKernelGGL(rope_kernel<F16>, grid, block, 0, stream, a); break;
    case LMH_BF16: hipLaunchKernelGGL(rope_kernel<BF16>, grid, block, 0, stream, a); break;
    default: return fail(LMH_E_UNSUPPORTED, "rope: unknown dtype %d", dtype);
  }
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

int launch_kv_append(const KvAppendArgs &a, int dtype, hipStream_t stream) {
  const int64_t total = (int64_t)a.B * a.Hkv * a.T * a.D;
  dim3 grid(grid_for(total)), block(256);
  switch (dtype) {
    case LMH_F32: hipLaunchKernelGGL(kv_append_kernel<F32>, grid, block, 0, stream, a); break;
    case LMH_F16: hipLaunchKernelGGL(kv_append_kernel<F16>, grid, block, 0, stream, a); break;
    case LMH_BF16: hipLaunchKernelGGL(kv_append_kernel<BF16>, grid, block, 0, stream, a); break;
    default: return fail(LMH_E_UNSUPPORTED, "kv append: unknown dtype %d", dtype);
  }
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

}  // namespace lmh
