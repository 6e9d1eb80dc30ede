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
// Both are a few bytes of traffic per element and HBM-bound. The kernels that run for the usual head
// dims move 16-byte chunks: a thread owns the chunk of pairs (j .. j+V-1) — chunk c of the first half
// of the row and chunk c of the second half, or one chunk of interleaved pairs — and, for the
// standalone rotary embedding, evaluates its sin / cos once and walks the heads with them (the angle
// does not depend on the head). Rows whose head dim or alignment does not allow 16-byte chunks take
// the one-element-per-thread kernels.
#include "common.hpp"
#include "dtypes.hpp"
#include "rope.hpp"

namespace lmh {
namespace {

template <typename E>
__global__ __launch_bounds__(256) void rope_kernel(RopeArgs a) {
  request_args(a);
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
    rope_pair(E::ld(xp[d0]), E::ld(xp[d1]), pos, j, a.D, a.log2_base, &o0, &o1);
    op[d0] = E::st(o0);
    op[d1] = E::st(o1);
  }
}

template <typename E>
__global__ __launch_bounds__(256) void kv_append_kernel(KvAppendArgs a) {
  request_args(a);
  using raw = typename E::raw;
  const int64_t total = (int64_t)a.B * a.Hkv * a.T * a.D;
  const int half = a.D / 2;
  const int64_t total_q = a.q ? (int64_t)a.B * a.Hq * a.T * half : 0;  // pairs of this step's queries to rotate in place
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total + total_q; idx += (int64_t)gridDim.x * blockDim.x) {
    if (idx >= total) {
      const int64_t r = idx - total;
      const int j = (int)(r % half);
      const int t = (int)((r / half) % a.T);
      const int64_t bh = r / ((int64_t)half * a.T);  // b * Hq + h
      const int b = (int)(bh / a.Hq);
      const int d0 = a.interleaved ? 2 * j : j;
      const int d1 = a.interleaved ? 2 * j + 1 : j + half;
      raw *qp = reinterpret_cast<raw *>(a.q) + (bh * a.T + t) * a.D;
      float o0, o1;
      rope_pair(E::ld(qp[d0]), E::ld(qp[d1]), (float)((a.pos ? a.pos[b] : a.pos_all) + t), j, a.D, a.log2_base, &o0, &o1);
      qp[d0] = E::st(o0);
      qp[d1] = E::st(o1);
      continue;
    }
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
      rope_pair(x0, x1, (float)row, j, a.D, a.log2_base, &o0, &o1);
      kc[d] = E::st(first ? o0 : o1);
    }
  }
}

// 16 bytes of a row, as raw elements
template <typename E>
union Chunk {
  uint4 u;
  typename E::raw e[E::kVec];
};

// x0[i], x1[i] -> rotated in place by (sn[i], cs[i]); same expressions as rope_pair
template <typename E>
__device__ inline void rotate_chunks(Chunk<E> &c0, Chunk<E> &c1, const float *sn, const float *cs) {
#pragma unroll
  for (int i = 0; i < E::kVec; i++) {
    float o0, o1;
    rope_rotate(E::ld(c0.e[i]), E::ld(c1.e[i]), sn[i], cs[i], &o0, &o1);
    c0.e[i] = E::st(o0);
    c1.e[i] = E::st(o1);
  }
}
template <typename E>
__device__ inline void rotate_interleaved(Chunk<E> &c, const float *sn, const float *cs) {
#pragma unroll
  for (int i = 0; i < E::kVec / 2; i++) {
    float o0, o1;
    rope_rotate(E::ld(c.e[2 * i]), E::ld(c.e[2 * i + 1]), sn[i], cs[i], &o0, &o1);
    c.e[2 * i] = E::st(o0);
    c.e[2 * i + 1] = E::st(o1);
  }
}
template <typename E>
__device__ inline void sincos_pairs(float pos, int j0, int n, int D, float log2_base, float *sn, float *cs) {
#pragma unroll
  for (int i = 0; i < E::kVec; i++) {
    if (i >= n) break;
    sincos_angle(pos * rope_inv_freq(j0 + i, D, log2_base), &sn[i], &cs[i]);
  }
}

// Rotary embedding, 16-byte chunks. grid.x covers (b, s, chunk), grid.y blocks of heads.
// IL = false: thread owns pairs j = c V .. c V + V - 1, i.e. chunk c of each half of the row.
// IL = true : thread owns pairs j = c V/2 .. , i.e. chunk c of the row.
template <typename E, bool IL>
__global__ __launch_bounds__(256) void rope_vec_kernel(RopeArgs a, int heads_per_block) {
  request_args(a);
  request_arg(heads_per_block);
  using raw = typename E::raw;
  constexpr int V = E::kVec;
  const int half = a.D / 2;
  const int cpr = IL ? a.D / V : half / V;  // chunks (threads) per row
  const int64_t total = (int64_t)a.B * a.S * cpr;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % cpr);
  const int s = (int)((idx / cpr) % a.S);
  const int b = (int)(idx / ((int64_t)cpr * a.S));
  const float pos = (float)((a.pos0 ? a.pos0[b] : a.prev_seq) + s);
  float sn[V], cs[V];
  sincos_pairs<E>(pos, IL ? c * (V / 2) : c * V, IL ? V / 2 : V, a.D, a.log2_base, sn, cs);
  // Heads in batches of kHeadBatch: all of a batch's loads are issued before the first is used, so a thread has up
  // to 2 * kHeadBatch 16-byte loads in flight (the ~1000 workgroups of a launch alone do not keep HBM busy).
  constexpr int kHeadBatch = 4;
  const int h0 = blockIdx.y * heads_per_block, h1 = min(a.H, h0 + heads_per_block);
  const raw *xrow = reinterpret_cast<const raw *>(a.x) + b * a.xs[0] + (int64_t)s * a.xs[2];
  raw *orow = reinterpret_cast<raw *>(a.out) + b * a.os[0] + (int64_t)s * a.os[2];
  for (int hb = h0; hb < h1; hb += kHeadBatch) {
    Chunk<E> c0[kHeadBatch], c1[kHeadBatch];
#pragma unroll
    for (int i = 0; i < kHeadBatch; i++) {
      if (hb + i >= h1) break;
      const raw *xp = xrow + (hb + i) * a.xs[1];
      c0[i].u = *reinterpret_cast<const uint4 *>(xp + c * V);
      if (!IL) c1[i].u = *reinterpret_cast<const uint4 *>(xp + half + c * V);
    }
#pragma unroll
    for (int i = 0; i < kHeadBatch; i++) {
      if (hb + i >= h1) break;
      raw *op = orow + (hb + i) * a.os[1];
      if (IL) {
        rotate_interleaved<E>(c0[i], sn, cs);
        *reinterpret_cast<uint4 *>(op + c * V) = c0[i].u;
      } else {
        rotate_chunks<E>(c0[i], c1[i], sn, cs);
        *reinterpret_cast<uint4 *>(op + c * V) = c0[i].u;
        *reinterpret_cast<uint4 *>(op + half + c * V) = c1[i].u;
      }
    }
  }
}

// Cache append, 16-byte chunks: a thread owns chunk c of each half of the new rows at (b, t) and walks the KV
// heads of its block (D is a multiple of 2 V), rotating K on the way when asked to. The angle depends on the row
// position and the pair, not on the head, so the sin / cos are evaluated once per thread (they were 17 % of a
// whole-prompt append when every (b, head, t) thread evaluated its own). grid.x covers (b, t, chunk), grid.y
// blocks of heads.
template <typename E>
__global__ __launch_bounds__(256) void kv_append_vec_kernel(KvAppendArgs a, int heads_per_block) {
  request_args(a);
  request_arg(heads_per_block);
  using raw = typename E::raw;
  constexpr int V = E::kVec;
  const int half = a.D / 2;
  const int cpr = half / V;
  const int64_t total = (int64_t)a.B * a.T * cpr;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % cpr);
  const int t = (int)((idx / cpr) % a.T);
  const int b = (int)(idx / ((int64_t)cpr * a.T));
  const int row = (a.pos ? a.pos[b] : a.pos_all) + t;
  if (row < 0 || row >= a.Lmax) return;  // a full cache drops the row instead of writing out of bounds
  const int d0 = c * V, d1 = half + c * V;
  float sn0[V], cs0[V], sn1[V / 2], cs1[V / 2];
  if (a.rope_k) {
    if (a.interleaved) {
      sincos_pairs<E>((float)row, d0 / 2, V / 2, a.D, a.log2_base, sn0, cs0);
      sincos_pairs<E>((float)row, d1 / 2, V / 2, a.D, a.log2_base, sn1, cs1);
    } else {
      sincos_pairs<E>((float)row, d0, V, a.D, a.log2_base, sn0, cs0);
    }
  }
  const int h0 = blockIdx.y * heads_per_block, h1 = min(a.Hkv, h0 + heads_per_block);
  for (int h = h0; h < h1; h++) {
    const int64_t src = (((int64_t)b * a.Hkv + h) * a.T + t) * a.D;
    const raw *kn = reinterpret_cast<const raw *>(a.k_new) + src;
    const raw *vn = reinterpret_cast<const raw *>(a.v_new) + src;
    raw *kc = reinterpret_cast<raw *>(a.k_cache) + b * a.ks[0] + h * a.ks[1] + (int64_t)row * a.ks[2];
    raw *vc = reinterpret_cast<raw *>(a.v_cache) + b * a.vs[0] + h * a.vs[1] + (int64_t)row * a.vs[2];
    Chunk<E> k0, k1;
    k0.u = load_stream_128(kn + d0);
    k1.u = load_stream_128(kn + d1);
    const uint4 v0 = load_stream_128(vn + d0), v1 = load_stream_128(vn + d1);
    if (a.rope_k) {
      if (a.interleaved) {
        rotate_interleaved<E>(k0, sn0, cs0);
        rotate_interleaved<E>(k1, sn1, cs1);
      } else {
        rotate_chunks<E>(k0, k1, sn0, cs0);
      }
    }
    *reinterpret_cast<uint4 *>(kc + d0) = k0.u;
    *reinterpret_cast<uint4 *>(kc + d1) = k1.u;
    *reinterpret_cast<uint4 *>(vc + d0) = v0;
    *reinterpret_cast<uint4 *>(vc + d1) = v1;
  }
}

bool chunks_ok(const void *p0, const void *p1, const int64_t *s0, const int64_t *s1, int vec) {
  if ((reinterpret_cast<uintptr_t>(p0) | reinterpret_cast<uintptr_t>(p1)) & 15u) return false;
  for (int i = 0; i < 3; i++)
    if (s0[i] % vec != 0 || s1[i] % vec != 0) return false;
  return true;
}

template <typename E>
void launch_rope_vec(const RopeArgs &a, hipStream_t stream) {
  const int cpr = a.interleaved ? a.D / E::kVec : a.D / 2 / E::kVec;
  const int64_t blocks_x = ((int64_t)a.B * a.S * cpr + 255) / 256;
  // about 1024 workgroups fill the chip; beyond that, more heads per thread amortise the sin / cos
  // (C2's Q, 25 MB: 16.9 us with one head per thread, 11.0 us at 3; large tensors lose ~5 % to the longer threads)
#ifndef LMH_ROPE_WGS
#define LMH_ROPE_WGS 1024
#endif
  int blocks_y = (int)((LMH_ROPE_WGS + blocks_x - 1) / blocks_x);
  blocks_y = blocks_y < 1 ? 1 : (blocks_y > a.H ? a.H : blocks_y);
  const int heads_per_block = (a.H + blocks_y - 1) / blocks_y;
  blocks_y = (a.H + heads_per_block - 1) / heads_per_block;
  dim3 grid((unsigned)blocks_x, (unsigned)blocks_y), block(256);
  if (a.interleaved)
    hipLaunchKernelGGL((rope_vec_kernel<E, true>), grid, block, 0, stream, a, heads_per_block);
  else
    hipLaunchKernelGGL((rope_vec_kernel<E, false>), grid, block, 0, stream, a, heads_per_block);
}

int grid_for(int64_t total) {
  int64_t blocks = (total + 255) / 256;
  return (int)(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

}  // namespace

int launch_rope(const RopeArgs &a, int dtype, hipStream_t stream) {
  const int vec = dtype == LMH_F32 ? 4 : 8;
  const int64_t vec_threads = (int64_t)a.B * a.S * (a.D / vec);
  if (a.D % (a.interleaved ? vec : 2 * vec) == 0 && chunks_ok(a.x, a.out, a.xs, a.os, vec) &&
      a.H <= 65535 && vec_threads / 256 < (int64_t(1) << 31)) {
    switch (dtype) {
      case LMH_F32: launch_rope_vec<F32>(a, stream); break;
      case LMH_F16: launch_rope_vec<F16>(a, stream); break;
      case LMH_BF16: launch_rope_vec<BF16>(a, stream); break;
      default: return fail(LMH_E_UNSUPPORTED, "rope: unknown dtype %d", dtype);
    }
    LMH_HIP_TRY(hipGetLastError());
    return LMH_OK;
  }
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
  const int vec = dtype == LMH_F32 ? 4 : 8;
  const int64_t vec_chunks = (int64_t)a.B * a.Hkv * a.T * (a.D / (2 * vec));  // 16-byte chunk pairs to move
  const int64_t blocks_x = ((int64_t)a.B * a.T * (a.D / (2 * vec)) + 255) / 256;
  if (a.D % (2 * vec) == 0 && chunks_ok(a.k_cache, a.v_cache, a.ks, a.vs, vec) &&
      ((reinterpret_cast<uintptr_t>(a.k_new) | reinterpret_cast<uintptr_t>(a.v_new)) & 15u) == 0 &&
      vec_chunks >= 64 * 256 && blocks_x < (int64_t(1) << 31) && a.Hkv <= 65535) {  // a decode step's few rows: one element per thread is quicker
    // about 2048 workgroups keep enough loads in flight; beyond that a thread walks more heads with one set of sin / cos
    int blocks_y = (int)((2048 + blocks_x - 1) / blocks_x);
    blocks_y = blocks_y < 1 ? 1 : (blocks_y > a.Hkv ? a.Hkv : blocks_y);
    const int heads_per_block = (a.Hkv + blocks_y - 1) / blocks_y;
    blocks_y = (a.Hkv + heads_per_block - 1) / heads_per_block;
    dim3 grid((unsigned)blocks_x, (unsigned)blocks_y), block(256);
    switch (dtype) {
      case LMH_F32: hipLaunchKernelGGL(kv_append_vec_kernel<F32>, grid, block, 0, stream, a, heads_per_block); break;
      case LMH_F16: hipLaunchKernelGGL(kv_append_vec_kernel<F16>, grid, block, 0, stream, a, heads_per_block); break;
      case LMH_BF16: hipLaunchKernelGGL(kv_append_vec_kernel<BF16>, grid, block, 0, stream, a, heads_per_block); break;
      default: return fail(LMH_E_UNSUPPORTED, "kv append: unknown dtype %d", dtype);
    }
    LMH_HIP_TRY(hipGetLastError());
    if (!a.q) return LMH_OK;
    // prompt-sized: the queries take the rotary kernel of their own
    RopeArgs r;
    r.out = a.q; r.x = a.q; r.pos0 = a.pos; r.prev_seq = a.pos_all;
    r.B = a.B; r.H = a.Hq; r.S = a.T; r.D = a.D;
    r.xs[0] = r.os[0] = (int64_t)a.Hq * a.T * a.D; r.xs[1] = r.os[1] = (int64_t)a.T * a.D; r.xs[2] = r.os[2] = a.D;
    r.log2_base = a.log2_base; r.interleaved = a.interleaved;
    return launch_rope(r, dtype, stream);
  }
  const int64_t total = (int64_t)a.B * a.Hkv * a.T * a.D + (a.q ? (int64_t)a.B * a.Hq * a.T * (a.D / 2) : 0);
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
