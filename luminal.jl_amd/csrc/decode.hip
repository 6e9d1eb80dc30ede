// Single-token decode attention over a KV cache, flash-decoding style.
//
// Semantics: the cached attention of reference src/Whisper.jl:584-620 (attend over rows
// 0 .. step_pos of a (B, H, max_seq, D) cache, plain softmax) with the GQA head sharing of
// reference src/NN.jl:305-317, per-sequence lengths and no cache rewrite.
//
// The op is HBM-bound: every K and V element has to cross the memory bus once and is used for
// 2*G flops. The design follows from that:
//   * one workgroup per (sequence, KV head, KV split): the G query heads that share a KV head are
//     processed together from registers, so K/V are read once per KV head, not once per query
//     head;
//   * a key row is covered by LPK adjacent lanes, each issuing one 128-bit load, so a wave's load
//     instruction touches 64/LPK complete, contiguous rows;
//   * U independent K loads and U V loads are in flight per lane before the first use;
//   * ragged lengths: grid.x spans ceil(Lmax/chunk) splits, a workgroup whose split starts past
//     kv_len[b] exits at once, and the merge kernel reads only the splits that exist;
//   * split partials (running max, sum, un-normalised output) go to a caller-owned workspace and
//     a second small kernel merges them with the log-sum-exp identity.
#include "common.hpp"
#include "dtypes.hpp"
#include "rope.hpp"

namespace lmh {
namespace {

constexpr int kWaves = 4;
constexpr int kUnroll = 4;  // key steps per wave per iteration
constexpr float kLog2e = 1.4426950408889634f;

// v_mov_b32_dpp with a compile-time lane pattern; the compiler folds it into the consuming VALU op.
template <int CTRL>
__device__ inline float dpp(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <- lane 7-i of its 8-lane half row
constexpr int kDppMirror = 0x140;     // lane i <- lane 15-i of its 16-lane row

// All-reduce (sum) over the LPK adjacent lanes that share a key. Up to 16 lanes this is pure DPP
// (no LDS round trip): after the two quad steps every lane of a quad holds the quad sum, so the
// mirror patterns, which pair quad 0 with 1 (and 2 with 3), then half row 0 with 1, finish it.
template <int LPK>
__device__ inline float sum_within_key(float x) {
  if (LPK >= 2) x += dpp<kDppXor1>(x);
  if (LPK >= 4) x += dpp<kDppXor2>(x);
  if (LPK >= 8) x += dpp<kDppHalfMirror>(x);
  if (LPK >= 16) x += dpp<kDppMirror>(x);
  if (LPK >= 32) x += __shfl_xor(x, 16);
  if (LPK >= 64) x += __shfl_xor(x, 32);
  return x;
}
// Reductions over the key slots of a wave (lane bits at and above LPK); used once, after the loop.
template <int LPK>
__device__ inline float sum_across_slots(float x) {
#pragma unroll
  for (int off = LPK; off < 64; off <<= 1) x += __shfl_xor(x, off);
  return x;
}
template <int LPK>
__device__ inline float max_across_slots(float x) {
#pragma unroll
  for (int off = LPK; off < 64; off <<= 1) x = fmaxf(x, __shfl_xor(x, off));
  return x;
}

// q in the form the dot product wants: fp32 for fp32 tensors, the original packed 16-bit pairs for
// fp16 / bf16 (v_dot2_f32_f16 / v_dot2_f32_bf16: two exact products + fp32 accumulate per op).
template <typename E>
struct QFrag;
template <>
struct QFrag<F32> {
  float q[4];
  __device__ void load(const float *p, bool ok) {
#pragma unroll
    for (int e = 0; e < 4; e++) q[e] = ok ? p[e] : 0.f;
  }
  __device__ float dot(const Vec128<F32> &k) const { return q[0] * k.r.x + q[1] * k.r.y + q[2] * k.r.z + q[3] * k.r.w; }
};
template <>
struct QFrag<F16> {
  uint32_t q[4];
  __device__ void load(const _Float16 *p, bool ok) {
    const uint16_t *u = reinterpret_cast<const uint16_t *>(p);
#pragma unroll
    for (int e = 0; e < 4; e++) q[e] = ok ? ((uint32_t)u[2 * e] | ((uint32_t)u[2 * e + 1] << 16)) : 0u;
  }
  __device__ float dot(const Vec128<F16> &k) const {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const uint32_t w[4] = {k.r.x, k.r.y, k.r.z, k.r.w};
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++)
      acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, q[e]), __builtin_bit_cast(h2, w[e]), acc, false);
    return acc;
  }
};
template <>
struct QFrag<BF16> {
  uint32_t q[4];
  __device__ void load(const uint16_t *u, bool ok) {
#pragma unroll
    for (int e = 0; e < 4; e++) q[e] = ok ? ((uint32_t)u[2 * e] | ((uint32_t)u[2 * e + 1] << 16)) : 0u;
  }
  __device__ float dot(const Vec128<BF16> &k) const {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    const uint32_t w[4] = {k.r.x, k.r.y, k.r.z, k.r.w};
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 4; e++)
      acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, q[e]), __builtin_bit_cast(b2, w[e]), acc, false);
    return acc;
  }
};

// E: element type; LPK: lanes per key row (power of two, LPK * E::kVec >= D); G: query heads
// handled per workgroup (the GQA group, or a slice of it).
//
// Every key slot (a group of LPK lanes) runs its own online softmax over the keys it sees: the
// running max, sum and output slice are slot-local, so the loop has no traffic between slots and,
// for LPK <= 16, none through LDS at all. Slots, then waves, are merged once after the loop.
template <typename E, int LPK, int G>
__global__ __launch_bounds__(kWaves * 64) void decode_split_kernel(DecodeArgs a, int g_chunks) {
  request_args(a);
  request_arg(g_chunks);
  using raw = typename E::raw;
  constexpr int VEC = E::kVec;
  constexpr int KPW = 64 / LPK;                          // keys per wave per load step
  constexpr int KEYS_PER_ITER = kWaves * kUnroll * KPW;  // keys per workgroup iteration

  const int split = blockIdx.x;
  const int kvh = blockIdx.y / g_chunks;
  const int g0 = (blockIdx.y % g_chunks) * G;  // first group member handled here
  const int b = blockIdx.z;
  const int group = a.Hq / a.Hkv;

  int L = a.kv_len ? a.kv_len[b] : a.Lmax;
  L = min(max(L, 0), a.Lmax);
  const int start = split * a.chunk;
  const int tid = threadIdx.x;
  if (start >= L) {  // ragged tail: this split does not exist for sequence b
    // ... and with a single split nobody else writes the rows of a sequence without keys: zeros, like every
    // other kernel of the library
    if (a.num_splits == 1) {
      for (int idx = tid; idx < G * a.D; idx += kWaves * 64) {
        const int gi = g0 + idx / a.D;
        if (gi >= group) continue;
        const int64_t off = b * a.os[0] + q_head_of(kvh, gi, a.Hq, a.Hkv, a.head_map) * a.os[1] + idx % a.D;
        if (a.out_f32) reinterpret_cast<float *>(a.out)[off] = 0.f;
        else reinterpret_cast<raw *>(a.out)[off] = E::st(0.f);
      }
    }
    return;
  }
  const int end = min(L, start + a.chunk);

  const int lane = tid & 63, wave = tid >> 6;
  const int slot = lane / LPK;
  const int c = lane % LPK;
  const int d0 = c * VEC;
  const bool lane_active = d0 < a.D;  // D is a multiple of VEC (checked on the host)

  QFrag<E> qf[G];
#pragma unroll
  for (int g = 0; g < G; g++) {
    const int gi = g0 + g;
    const bool head_ok = gi < group;
    const int hq = q_head_of(kvh, head_ok ? gi : 0, a.Hq, a.Hkv, a.head_map);
    const raw *qp = reinterpret_cast<const raw *>(a.q) + b * a.qs[0] + hq * a.qs[1];
    qf[g].load(qp + (lane_active ? d0 : 0), lane_active && head_ok);
  }
  const float qmul = a.scale * kLog2e;  // scores in log2 units: softmax runs on exp2

  const raw *kbase = reinterpret_cast<const raw *>(a.k) + b * a.ks[0] + kvh * a.ks[1] + d0;
  const raw *vbase = reinterpret_cast<const raw *>(a.v) + b * a.vs[0] + kvh * a.vs[1] + d0;

  float m[G], l[G], acc[G][VEC];
#pragma unroll
  for (int g = 0; g < G; g++) {
    m[g] = -INFINITY;
    l[g] = 0.f;
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[g][e] = 0.f;
  }

  for (int it0 = start; it0 < end; it0 += KEYS_PER_ITER) {
    Vec128<E> kr[kUnroll], vr[kUnroll];
    bool valid[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int key = it0 + (wave * kUnroll + u) * KPW + slot;
      valid[u] = key < end;
      if (valid[u] && lane_active) {
        kr[u].load_stream(kbase + (int64_t)key * a.ks[2]);
      } else {
        kr[u].zero();
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      const int key = it0 + (wave * kUnroll + u) * KPW + slot;
      if (valid[u] && lane_active) {
        vr[u].load_stream(vbase + (int64_t)key * a.vs[2]);
      } else {
        vr[u].zero();
      }
    }

    float s[kUnroll][G];
    float blk_max[G];
#pragma unroll
    for (int g = 0; g < G; g++) blk_max[g] = -INFINITY;
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
#pragma unroll
      for (int g = 0; g < G; g++) {
        const float dot = sum_within_key<LPK>(qf[g].dot(kr[u])) * qmul;
        s[u][g] = valid[u] ? dot : -INFINITY;
        blk_max[g] = fmaxf(blk_max[g], s[u][g]);
      }
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
      const float m_new = fmaxf(m[g], blk_max[g]);
      // m_new is -inf only while this slot has seen no valid key; then everything stays 0.
      const float alpha = (m[g] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m[g] - m_new);
      m[g] = m_new;
      l[g] *= alpha;
#pragma unroll
      for (int e = 0; e < VEC; e++) acc[g][e] *= alpha;
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
      float vf[VEC];
      vr[u].unpack(vf);
#pragma unroll
      for (int g = 0; g < G; g++) {
        const float p = valid[u] ? __builtin_amdgcn_exp2f(s[u][g] - m[g]) : 0.f;
        l[g] += p;
#pragma unroll
        for (int e = 0; e < VEC; e++) acc[g][e] += p * vf[e];
      }
    }
  }

  // Merge the key slots of each wave (bring them to the wave's max first), then the waves.
  __shared__ float sm_m[kWaves][G];
  __shared__ float sm_l[kWaves][G];
  __shared__ float sm_acc[kWaves][G][LPK * VEC];
#pragma unroll
  for (int g = 0; g < G; g++) {
    const float m_wave = max_across_slots<LPK>(m[g]);
    const float f = (m[g] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m[g] - m_wave);
    l[g] = sum_across_slots<LPK>(l[g] * f);
#pragma unroll
    for (int e = 0; e < VEC; e++) acc[g][e] = sum_across_slots<LPK>(acc[g][e] * f);
    if (slot == 0) {
#pragma unroll
      for (int e = 0; e < VEC; e++) sm_acc[wave][g][d0 + e] = acc[g][e];
      if (c == 0) {
        sm_m[wave][g] = m_wave;
        sm_l[wave][g] = l[g];
      }
    }
  }
  __syncthreads();

  for (int idx = tid; idx < G * a.D; idx += kWaves * 64) {
    const int g = idx / a.D, d = idx % a.D;
    const int gi = g0 + g;
    if (gi >= group) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; w++) M = fmaxf(M, sm_m[w][g]);
    float lsum = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
      const float f = (sm_m[w][g] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(sm_m[w][g] - M);
      lsum += sm_l[w][g] * f;
      o += sm_acc[w][g][d] * f;
    }
    const int hq = q_head_of(kvh, gi, a.Hq, a.Hkv, a.head_map);
    if (a.num_splits == 1) {
      const int64_t off = b * a.os[0] + hq * a.os[1] + d;
      if (a.out_f32) reinterpret_cast<float *>(a.out)[off] = o / lsum;
      else reinterpret_cast<raw *>(a.out)[off] = E::st(o / lsum);
    } else {
      const int64_t row = ((int64_t)b * a.Hq + hq) * a.num_splits + split;
      a.ws_o[row * a.D + d] = o;
      if (d == 0) {
        a.ws_ml[row * 2 + 0] = M;
        a.ws_ml[row * 2 + 1] = lsum;
      }
    }
  }
}

// out[b,hq,:] = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M) over the splits that exist.
// One workgroup per (b, hq). The slot statistics are fetched in parallel (one slot per thread), reduced
// across the workgroup, and the per-slot weights go through LDS, so the loop over slots that follows
// issues independent loads of the partial outputs instead of a chain of dependent ones.
constexpr int kMergeThreads = 128;
constexpr int kMergeMaxSlots = 1024;  // weights kept in LDS; more slots than this take the strided path below
constexpr int kMergePrefetch = 16;     // partial rows fetched before the slot statistics are known
// STEP (lmh_decode_step): the row this step appends, kv_len[b], never went through the split kernel. It joins here as
// one more partial — score q . k_new (both rotated at position kv_len[b] when a.q_rope, and rounded to the element
// type as the stored rows are), sum 1, output v_new — and the workgroup of the first query head of every KV head
// writes the row into the caches (the reference rebuilds them with _kv_scatter, src/Whisper.jl:552-570).
template <typename E, bool STEP>
__global__ __launch_bounds__(kMergeThreads) void decode_merge_kernel(DecodeArgs a) {
  request_args(a);
  using raw = typename E::raw;
  __shared__ float w_s[kMergeMaxSlots];
  __shared__ float red_m[kMergeThreads / 64], red_l[kMergeThreads / 64], red_s[kMergeThreads / 64];
  const int hq = blockIdx.x, b = blockIdx.y;
  const int tid = threadIdx.x;
  const int64_t off = b * a.os[0] + hq * a.os[1];
  const int64_t row0 = ((int64_t)b * a.Hq + hq) * a.num_splits;
  const float2 *ml = reinterpret_cast<const float2 *>(a.ws_ml) + row0;
  const float *po = a.ws_o + row0 * a.D;

  // The kernel is a chain of round trips to memory the split kernel has just written (kv_len, the slot statistics,
  // the partial rows), each about as long as the arithmetic of the whole kernel. The rows of the first slots do
  // not depend on the others: they are requested first, and travel while the statistics are reduced. Rows of
  // slots that turn out not to exist or to be empty are unset memory and are discarded unread below.
  float pre[kMergePrefetch];
  const int n_pre = min(a.num_splits, kMergePrefetch);
#pragma unroll
  for (int u = 0; u < kMergePrefetch; u++) pre[u] = (u < n_pre && tid < a.D) ? po[(int64_t)u * a.D + tid] : 0.f;

  int L = a.kv_len ? a.kv_len[b] : a.Lmax;
  L = min(max(L, 0), a.Lmax);
  const int n = (L + a.chunk - 1) / a.chunk;

  // (this thread's first slot statistics are requested before the new row's arithmetic, not after its barrier)
  const float2 ml_first = tid < n ? ml[tid] : make_float2(-INFINITY, 0.f);
  // the new row: its score in log2 units, and (first query head of the KV head only) its place in the caches
  float m_new = -INFINITY;
  const raw *v_new_row = nullptr;
  if (STEP && L < a.Lmax) {
    const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
    const bool writer = q_head_of(kvh, 0, a.Hq, a.Hkv, a.head_map) == hq;
    const raw *q_row = reinterpret_cast<const raw *>(a.q) + b * a.qs[0] + hq * a.qs[1];
    const raw *k_new_row = reinterpret_cast<const raw *>(a.k_new) + ((int64_t)b * a.Hkv + kvh) * a.D;
    v_new_row = reinterpret_cast<const raw *>(a.v_new) + ((int64_t)b * a.Hkv + kvh) * a.D;
    raw *k_dst = const_cast<raw *>(reinterpret_cast<const raw *>(a.k)) + b * a.ks[0] + kvh * a.ks[1] + (int64_t)L * a.ks[2];
    raw *v_dst = const_cast<raw *>(reinterpret_cast<const raw *>(a.v)) + b * a.vs[0] + kvh * a.vs[1] + (int64_t)L * a.vs[2];
    auto ld = [](raw x) { return E::ld(x); };
    float dot = 0.f;
    for (int d = tid; d < a.D; d += kMergeThreads) {
      raw qr = q_row[d], kr = k_new_row[d];
      if (a.q_rope) {
        qr = E::st(rope_element(q_row, d, a.D, (float)L, a.rope_log2_base, a.rope_interleaved != 0, ld));
        kr = E::st(rope_element(k_new_row, d, a.D, (float)L, a.rope_log2_base, a.rope_interleaved != 0, ld));
      }
      dot += E::ld(qr) * E::ld(kr);
      if (writer) {
        k_dst[d] = kr;
        v_dst[d] = v_new_row[d];
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) dot += __shfl_xor(dot, o);
    if ((tid & 63) == 0) red_s[tid >> 6] = dot;
    __syncthreads();
    dot = 0.f;
#pragma unroll
    for (int w = 0; w < kMergeThreads / 64; w++) dot += red_s[w];
    m_new = dot * a.scale * kLog2e;
  }

  // running max over the slots
  float M = fmaxf(m_new, ml_first.x);
  for (int s = tid + kMergeThreads; s < n; s += kMergeThreads) M = fmaxf(M, ml[s].x);
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) M = fmaxf(M, __shfl_xor(M, o));
  if ((tid & 63) == 0) red_m[tid >> 6] = M;
  __syncthreads();
  M = red_m[0];
#pragma unroll
  for (int w = 1; w < kMergeThreads / 64; w++) M = fmaxf(M, red_m[w]);

  // weights 2^(m_s - M) (0 for a slot marked (-inf, 0): it was folded into an earlier slot of the same
  // run and its output row is unset) and the normaliser
  float lsum = 0.f;
  for (int s = tid; s < n; s += kMergeThreads) {
    const float2 v = s == tid ? ml_first : ml[s];
    const float w = v.x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(v.x - M);
    if (s < kMergeMaxSlots) w_s[s] = w;
    lsum += v.y * w;
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) lsum += __shfl_xor(lsum, o);
  if ((tid & 63) == 0) red_l[tid >> 6] = lsum;
  __syncthreads();
  lsum = 0.f;
#pragma unroll
  for (int w = 0; w < kMergeThreads / 64; w++) lsum += red_l[w];
  const float w_new = (STEP && v_new_row) ? __builtin_amdgcn_exp2f(m_new - M) : 0.f;  // the new row's sum is 1
  lsum += w_new;
  const float inv = lsum > 0.f ? 1.f / lsum : 0.f;

  for (int d = tid; d < a.D; d += kMergeThreads) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    int s = 0;
    const int n_lds = min(n, kMergeMaxSlots);
    if (d == tid) {  // the prefetched rows (same summation order as below: slot s adds to acc[s % 4])
      const int n_p = min(n_lds, n_pre) & ~3;
#pragma unroll
      for (int u = 0; u < kMergePrefetch; u++) {
        if (u < n_p) {
          const float w = w_s[u];
          // the row of a zero-weight slot is unset memory: select, do not multiply
          acc[u & 3] += w != 0.f ? pre[u] * w : 0.f;
        }
      }
      s = n_p;
    }
    for (; s + 4 <= n_lds; s += 4) {
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const float w = w_s[s + u];
        const float x = po[(int64_t)(s + u) * a.D + d];
        acc[u] += w != 0.f ? x * w : 0.f;
      }
    }
    for (; s < n; s++) {
      const float w = s < kMergeMaxSlots ? w_s[s] : (ml[s].x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml[s].x - M));
      const float x = po[(int64_t)s * a.D + d];
      acc[0] += w != 0.f ? x * w : 0.f;
    }
    float o = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    if (STEP && v_new_row) o += w_new * E::ld(v_new_row[d]);
    if (a.out_f32) reinterpret_cast<float *>(a.out)[off + d] = o * inv;
    else reinterpret_cast<raw *>(a.out)[off + d] = E::st(o * inv);
  }
}

template <typename E>
int launch_merge(const DecodeArgs &a, hipStream_t stream) {
  if (a.step) {  // (always with partials: lmh_decode_step asks for two splits or more)
    hipLaunchKernelGGL((decode_merge_kernel<E, true>), dim3(a.Hq, a.B), dim3(kMergeThreads), 0, stream, a);
    LMH_HIP_TRY(hipGetLastError());
  } else if (a.num_splits > 1) {
    hipLaunchKernelGGL((decode_merge_kernel<E, false>), dim3(a.Hq, a.B), dim3(kMergeThreads), 0, stream, a);
    LMH_HIP_TRY(hipGetLastError());
  }
  return LMH_OK;
}

template <typename E, int LPK>
int launch_for_lpk(const DecodeArgs &a, hipStream_t stream) {
  const int group = a.Hq / a.Hkv;
  dim3 block(kWaves * 64);
#define LMH_DECODE_LAUNCH(GG)                                                               \
  do {                                                                                      \
    const int g_chunks = (group + (GG)-1) / (GG);                                           \
    dim3 grid(a.num_splits, a.Hkv * g_chunks, a.B);                                         \
    hipLaunchKernelGGL((decode_split_kernel<E, LPK, GG>), grid, block, 0, stream, a, g_chunks); \
  } while (0)
  if (group == 1) LMH_DECODE_LAUNCH(1);
  else if (group == 2) LMH_DECODE_LAUNCH(2);
  else if (group <= 4) LMH_DECODE_LAUNCH(4);
  else LMH_DECODE_LAUNCH(8);
#undef LMH_DECODE_LAUNCH
  LMH_HIP_TRY(hipGetLastError());
  return launch_merge<E>(a, stream);
}

template <typename E>
int launch_for_dtype(const DecodeArgs &a, hipStream_t stream) {
  const int chunks = (a.D + E::kVec - 1) / E::kVec;
  if (chunks <= 4) return launch_for_lpk<E, 4>(a, stream);
  if (chunks <= 8) return launch_for_lpk<E, 8>(a, stream);
  if (chunks <= 16) return launch_for_lpk<E, 16>(a, stream);
  if (chunks <= 32) return launch_for_lpk<E, 32>(a, stream);
  if (chunks <= 64) return launch_for_lpk<E, 64>(a, stream);
  return fail(LMH_E_UNSUPPORTED, "decode attention: head dim %d too large", a.D);
}

}  // namespace

int decode_chunk_for(int Lmax, int num_splits) {
  if (num_splits < 1) num_splits = 1;
  int chunk = (Lmax + num_splits - 1) / num_splits;
  chunk = (chunk + 63) / 64 * 64;
  return chunk < 64 ? 64 : chunk;
}

int launch_decode(const DecodeArgs &a, int dtype, hipStream_t stream) {
  // (the matrix-core kernel deals its (b, kv head slice, chunk) units in 32-bit arithmetic)
  const int64_t mfma_units = (int64_t)a.B * a.Hkv * ((a.Hq / a.Hkv + 15) / 16) * a.num_splits;
  if (a.mfma_ok && decode_mfma_supported(dtype, a.D, a.B) && mfma_units < (int64_t(1) << 31)) {
    const int rc = launch_decode_mfma_split(a, dtype, stream);
    if (rc != LMH_OK) return rc;
    return dtype == LMH_F16 ? launch_merge<F16>(a, stream) : launch_merge<BF16>(a, stream);
  }
  if (a.step) return fail(LMH_E_UNSUPPORTED, "decode step: only the matrix-core decode kernel rotates q as it loads it");
  switch (dtype) {
    case LMH_F32: return launch_for_dtype<F32>(a, stream);
    case LMH_F16: return launch_for_dtype<F16>(a, stream);
    case LMH_BF16: return launch_for_dtype<BF16>(a, stream);
  }
  return fail(LMH_E_UNSUPPORTED, "decode attention: unknown dtype %d", dtype);
}

}  // namespace lmh
