// Single-token GQA decode attention on the matrix cores (fp16 / bf16 caches).
//
// Decode is HBM-bound: the only thing that matters is keeping >= 6 TB/s of K/V reads in flight.
// On the vector ALUs the 2*G flops per cache element (plus 16-bit unpacking and the cross-lane
// dot-product reductions) keep the VALUs ~60 % busy at 5 TB/s, which caps the kernel below the
// memory roofline. The matrix cores are otherwise idle, so the G query heads of a KV head are
// padded to a 16-wide MFMA operand and both products run as v_mfma_f32_16x16x32: per 32 keys a
// wave then issues 16 MFMAs and ~100 VALU instructions instead of ~900, and the kernel is left
// waiting on memory only. (Same semantics as decode.hip: reference src/Whisper.jl:584-620 with the
// GQA head sharing of src/NN.jl:305-317.)
//
// Data flow per wave, 32 keys at a time (each wave owns a private LDS region, so the loop has no
// workgroup barrier):
//   global --128-bit coalesced loads (16 lanes per 256-byte row)--> registers (prefetched one
//   block ahead) --> LDS, row-major, padded rows
//   S^T[key, head] = K Q^T : A = K fragment (plain 128-bit LDS read), B = Q^T (registers, loaded once)
//   online softmax on the accumulator: lane (head n, g) holds keys 4g..4g+3 of each 16-key half; the
//   4 lanes of a head agree on the max through two lane exchanges
//   O^T[d, head] += V^T P^T : A = V^T fragment via the transposing LDS read ds_read_b64_tr_b16,
//   B = P^T = the softmax registers converted to 16 bit (never leaves the register file), as a
//   head + remainder pair so that P keeps ~16 significant bits
//
// Scheduling: a rectangular (split, kv head, batch) grid wastes a ragged batch twice — workgroups
// whose split lies past kv_len[b] still have to be dispatched (≈40 % of the grid for lengths spread
// over [Lmax/4, Lmax]), and every workgroup pays its own ramp-up. Instead the kernel is persistent:
// the launch has as many workgroups as fit on the chip, every workgroup builds the prefix sum of
// ceil(kv_len[b] / chunk) over the batch in LDS, and takes an equal, contiguous share of the
// existing (b, kv head, chunk) units. Inside its share it streams through maximal runs of chunks of
// one (b, kv head) with a single softmax state, so partials are written once per run, not once per
// chunk (the other chunk slots of the run get an "empty" marker the merge kernel skips).
// Split-KV partial layout and the merge kernel are shared with decode.hip.
#include "common.hpp"
#include "dtypes.hpp"
#include "rope.hpp"

namespace lmh {
namespace {

constexpr int kWaves = 4;
constexpr int kBlk = 32;  // keys per wave per step
constexpr float kLog2e = 1.4426950408889634f;

typedef short shortx8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) shortx4_t lds_shortx4_t;

struct Mfma16F16 {
  using vec8 = half8_t;
  __device__ static floatx4_t mfma(vec8 a, vec8 b, floatx4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  __device__ static _Float16 cvt(float x) { return (_Float16)x; }
  __device__ static uint16_t cvt_bits(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }
};
struct Mfma16BF16 {
  using vec8 = bf16x8_t;
  __device__ static floatx4_t mfma(vec8 a, vec8 b, floatx4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static __bf16 cvt(float x) { return (__bf16)x; }
  __device__ static uint16_t cvt_bits(float x) { return f32_to_bf16_bits(x); }
};

// Compiler-level ordering of one wave's LDS writes against its later LDS reads by other lanes.
// The hardware executes a wave's LDS instructions in order; this only pins the program order.
__device__ inline void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int kMaxBatchPersistent = 1024;  // prefix sums live in LDS

template <typename MT, int D>
__global__ __launch_bounds__(kWaves * 64) void decode_mfma_kernel(DecodeArgs a, int g_chunks) {
  request_args(a);
  request_arg(g_chunks);
  using vec8 = typename MT::vec8;
  constexpr int KS = D / 32;             // k-steps of S^T = K Q^T
  constexpr int DB = D / 16;             // 16-row blocks of O^T
  constexpr int CPR = D / 8;             // 16-byte chunks per cache row
  constexpr int NL = kBlk * CPR / 64;    // 128-bit loads per lane per 32-key tile
  constexpr int LDK = D + 8;             // LDS row strides (elements): chosen so that the 16 rows a
  constexpr int LDV = D + 16;            // fragment read touches fall on different banks
  constexpr int kTileBytes = kBlk * (LDK + LDV) * 2;
  constexpr int kMergeBytes = kWaves * 16 * (D + 2) * 4;
  constexpr int kSmemBytes = kWaves * kTileBytes > kMergeBytes ? kWaves * kTileBytes : kMergeBytes;
  __shared__ __attribute__((aligned(16))) unsigned char smem[kSmemBytes];
  __shared__ int s_pref[kMaxBatchPersistent + 1];  // s_pref[b] = chunks of sequences 0..b-1

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, g = lane >> 4;
  const int group = a.Hq / a.Hkv;
  const int kv_slots = a.Hkv * g_chunks;  // (kv head, slice of <= 16 group members) pairs

  // ---- this workgroup's share of the (b, kv slot, chunk) units ----
  // s_pref = exclusive prefix sum of the chunks per sequence. Without kv_len it is a closed form; with it, the
  // first wave scans 64 sequences at a time with lane shifts (a serial loop over B = 64 by one thread was 3 us).
  if (!a.kv_len) {
    const int per_seq = (a.Lmax + a.chunk - 1) / a.chunk;
    for (int i = tid; i <= a.B; i += kWaves * 64) s_pref[i] = i * per_seq;
  } else if (wave == 0) {
    int carry = 0;
    for (int base = 0; base < a.B; base += 64) {
      const int i = base + lane;
      int v = 0;
      if (i < a.B) v = (min(max(a.kv_len[i], 0), a.Lmax) + a.chunk - 1) / a.chunk;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(v, off);
        if (lane >= off) v += up;
      }
      if (i < a.B) s_pref[i + 1] = carry + v;
      carry += __shfl(v, 63);
    }
    if (lane == 0) s_pref[0] = 0;
  }
  __syncthreads();
  // Equal contiguous shares of the units, in 32-bit arithmetic (the launcher routes batches with 2^31 units or more to
  // the other kernel): the first total % grid workgroups take one unit more. 64-bit divisions are ~100 scalar
  // instructions each on this hardware, and five of them stood between a workgroup's start and its first load.
  const uint32_t total_units = (uint32_t)s_pref[a.B] * (uint32_t)kv_slots;
  const uint32_t share = total_units / gridDim.x, extra = total_units % gridDim.x;
  uint32_t u = blockIdx.x * share + min((uint32_t)blockIdx.x, extra);
  const uint32_t u_end = u + share + (blockIdx.x < extra ? 1u : 0u);

  // Per-lane byte offsets of the NL 16-byte loads of a 32-key block, relative to the block's first row: load r of lane l
  // fetches chunk (r * 64 + l) of the block, i.e. row (r * 64 + l) / CPR, 16-byte column (r * 64 + l) % CPR. They do not
  // depend on the block, so they are computed once; a block's own position goes into the scalar offset of the load.
  int k_voff[NL], v_voff[NL];
#pragma unroll
  for (int r = 0; r < NL; r++) {
    const int id = r * 64 + lane;
    k_voff[r] = (int)(((id / CPR) * a.ks[2] + (id % CPR) * 8) * 2);
    v_voff[r] = (int)(((id / CPR) * a.vs[2] + (id % CPR) * 8) * 2);
  }
  const int k_row_bytes = (int)(a.ks[2] * 2), v_row_bytes = (int)(a.vs[2] * 2);

  uint16_t *Ks = reinterpret_cast<uint16_t *>(smem + wave * kTileBytes);
  uint16_t *Vs = Ks + kBlk * LDK;
  const float c = a.scale * kLog2e;
  const int k_frag_off = n * LDK + 8 * g;                             // + 16*hb*LDK + 32*ks
  const int v_frag_off = (4 * g + (n >> 2)) * LDV + 4 * (n & 3);      // + 16*hb*LDV + 16*db

  while (u < u_end) {
    // segment = the maximal run of units of one (b, kv slot) inside [u, u_end)
    int lo = 0, hi = a.B;  // largest b with s_pref[b] * kv_slots <= u
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if ((uint32_t)s_pref[mid] * (uint32_t)kv_slots <= u) lo = mid; else hi = mid;
    }
    const int b = lo;
    const int n_chunks = s_pref[b + 1] - s_pref[b];
    const uint32_t rem = u - (uint32_t)s_pref[b] * (uint32_t)kv_slots;
    const int slot_id = (int)(rem / (uint32_t)n_chunks);
    const int c0 = (int)(rem % (uint32_t)n_chunks);
    const int c1 = (int)min((uint32_t)n_chunks, c0 + (u_end - u));
    u += (uint32_t)(c1 - c0);
    const int kvh = slot_id / g_chunks;
    const int g0 = (slot_id % g_chunks) * 16;  // first group member handled here
    const int n_heads = min(16, group - g0);
    int L = a.kv_len ? a.kv_len[b] : a.Lmax;
    L = min(max(L, 0), a.Lmax);
    const int start = c0 * a.chunk;
    const int end = min(L, c1 * a.chunk);
    const int split = c0;


  // Q^T fragments (B operand): lane (head n, g) holds q[head][32*ks + 8*g .. +7]; zero for padding heads
  vec8 qreg[KS];
  {
    const bool head_ok = n < n_heads;
    const int hq = q_head_of(kvh, head_ok ? g0 + n : 0, a.Hq, a.Hkv, a.head_map);
    const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + b * a.qs[0] + hq * a.qs[1];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      uint4 raw = make_uint4(0, 0, 0, 0);
      if (head_ok) raw = *reinterpret_cast<const uint4 *>(qp + 32 * ks + 8 * g);
      qreg[ks] = __builtin_bit_cast(vec8, raw);
    }
  }

  const uint16_t *kbase = reinterpret_cast<const uint16_t *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const uint16_t *vbase = reinterpret_cast<const uint16_t *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  floatx4_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++) oacc[db] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  float m_i = -INFINITY;  // running max of the raw scores of head n (same in the 4 lanes of a head)
  float l_i = 0.f;        // this lane's share of the running sum

  // Raw buffer descriptors over the valid rows [0, end) of this (b, kv head) slice: a load past `end` returns zeros
  // without a branch, so the loads of a block are NL back-to-back instructions (address = lane-invariant offset +
  // scalar block offset). Non-temporal, like every cache stream of this library.
  const __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t *>(kbase), 0, __builtin_amdgcn_readfirstlane(end * k_row_bytes), 0x00020000);
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t *>(vbase), 0, __builtin_amdgcn_readfirstlane(end * v_row_bytes), 0x00020000);
  uint4 kreg[NL], vreg[NL];
  auto load_tile = [&](int key0) {
    const int k_soff = __builtin_amdgcn_readfirstlane(key0 * k_row_bytes);
    const int v_soff = __builtin_amdgcn_readfirstlane(key0 * v_row_bytes);
#pragma unroll
    for (int r = 0; r < NL; r++) {
      kreg[r] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(k_rsrc, k_voff[r], k_soff, 2));
      vreg[r] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, v_voff[r], v_soff, 2));
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int r = 0; r < NL; r++) {
      const int id = r * 64 + lane;
      const int row = id / CPR, col = id % CPR;
      *reinterpret_cast<uint4 *>(&Ks[row * LDK + col * 8]) = kreg[r];
      *reinterpret_cast<uint4 *>(&Vs[row * LDV + col * 8]) = vreg[r];
    }
  };

  auto rotate_q = [&]() {
    // lmh_decode_step: this step's query is rotated at the position of the row the step appends, kv_len[b], as it is
    // loaded (apply_rotary_embeddings on the queries, reference src/NN.jl:356). Lane (n, g) holds elements
    // 32 ks + 8 g + e: the partner j + D/2 sits in fragment ks + KS/2 of the same lane when KS is even (the launcher
    // sends other head dims elsewhere), interleaved partners are neighbours inside a fragment.
    if (a.q_rope) {
      const float pos = (float)L;
      if (!a.rope_interleaved) {
        if constexpr (KS % 2 == 0) {
          constexpr int HK = KS / 2;
#pragma unroll
          for (int ks = 0; ks < HK; ks++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
              float o0, o1;
              rope_pair((float)qreg[ks][e], (float)qreg[ks + HK][e], pos, 32 * ks + 8 * g + e, D, a.rope_log2_base, &o0, &o1);
              qreg[ks][e] = MT::cvt(o0);
              qreg[ks + HK][e] = MT::cvt(o1);
            }
        }
      } else {
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            float o0, o1;
            rope_pair((float)qreg[ks][e], (float)qreg[ks][e + 1], pos, (32 * ks + 8 * g + e) / 2, D, a.rope_log2_base, &o0, &o1);
            qreg[ks][e] = MT::cvt(o0);
            qreg[ks][e + 1] = MT::cvt(o1);
          }
      }
    }
  };
  const int n_blocks = (end - start + kBlk - 1) / kBlk;
  if (wave < n_blocks) load_tile(start + wave * kBlk);
  rotate_q();  // (after the first loads are on their way: the rotation is a few hundred instructions per segment)

  for (int blk = wave; blk < n_blocks; blk += kWaves) {
    const int key0 = start + blk * kBlk;
    wave_lds_fence();  // the previous block's fragment reads precede these writes
    store_tile();
    wave_lds_fence();
    if (blk + kWaves < n_blocks) load_tile(key0 + kWaves * kBlk);  // in flight during the math below

    // ---- S^T = K Q^T for the two 16-key halves ----
    floatx4_t sacc[2];
#pragma unroll
    for (int hb = 0; hb < 2; hb++) {
      sacc[hb] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const vec8 kf = *reinterpret_cast<const vec8 *>(&Ks[k_frag_off + 16 * hb * LDK + 32 * ks]);
        sacc[hb] = MT::mfma(kf, qreg[ks], sacc[hb]);
      }
    }
    if (key0 + kBlk > end) {  // ragged last block
#pragma unroll
      for (int hb = 0; hb < 2; hb++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (key0 + 16 * hb + 4 * g + i >= end) sacc[hb][i] = -INFINITY;
    }

    // ---- online softmax; lane (n, g) owns head n ----
    float mx = fmaxf(fmaxf(fmaxf(sacc[0][0], sacc[0][1]), fmaxf(sacc[0][2], sacc[0][3])),
                     fmaxf(fmaxf(sacc[1][0], sacc[1][1]), fmaxf(sacc[1][2], sacc[1][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_i, mx);  // finite: key0 < end, so every head sees a key in this block
    const float alpha = __builtin_amdgcn_exp2f((m_i - m_new) * c);
    const float mc = m_new * c;
    m_i = m_new;
    // P is split into a 16-bit head and a 16-bit remainder (p = hi + lo to ~16 significant bits) and
    // both are multiplied with V: the matrix cores have time to spare here, and it keeps the result
    // independent of where the split boundaries fall to ~1e-5 instead of the 2^-9 of a single bf16 P.
    float psum = 0.f;
    vec8 pf, pf_lo;
#pragma unroll
    for (int hb = 0; hb < 2; hb++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const float p = __builtin_amdgcn_exp2f(sacc[hb][i] * c - mc);
        psum += p;
        pf[4 * hb + i] = MT::cvt(p);
        pf_lo[4 * hb + i] = MT::cvt(p - (float)pf[4 * hb + i]);
      }
    l_i = l_i * alpha + psum;
#pragma unroll
    for (int db = 0; db < DB; db++) oacc[db] *= alpha;

    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int db = 0; db < DB; db++) {
      const uint16_t *vaddr = &Vs[v_frag_off + 16 * db];
      const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr));
      const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr + 16 * LDV));
      const shortx8_t v8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      oacc[db] = MT::mfma(__builtin_bit_cast(vec8, v8), pf, oacc[db]);
      oacc[db] = MT::mfma(__builtin_bit_cast(vec8, v8), pf_lo, oacc[db]);
    }
  }

  // ---- merge the 4 waves, then write the split partial (or the final output) ----
  l_i += __shfl_xor(l_i, 16);
  l_i += __shfl_xor(l_i, 32);
  __syncthreads();  // all waves are done with their tiles: the memory is reused for the merge
  float *sm_o = reinterpret_cast<float *>(smem);              // [kWaves][16][D]
  float *sm_m = sm_o + kWaves * 16 * D;                       // [kWaves][16]
  float *sm_l = sm_m + kWaves * 16;                           // [kWaves][16]
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 4; i++) sm_o[(wave * 16 + n) * D + 16 * db + 4 * g + i] = oacc[db][i];
  if (g == 0) {
    sm_m[wave * 16 + n] = m_i * c;  // log2 units, like the vector kernel's partials
    sm_l[wave * 16 + n] = l_i;
  }
  __syncthreads();

  for (int idx = tid; idx < n_heads * D; idx += kWaves * 64) {
    const int h = idx / D, d = idx % D;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; w++) M = fmaxf(M, sm_m[w * 16 + h]);
    float lsum = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) {
      const float mw = sm_m[w * 16 + h];
      const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - M);
      lsum += sm_l[w * 16 + h] * f;
      o += sm_o[(w * 16 + h) * D + d] * f;
    }
    const int hq = q_head_of(kvh, g0 + h, a.Hq, a.Hkv, a.head_map);
    if (a.num_splits == 1) {
      const int64_t off = b * a.os[0] + hq * a.os[1] + d;
      if (a.out_f32) reinterpret_cast<float *>(a.out)[off] = o / lsum;
      else reinterpret_cast<uint16_t *>(a.out)[off] = MT::cvt_bits(o / lsum);
    } else {
      const int64_t row = ((int64_t)b * a.Hq + hq) * a.num_splits + split;
      a.ws_o[row * D + d] = o;
      if (d == 0) {
        a.ws_ml[row * 2 + 0] = M;
        a.ws_ml[row * 2 + 1] = lsum;
      }
    }
  }
  // the other chunk slots of this run hold nothing: mark them so the merge kernel skips them
  if (a.num_splits > 1) {
    for (int idx = tid; idx < n_heads * (c1 - c0 - 1); idx += kWaves * 64) {
      const int h = idx / (c1 - c0 - 1), cs = c0 + 1 + idx % (c1 - c0 - 1);
      const int hq = q_head_of(kvh, g0 + h, a.Hq, a.Hkv, a.head_map);
      const int64_t row = ((int64_t)b * a.Hq + hq) * a.num_splits + cs;
      a.ws_ml[row * 2 + 0] = -INFINITY;
      a.ws_ml[row * 2 + 1] = 0.f;
    }
  }
  __syncthreads();  // the merge buffers are tile memory again in the next segment
  }  // while (u < u_end)

  // A sequence without keys has no unit. With several splits the merge kernel writes its zeros; with one split
  // nothing else would write its output rows.
  if (a.num_splits == 1) {
    for (int b = blockIdx.x; b < a.B; b += gridDim.x) {
      if (s_pref[b + 1] != s_pref[b]) continue;
      for (int idx = tid; idx < a.Hq * D; idx += kWaves * 64) {
        const int64_t off = b * a.os[0] + (idx / D) * a.os[1] + idx % D;
        if (a.out_f32) reinterpret_cast<float *>(a.out)[off] = 0.f;
        else reinterpret_cast<uint16_t *>(a.out)[off] = 0;
      }
    }
  }
}

template <typename MT, int D>
int launch_for_d(const DecodeArgs &a, hipStream_t stream) {
  // Persistent launch: as many workgroups as the chip holds at once (never more than there are units).
  // Same for every device this library runs on (gfx950 only); initialised once, thread-safely.
  static const int wgs_per_device = [] {
    int dev = 0, per_cu = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, decode_mfma_kernel<MT, D>, kWaves * 64, 0) != hipSuccess) {
      (void)hipGetLastError();
      return 256;  // one workgroup per CU: correct for any value, only the balance changes
    }
    return (per_cu < 1 ? 1 : per_cu) * prop.multiProcessorCount;
  }();
  const int group = a.Hq / a.Hkv;
  const int g_chunks = (group + 15) / 16;
  const int64_t max_units = (int64_t)a.B * a.Hkv * g_chunks * a.num_splits;
  if (max_units >= (int64_t(1) << 31)) return fail(LMH_E_UNSUPPORTED, "MFMA decode: %lld units do not fit 32 bits", (long long)max_units);
  const int n_wgs = (int)(max_units < wgs_per_device ? max_units : wgs_per_device);
  hipLaunchKernelGGL((decode_mfma_kernel<MT, D>), dim3(n_wgs), dim3(kWaves * 64), 0, stream, a, g_chunks);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

template <typename MT>
int launch_for_type(const DecodeArgs &a, hipStream_t stream) {
  switch (a.D) {
    case 64: return launch_for_d<MT, 64>(a, stream);
    case 96: return launch_for_d<MT, 96>(a, stream);
    case 128: return launch_for_d<MT, 128>(a, stream);
    case 256: return launch_for_d<MT, 256>(a, stream);
  }
  return fail(LMH_E_UNSUPPORTED, "MFMA decode: head dim %d not tiled", a.D);
}

}  // namespace

// The query rotation of lmh_decode_step happens in registers: the partner of every element must be in the same lane.
bool decode_mfma_rope_ok(int D, int interleaved) { return interleaved || (D / 32) % 2 == 0; }

bool decode_mfma_supported(int dtype, int D, int B) {
  return (dtype == LMH_F16 || dtype == LMH_BF16) && (D == 64 || D == 96 || D == 128 || D == 256) &&
         B <= kMaxBatchPersistent;
}

// Enqueues only the split kernel; the caller adds the merge kernel when num_splits > 1.
int launch_decode_mfma_split(const DecodeArgs &a, int dtype, hipStream_t stream) {
  if (dtype == LMH_F16) return launch_for_type<Mfma16F16>(a, stream);
  if (dtype == LMH_BF16) return launch_for_type<Mfma16BF16>(a, stream);
  return fail(LMH_E_UNSUPPORTED, "MFMA decode: dtype %d has no matrix-core path", dtype);
}

}  // namespace lmh
