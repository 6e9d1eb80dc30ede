// Flash attention forward in fp32 on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32).
//
// fp32 is the reference's only element type (flash_attn_cpu, reference src/Execution.jl:453-479), and its
// parity budget (1e-5 of the output range) rules out half-precision operands, so this kernel keeps Q, K,
// V and P in fp32 end to end; only the order of the fp32 additions differs from the reference's loop.
//
// Same structure as prefill_mfma.hip: a workgroup of 4 waves owns 128 query rows of one (b, hq), a wave
// 32 of them with its Q fragments in registers; scores are computed transposed, S^T = K Q^T, so a lane
// holds one query column and the softmax statistics are per-lane scalars; the accumulator registers that
// hold P are directly the B operands of O^T = V^T P^T (no conversion, no LDS round trip). Differences:
//   * the MFMA contracts 2 elements at a time (lane half g supplies one of them), so a 128-bit K fragment
//     read feeds four MFMAs: the head dim is contracted in the order d = 8j + 4g + e, the same in Q and K;
//   * the contraction over keys in the second product follows the accumulator layout: MFMA i of a 32-key
//     tile pairs key 8(i/4) + (i%4) from lanes 0-31 with key 8(i/4) + 4 + (i%4) from lanes 32-63, and the
//     V^T fragment is one 32-bit LDS read of those two rows;
//   * tiles are 32 keys (fp32 tiles are twice as large in LDS) and exp2 runs on v_exp_f32 with the scale
//     folded into the argument, as in the half-precision kernel.
// The matrix pipe does 64 flops per cycle per SIMD in fp32 (157 TFLOP/s peak), 16 times less than in
// fp16, so the ~70 vector instructions and ~80 LDS reads per tile hide behind 64-128 MFMAs of 64 cycles.
#include "common.hpp"
#include "dtypes.hpp"
#include "rope.hpp"

namespace lmh {
namespace {

constexpr int BN = 32;   // keys a wave takes per tile
constexpr int kPadK = 4;  // floats: a row stride of D + 4 puts 16 consecutive rows' 16-byte reads on distinct banks
constexpr int kPadV = 8;  // floats: rows key and key + 4 (the two halves of a wave) land 32 banks apart
constexpr float kLog2e = 1.4426950408889634f;
// Byte offset no K/V slice reaches (the host routes larger ones elsewhere): a buffer load there is out of
// range and returns zeros.
constexpr int kOutOfRange = 0x7ffffff0;
constexpr float kLazyRescale = 8.0f;  // see prefill_mfma.hip: the running max is raised only when outgrown by 2^8
typedef float floatx4_t __attribute__((ext_vector_type(4)));

// KSPLIT = 1: the four waves own 4 x 32 query rows and walk the same 32-key tiles.
// KSPLIT = 2, 4: for launches far too small to fill the chip (the reference's own test sizes), where the
// time is one wave's walk over its keys at 64 cycles per MFMA. The workgroup owns 128 / KSPLIT query rows
// and stages tiles of 32 KSPLIT keys; wave group kg takes keys 32 kg .. 32 kg + 31 of every tile with its
// own running max / sum / output, and the groups are merged through LDS at the end.
template <int D, bool CAUSAL, int KSPLIT>
__global__ __launch_bounds__(256, (KSPLIT > 1 ? 1 : D <= 96 ? 3 : 2)) void prefill_f32_kernel(PrefillArgs a, int n_q_tiles, int n_bh_groups) {
  request_args(a);
  request_arg(n_q_tiles);
  request_arg(n_bh_groups);
  constexpr int BM = 128 / KSPLIT;  // query rows per workgroup
  constexpr int BT = BN * KSPLIT;   // keys per staged tile
  constexpr int RG = 4 / KSPLIT;    // waves (32-row groups) per key group
  constexpr int KJ = D / 8;         // 128-bit K fragments per tile (4 MFMAs each)
  constexpr int DB = D / 32;        // 32-row blocks of O^T
  constexpr int CPR = D / 4;        // 16-byte chunks per K/V row of the tiling
  // the tensors' own head dim a.D may be smaller than the tiled D (any multiple of 8): the missing
  // columns are never fetched (zeros in Q, K and V) and never stored.
  const int cpr = a.D / 4;
  constexpr int LDK = D + kPadK;    // LDS row strides in floats
  constexpr int LDV = D + kPadV;

  constexpr int KC = LDK / 4, VC = LDV / 4;                            // 16-byte chunks per LDS row
  constexpr int KI = (BT * KC + 63) / 64, VI = (BT * VC + 63) / 64;  // 1 KB blocks per tile (the last may be half used)
  __shared__ __attribute__((aligned(16))) float Ks2[2][KI * 256];     // double-buffered tiles, whole blocks
  __shared__ __attribute__((aligned(16))) float Vs2[2][VI * 256];

  // ---- which (b, hq, query tile) this workgroup owns: see prefill_mfma.hip ----
  const int bid = blockIdx.x;
  const int xcd = bid & 7;
  const int idx = bid >> 3;
  const int tile_rank = idx / n_bh_groups;
  const int bh = (idx % n_bh_groups) * 8 + xcd;
  if (bh >= a.B * a.Hq) return;
  const int b = bh / a.Hq, hq = bh % a.Hq;
  const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
  const int q_tile = CAUSAL ? (n_q_tiles - 1 - tile_rank) : tile_rank;
  const int q0 = q_tile * BM;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, g = lane >> 5;
  const int kg = wave / RG;  // key group of this wave (always 0 when KSPLIT == 1)
  const int wave_q_lo = q0 + (wave % RG) * 32;
  const int wave_q_hi = wave_q_lo + 31;
  const int qi = wave_q_lo + n;

  int n_keys = a.kv_len ? a.kv_len[b] : a.Sk;
  n_keys = min(max(n_keys, 0), a.Sk);
  int k_end = n_keys;
  if (CAUSAL) k_end = min(k_end, q0 + BM);
  const int n_kv_tiles = (k_end + BT - 1) / BT;

  const float *qp = reinterpret_cast<const float *>(a.q) + b * a.qs[0] + hq * a.qs[1];
  const float *kp = reinterpret_cast<const float *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const float *vp = reinterpret_cast<const float *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  // ---- Q fragments: lane (n, g) holds q[qi][8j + 4g .. + 3] for every j ----
  floatx4_t qf[KJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    float4 raw = make_float4(0.f, 0.f, 0.f, 0.f);
    if (qi < a.Sq && 8 * j + 4 * g < a.D) raw = *reinterpret_cast<const float4 *>(qp + (int64_t)qi * a.qs[2] + 8 * j + 4 * g);
    qf[j] = (floatx4_t){raw.x, raw.y, raw.z, raw.w};
  }

  floatx16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;
  float m_i = -INFINITY;  // running max of the raw (unscaled) scores of query qi
  float l_i = 0.f;        // this lane's half of the running sum
  const float c = a.scale * kLog2e;

  // ---- tile staging: global memory -> LDS directly (buffer_load_dwordx4 ... lds), one tile ahead; see
  // prefill_mfma.hip. A wave-wide load fills a 1 KB block, lane l's 16 bytes at block + 16 l from that lane's
  // own global offset; lanes on a padding chunk, past the tile's last row or past the tensors' head dim fetch
  // out of range (zeros), rows past n_keys read as zero through the descriptor's bounds. ----
  typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) void lds_void_t;
  constexpr int KBW = (KI + 3) / 4, VBW = (VI + 3) / 4;  // blocks per wave (rounded up)
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  __builtin_assume(wave_u >= 0 && wave_u < 4);
  auto make_desc = [](const float *base, int bytes) {
    const uint64_t p = (uint64_t)base;
    i32x4_t d;
    d[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    d[1] = __builtin_amdgcn_readfirstlane((int)((p >> 32) & 0xffff));  // stride 0: raw buffer
    d[2] = __builtin_amdgcn_readfirstlane(bytes);
    d[3] = 0x00020000;
    return d;
  };
  const i32x4_t k_desc = make_desc(kp, (int)((int64_t)n_keys * a.ks[2] * 4));
  const i32x4_t v_desc = make_desc(vp, (int)((int64_t)n_keys * a.vs[2] * 4));
  int k_voff[KBW], v_voff[VBW];
#pragma unroll
  for (int j = 0; j < KBW; j++) {
    const int ch = (wave + 4 * j) * 64 + lane;
    const int row = ch / KC, col = ch % KC;
    k_voff[j] = (row < BT && col < cpr) ? (int)((row * a.ks[2] + col * 4) * 4) : kOutOfRange;
  }
#pragma unroll
  for (int j = 0; j < VBW; j++) {
    const int ch = (wave + 4 * j) * 64 + lane;
    const int row = ch / VC, col = ch % VC;
    v_voff[j] = (row < BT && col < cpr) ? (int)((row * a.vs[2] + col * 4) * 4) : kOutOfRange;
  }
  const int k_tile_bytes = (int)(BT * a.ks[2] * 4), v_tile_bytes = (int)(BT * a.vs[2] * 4);
  const uint32_t k_lds0 = (uint32_t)(uintptr_t)(lds_void_t *)&Ks2[0][0] + wave_u * 1024;
  const uint32_t v_lds0 = (uint32_t)(uintptr_t)(lds_void_t *)&Vs2[0][0] + wave_u * 1024;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is a reserved register; it is only written here
  auto load_block = [](i32x4_t desc, uint32_t lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(desc), "s"(soff) : "memory", "m0");
  };
#pragma clang diagnostic pop
  auto load_tile = [&](int kt, int buf) {
#pragma unroll
    for (int j = 0; j < KBW; j++)
      if (wave_u + 4 * j < KI) load_block(k_desc, k_lds0 + buf * (KI * 1024) + j * 4096, k_voff[j], kt * k_tile_bytes);
#pragma unroll
    for (int j = 0; j < VBW; j++)
      if (wave_u + 4 * j < VI) load_block(v_desc, v_lds0 + buf * (VI * 1024) + j * 4096, v_voff[j], kt * v_tile_bytes);
  };

  const int k_frag_off = n * LDK + 4 * g;  // + 8 * j
  const int v_frag_off = 4 * g * LDV + n;  // + (8 * (i / 4) + i % 4) * LDV + 32 * db

  if (n_kv_tiles > 0) load_tile(0, 0);
  // Rotary embedding of the query fragments in registers (PrefillArgs::q_rope; the head dim equals the tiling). Lane
  // (n, g) holds elements 8 j + 4 g + e: the partner j' + D/2 of element j' is fragment j + D/16 of the same lane, the
  // interleaved pairs are neighbours. inv_freq is computed once per workgroup into the second K buffer, which nothing
  // writes before the loop's first barrier.
  if (a.q_rope) {
    float *table = &Ks2[1][0];
    if (tid < D / 2) table[tid] = rope_inv_freq(tid, D, a.q_log2_base);
    __syncthreads();
    const float pos = (float)((a.q_pos0 ? a.q_pos0[b] : a.q_prev_seq) + qi);
    if (!a.q_interleaved) {
#pragma unroll
      for (int j = 0; j < KJ / 2; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          float sn, cs, o0, o1;
          sincos_angle(pos * table[8 * j + 4 * g + e], &sn, &cs);
          rope_rotate(qf[j][e], qf[j + KJ / 2][e], sn, cs, &o0, &o1);
          qf[j][e] = o0;
          qf[j + KJ / 2][e] = o1;
        }
    } else {
#pragma unroll
      for (int j = 0; j < KJ; j++)
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          float sn, cs, o0, o1;
          sincos_angle(pos * table[(8 * j + 4 * g + e) / 2], &sn, &cs);
          rope_rotate(qf[j][e], qf[j][e + 1], sn, cs, &o0, &o1);
          qf[j][e] = o0;
          qf[j][e + 1] = o1;
        }
    }
  }
  // The compiler does not model the asm loads or the asm wait below: make it wait for Q here, not inside the loop.
#pragma unroll
  for (int j = 0; j < KJ; j++) asm volatile("" :: "v"(qf[j]));

  for (int kt = 0; kt < n_kv_tiles; kt++) {
    // One barrier per tile: tile kt (fetched during the previous iteration) becomes visible, and every
    // wave is done with tile kt-1, whose buffer the fetch of tile kt+1 now overwrites.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's blocks of tile kt are in LDS
    __syncthreads();
    if (kt + 1 < n_kv_tiles) load_tile(kt + 1, (kt + 1) & 1);
    const float *Ks = Ks2[kt & 1] + kg * (BN * LDK);
    const float *Vs = Vs2[kt & 1] + kg * (BN * LDV);

    const int k0 = kt * BT + kg * BN;         // first key of this wave's share of the tile
    if (CAUSAL && k0 > wave_q_hi) continue;   // all of it above this wave's diagonal
    if (KSPLIT > 1 && k0 >= k_end) continue;  // ... or past the last key

    // ---- S^T = K Q^T: 32 keys x 32 queries, contraction over the head dim two elements per MFMA ----
    floatx16_t sacc;
#pragma unroll
    for (int i = 0; i < 16; i++) sacc[i] = 0.f;
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      const floatx4_t kf = *reinterpret_cast<const floatx4_t *>(&Ks[k_frag_off + 8 * j]);
#pragma unroll
      for (int e = 0; e < 4; e++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[e], qf[j][e], sacc, 0, 0, 0);
    }

    // ---- masking (diagonal tiles and the ragged last tile only) ----
    const bool need_mask = (k0 + BN > n_keys) || (CAUSAL && k0 + BN - 1 > wave_q_lo);
    if (need_mask) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int key = k0 + 8 * (i >> 2) + 4 * g + (i & 3);
        if (key >= n_keys || (CAUSAL && key > qi)) sacc[i] = -INFINITY;
      }
    }

    // ---- online softmax; all statistics are per lane (one query column) ----
    float mx = sacc[0];
#pragma unroll
    for (int i = 1; i < 16; i++) mx = fmaxf(mx, sacc[i]);
    mx = max_over_wave_halves(mx);
    // m_i is finite after the first tile (key 0 is visible to every query); -inf before it.
    if (__builtin_amdgcn_ballot_w64((mx - m_i) * c > kLazyRescale) != 0) {  // wave-uniform
      const float m_new = fmaxf(m_i, mx);
      const float alpha = __builtin_amdgcn_exp2f((m_i - m_new) * c);
      m_i = m_new;
      l_i *= alpha;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
    }
    const float mc = m_i * c;
    float l0 = 0.f, l1 = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) {
      sacc[i] = __builtin_amdgcn_exp2f(sacc[i] * c - mc);
      sacc[i + 1] = __builtin_amdgcn_exp2f(sacc[i + 1] * c - mc);
      l0 += sacc[i];
      l1 += sacc[i + 1];
    }
    l_i += l0 + l1;

    // ---- O^T += V^T P^T: MFMA i contracts the two keys lanes (., 0) and (., 1) hold in register i ----
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const float *vrow = &Vs[v_frag_off + (8 * (i >> 2) + (i & 3)) * LDV];
#pragma unroll
      for (int db = 0; db < DB; db++) oacc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * db], sacc[i], oacc[db], 0, 0, 0);
    }
  }

  // ---- key groups: fold the other groups' (m, l, O) into group 0's; lane for lane the same layout ----
  if (KSPLIT > 1) {
    constexpr int NF = DB * 16 + 2;  // floats per lane
    static_assert(KSPLIT == 1 || (KSPLIT - 1) * RG * NF * 64 * 4 <= (int)sizeof(Ks2), "merge buffer must fit in the K tiles");
    float *xch = &Ks2[0][0] + (wave % RG) * (NF * 64) + lane;  // [KSPLIT - 1][RG][NF][64 lanes]
    __syncthreads();  // every wave has read its last tile
    if (kg > 0) {
      float *w = xch + (kg - 1) * (RG * NF * 64);
      w[0] = m_i;
      w[64] = l_i;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) w[(2 + db * 16 + i) * 64] = oacc[db][i];
    }
    __syncthreads();
    if (kg > 0) return;
#pragma unroll
    for (int og = 1; og < KSPLIT; og++) {
      const float *r = xch + (og - 1) * (RG * NF * 64);
      const float m1 = r[0], l1 = r[64];
      const float m_new = fmaxf(m_i, m1);
      // a group that saw no key has m = -inf, l = 0, O = 0
      const float a0 = m_i == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m_i - m_new) * c);
      const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m1 - m_new) * c);
      m_i = m_new;
      l_i = l_i * a0 + l1 * a1;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] = oacc[db][i] * a0 + r[(2 + db * 16 + i) * 64] * a1;
    }
  }

  // ---- epilogue: out[qi][d] = O^T[d][qi] / l ----
  const float l_tot = sum_over_wave_halves(l_i);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (qi < a.Sq) {
    float *op = reinterpret_cast<float *>(a.out) + b * a.os[0] + hq * a.os[1] + (int64_t)qi * a.os[2];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int d = db * 32 + 8 * i4 + 4 * g;
        if (d >= a.D) continue;
        *reinterpret_cast<float4 *>(op + d) = make_float4(oacc[db][4 * i4 + 0] * inv, oacc[db][4 * i4 + 1] * inv,
                                                          oacc[db][4 * i4 + 2] * inv, oacc[db][4 * i4 + 3] * inv);
      }
  }
}

template <int D, int KSPLIT>
int launch_split(const PrefillArgs &a, hipStream_t stream) {
  const int n_q_tiles = (a.Sq + 128 / KSPLIT - 1) / (128 / KSPLIT);
  const int n_bh_groups = (a.B * a.Hq + 7) / 8;
  dim3 grid(8 * n_bh_groups * n_q_tiles), block(256);
  if (plan_only("prefill_f32_kernel<D=%d, %s, key groups=%d> workgroups=%u", D, a.causal ? "causal" : "full", KSPLIT, grid.x))
    return LMH_OK;
  if (a.causal)
    hipLaunchKernelGGL((prefill_f32_kernel<D, true, KSPLIT>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  else
    hipLaunchKernelGGL((prefill_f32_kernel<D, false, KSPLIT>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

template <int D>
int launch_for_d(const PrefillArgs &a, hipStream_t stream) {
  // The key-split workgroups hold tiles of 64 or 128 keys in LDS, one workgroup per CU: use them only while
  // every workgroup still gets a CU of its own. (Four-way needs 143 KB at D = 64 and does not fit beyond.)
  const int n_cus = device_cu_count();
  const int64_t wgs = (int64_t)((a.B * a.Hq + 7) / 8) * 8 * ((a.Sq + 127) / 128);
  if (D == 64 && 4 * wgs <= n_cus && a.Sk >= 4 * BN) return launch_split<D, (D == 64 ? 4 : 1)>(a, stream);
  if (2 * wgs <= n_cus && a.Sk >= 2 * BN) return launch_split<D, 2>(a, stream);
  return launch_split<D, 1>(a, stream);
}

}  // namespace

bool prefill_f32_mfma_supported(int dtype, int D) { return dtype == LMH_F32 && D >= 8 && D <= 128 && D % 8 == 0; }

int launch_prefill_f32_mfma(const PrefillArgs &a, hipStream_t stream) {
  if (a.D <= 64) return launch_for_d<64>(a, stream);
  if (a.D <= 96) return launch_for_d<96>(a, stream);
  if (a.D <= 128) return launch_for_d<128>(a, stream);
  return fail(LMH_E_UNSUPPORTED, "fp32 MFMA flash attention: head dim %d not tiled", a.D);
}

}  // namespace lmh
