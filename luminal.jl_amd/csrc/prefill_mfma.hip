// Flash attention forward on the gfx950 matrix cores (fp16 / bf16 in, fp32 accumulate).
//
// Same mathematics as flash_attn_cpu (reference src/Execution.jl:453-479) — online softmax with a
// running max m, running sum l and an un-normalised output row — evaluated 64 keys at a time for
// 128 or 256 query rows per workgroup instead of one (i, j) pair at a time.
//
// Tiling (wave64, v_mfma_f32_32x32x16):
//   * workgroup = 4 waves = 128 query rows of one (b, hq) (8 waves = 256 rows in launches large
//     enough to stay balanced with them); each wave owns 32 query rows and keeps their Q
//     fragments in registers for the whole kernel;
//   * the scores are computed TRANSPOSED, S^T = K Q^T (M = keys, N = queries). In the MFMA
//     accumulator layout a lane then holds one query column (n = lane % 32) and 16 of the 32 keys
//     of a block, so the softmax statistics (max, sum, rescale factor) are per-lane scalars and
//     the only cross-lane traffic is one exchange with lane ^ 32;
//   * the same registers, converted to half precision, are directly the B operand of the second
//     product O^T = V^T P^T (M = head dim, N = queries, contraction over keys), so P never
//     touches LDS;
//   * K and V tiles (64 keys) go from global memory straight into double-buffered LDS, row-major,
//     with LDS-writing buffer loads (no register staging, no LDS store instructions); the K
//     fragment is a plain 128-bit LDS read (contraction over the contiguous head dim), the V^T
//     fragment uses the gfx950 transposing LDS read ds_read_b64_tr_b16, which hands each lane 4
//     consecutive keys of its head-dim column;
//   * causal: key tiles beyond the workgroup's last query are never loaded, a wave skips tiles that
//     lie entirely above its diagonal, and only diagonal tiles pay for masking;
//   * blockIdx -> work mapping keeps all query tiles of a head on one XCD (private L2) and, for
//     causal, issues the long rows first.
#include <type_traits>

#include "prefill_mfma.hpp"
#include "rope.hpp"

#if (defined(LMH_FOLD_SCALE) || defined(LMH_ONLY_XCDS) || defined(LMH_WIDE_MARGIN) || defined(LMH_W64_KERNEL) || defined(LMH_NO_PAIR_KERNEL) || \
     defined(LMH_BF16_SPLIT_P) || defined(LMH_NO_MIXED_KEY_GROUPS)) && \
    !defined(LMH_MEASUREMENT_BUILD)
#error "LMH_FOLD_SCALE / LMH_ONLY_XCDS / LMH_WIDE_MARGIN / LMH_W64_KERNEL / LMH_NO_PAIR_KERNEL / LMH_BF16_SPLIT_P / LMH_NO_MIXED_KEY_GROUPS are experiment switches: they need -DLMH_MEASUREMENT_BUILD, which marks the library"
#endif

#ifndef LMH_WIDE_MARGIN
#define LMH_WIDE_MARGIN 0.9
#endif

namespace lmh {
namespace {


// Rotary embedding of the wave's query fragments in registers (PrefillArgs::q_rope). Lane (n, g) holds elements
// 16 ks + 8 g + e of its row; with the head dim equal to the tiling, the partner j + D/2 of element j sits in
// fragment ks + D/32 of the same lane (the interleaved pairs are neighbours inside a fragment). inv_freq does not
// depend on the row: the workgroup computes its D/2 values once into `table` (LDS that nothing else uses before the
// next barrier) and every lane multiplies them by its own position. Every thread of the workgroup must call this.
template <typename MT, int D>
__device__ inline void rotate_q_fragments_with_table(typename MT::vec8 (&qreg)[D / 16], const PrefillArgs &a, int b, int qi, int g, const float *table);
template <typename MT, int D>
__device__ inline void rotate_q_fragments(typename MT::vec8 (&qreg)[D / 16], const PrefillArgs &a, int b, int qi, int g, float *table) {
  if ((int)threadIdx.x < D / 2) table[threadIdx.x] = rope_inv_freq(threadIdx.x, D, a.q_log2_base);
  __syncthreads();
  rotate_q_fragments_with_table<MT, D>(qreg, a, b, qi, g, table);
}
// the rotation itself, given the workgroup's table of D / 2 inverse frequencies
template <typename MT, int D>
__device__ inline void rotate_q_fragments_with_table(typename MT::vec8 (&qreg)[D / 16], const PrefillArgs &a, int b, int qi, int g, const float *table) {
  constexpr int KS = D / 16, HK = D / 32;
  const float pos = (float)((a.q_pos0 ? a.q_pos0[b] : a.q_prev_seq) + qi);
  if (!a.q_interleaved) {
#pragma unroll
    for (int ks = 0; ks < HK; ks++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float sn, cs, o0, o1;
        sincos_angle(pos * table[16 * ks + 8 * g + e], &sn, &cs);
        rope_rotate((float)qreg[ks][e], (float)qreg[ks + HK][e], sn, cs, &o0, &o1);
        qreg[ks][e] = MT::cvt(o0);
        qreg[ks + HK][e] = MT::cvt(o1);
      }
  } else {
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        float sn, cs, o0, o1;
        sincos_angle(pos * table[(16 * ks + 8 * g + e) / 2], &sn, &cs);
        rope_rotate((float)qreg[ks][e], (float)qreg[ks][e + 1], sn, cs, &o0, &o1);
        qreg[ks][e] = MT::cvt(o0);
        qreg[ks][e + 1] = MT::cvt(o1);
      }
  }
}

// NW waves per workgroup, 32 query rows each, walking the same 64-key tiles (KSPLIT = 1).
// NW = 8 (256 query rows) stages every K/V tile once per 256 rows instead of once per 128: 3-8 % faster
// wherever there are enough workgroups to keep the balance. Head dims up to 96: two such workgroups =
// 4 waves per SIMD on a CU, at most 128 registers. D = 128: one workgroup per CU, 2 waves per SIMD, as
// with the 128-row workgroups there.
// KSPLIT = 2: for launches too small to fill the chip. The workgroup owns 64 query rows; waves 0-1
// take them against the first 32 keys of every tile, waves 2-3 against the second 32, each pair
// with its own running max / sum / output, merged through LDS at the end. Twice the workgroups,
// and a wave's share of a tile is half as long.
// The second launch bound is waves per SIMD.
// WPS: waves per SIMD the register budget is set for (3 x 4 waves, 2 x 8 waves or 1 x 8 waves per CU).
template <int D, int NW> constexpr int default_wps() { return D > 96 ? 2 : NW == 8 ? 4 : 3; }
template <typename MT, int D, bool CAUSAL, int KSPLIT, int NW, int WPS>
__global__ __launch_bounds__(64 * NW, WPS) void prefill_mfma_kernel(PrefillArgs a, int n_q_tiles, int n_bh_groups) {
  request_args(a);
  request_arg(n_q_tiles);
  request_arg(n_bh_groups);
  using vec8 = typename MT::vec8;
  constexpr int BM = 32 * NW / KSPLIT;  // query rows per workgroup
  // keys per staged tile: 64; 128 where one workgroup has the CU to itself and LDS and registers allow (half the
  // barriers and per-tile bookkeeping: 114.2 -> 111.9 us on B=1 H=32 S=4096 causal)
  constexpr int BT = (NW == 8 && WPS == 2 && D <= 96 && KSPLIT == 1) ? 2 * BN : BN;
  constexpr int RG = NW / KSPLIT;   // waves (32-row groups) per key group
  constexpr int NKB = BT / 32 / KSPLIT;   // 32-key blocks a wave takes per tile
  constexpr int BW = 32 * NKB;      // ... in keys
  constexpr int KS = D / 16;       // k-steps of the S^T product
  constexpr int DB = D / 32;       // 32-row blocks of O^T
  // D is the tiled head dim; the tensors' own head dim a.D may be smaller (any multiple of 8): the
  // missing columns are never fetched (zeros in Q, K and V) and never stored.
  const int cpr = a.D / 8;         // 16-byte chunks per K/V row in memory
  constexpr bool CV = MT::kConvertV;  // V tiles rewritten as fp16 on their way into LDS
  using pvec8 = typename MT::pvec8;
  constexpr int LDK = D + kPadK;   // LDS row strides in elements
  constexpr int LDV = D + pad_v<D>();

  __shared__ __attribute__((aligned(16))) uint16_t Ks2[2][BT * LDK];  // double-buffered tiles
  __shared__ __attribute__((aligned(16))) uint16_t Vs2[2][BT * LDV];

#ifdef LMH_ONLY_XCDS
  // Measurement build (results wrong by construction): only workgroups dispatched to the first LMH_ONLY_XCDS XCDs
  // work, the rest exit at once — the same instruction stream with part of the chip idle.
  if ((blockIdx.x & 7) >= LMH_ONLY_XCDS) return;
#endif
  // ---- which (b, hq, query tile) this workgroup owns ----
  const int bid = blockIdx.x;
  const int xcd = bid & 7;
  const int idx = bid >> 3;
  const int tile_rank = idx / n_bh_groups;
  const int bh = (idx % n_bh_groups) * 8 + xcd;
  if (bh >= a.B * a.Hq) return;
  const int b = bh / a.Hq, hq = bh % a.Hq;
  const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
  // Causal rows grow with the query index: long rows are issued first so that the short ones fill
  // the tail of the launch. (Pairing tile r with tile n-1-r in one workgroup equalises the work but
  // halves the number of workgroups; measured 15 % slower on the S = 4096 workload.)
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

  const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + b * a.qs[0] + hq * a.qs[1];
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  // ---- Q fragments: B operand of S^T = K Q^T; lane (n, g) holds q[qi][16*ks + 8*g .. +7] ----
  vec8 qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (qi < a.Sq && 16 * ks + 8 * g < a.D) raw = *reinterpret_cast<const uint4 *>(qp + (int64_t)qi * a.qs[2] + 16 * ks + 8 * g);
    qreg[ks] = __builtin_bit_cast(vec8, raw);
#ifdef LMH_FOLD_SCALE
    // Measurement build, not the shipped path: scale * log2(e) multiplied into the Q fragments (rounded to the element
    // type once more), the running max kept in log2 units and handed to the first QK^T MFMA of a block as its
    // accumulator input, so that the MFMAs deliver the argument of exp2 and the per-score v_fma disappears. The extra
    // rounding moves a logit by up to 2^-12 of its magnitude: 1.5e-4 of the output range at a row max of 4 (log2 units),
    // 4.5e-4 at 16, 1.5e-3 at 45, over the 2e-3 budget at a few hundred (the large-logit parity tests fail).
#pragma unroll
    for (int e = 0; e < 8; e++) qreg[ks][e] = MT::cvt((float)qreg[ks][e] * (a.scale * kLog2e));
#endif
  }

  floatx16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;
  float m_i = -INFINITY;  // running max of the raw (unscaled) scores of query qi
  float l_i = 0.f;        // this lane's half of the running sum
  const float c = a.scale * kLog2e;
#ifdef LMH_FOLD_SCALE
  float neg_mc = 0.f;     // minus the running max, in log2 units ...
  floatx16_t neg_mc16;    // ... and as the accumulator input of a block's first MFMA (rewritten only when the max is raised)
#pragma unroll
  for (int i = 0; i < 16; i++) neg_mc16[i] = 0.f;
  bool have_m = false;
#endif

  // ---- tile staging: global memory -> LDS directly (buffer_load_dwordx4 ... lds), one tile ahead ----
  // A tile of BT rows x LD elements is BT * LD / 512 blocks of 1 KB. One wave-wide load fills one block:
  // lane l's 16 bytes land at block + 16 l, fetched from that lane's own global offset, so the
  // padded row layout needs no register staging and no LDS store instructions. Lanes that fall on
  // a padding chunk fetch out of range. The descriptor's size is the end of the last valid key row:
  // rows past n_keys arrive as zeros without a branch, and the per-lane offsets are loop
  // invariants. Wave w issues blocks w, w + NW, ...
  // The load is written in asm because the compiler, when it knows of an LDS-writing load in
  // flight, waits for it before the next LDS read of the same array — which would serialise the
  // prefetch of tile kt + 1 with the fragment reads of tile kt. The wait that matters (this wave's
  // loads have landed, then the workgroup barrier) is written out at the top of the loop.
  typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) void lds_void_t;
  constexpr int KC = LDK / 8, VC = LDV / 8;            // 16-byte chunks per LDS row
  constexpr int KI = KC * BT / 64, VI = VC * BT / 64;  // 1 KB blocks per tile
  constexpr int KJ = (KI + NW - 1) / NW, VJ = (VI + NW - 1) / NW;  // blocks per wave (rounded up)
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  __builtin_assume(wave_u >= 0 && wave_u < NW);
  auto make_desc = [](const uint16_t *base, int bytes) {
    const uint64_t p = (uint64_t)base;
    i32x4_t d;
    d[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    d[1] = __builtin_amdgcn_readfirstlane((int)((p >> 32) & 0xffff));  // stride 0: raw buffer
    d[2] = __builtin_amdgcn_readfirstlane(bytes);
    d[3] = 0x00020000;
    return d;
  };
  const i32x4_t k_desc = make_desc(kp, (int)((int64_t)n_keys * a.ks[2] * 2));
  const i32x4_t v_desc = make_desc(vp, (int)((int64_t)n_keys * a.vs[2] * 2));
  int k_voff[KJ], v_voff[VJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    const int ch = (wave + NW * j) * 64 + lane;
    const int row = ch / KC, col = ch % KC;
    k_voff[j] = col < cpr ? (int)((row * a.ks[2] + col * 8) * 2) : kOutOfRange;
  }
#pragma unroll
  for (int j = 0; j < VJ; j++) {
    const int ch = (wave + NW * j) * 64 + lane;
    const int row = ch / VC, col = ch % VC;
    v_voff[j] = col < cpr ? (int)((row * a.vs[2] + col * 8) * 2) : kOutOfRange;
  }
  const int k_tile_bytes = (int)(BT * a.ks[2] * 2), v_tile_bytes = (int)(BT * a.vs[2] * 2);
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
    for (int j = 0; j < KJ; j++)
      if (wave_u + NW * j < KI)
        load_block(k_desc, k_lds0 + buf * (BT * LDK * 2) + j * (NW * 1024), k_voff[j], kt * k_tile_bytes);
    if constexpr (!CV) {
#pragma unroll
      for (int j = 0; j < VJ; j++)
        if (wave_u + NW * j < VI)
          load_block(v_desc, v_lds0 + buf * (BT * LDV * 2) + j * (NW * 1024), v_voff[j], kt * v_tile_bytes);
    }
  };

  // ---- MT::kConvertV: V tiles pass through registers and are stored in LDS as fp16 relative to the largest finite |v|
  // met so far. Tile kt + 1 is rewritten during iteration kt from registers loaded during iteration kt - 1; the
  // workgroup agrees on the largest value through v_top[parity of the tile], posted before the tile's barrier (only by
  // threads whose own largest exponent exceeds what they already know of) and read by everyone after it. A slot is
  // posted to again two barriers later, after every thread has read it, and never shrinks. ----
  constexpr int DC = D / 8;                                              // 16-byte chunks per tiled V row
  constexpr int VR = CV ? (BT * DC + 64 * NW - 1) / (64 * NW) : 1;       // chunks per thread and tile
  __shared__ uint32_t v_top[2];
  uint4 vreg[VR];
  int vr_voff[VR], vr_lds[VR];
  uint32_t top_run = 0;    // largest finite |v| bits up to the tile last rewritten (the same in every thread)
  int thr_next = 0, thr_cur = 0, thr_acc = 0;  // exponent base of the tile last rewritten / in use / of the accumulators
  bool v_special = false;  // this thread's registers hold an infinity or a NaN
  const __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t *>(vp), 0, __builtin_amdgcn_readfirstlane((int)((int64_t)n_keys * a.vs[2] * 2)), 0x00020000);
  if constexpr (CV) {
#pragma unroll
    for (int j = 0; j < VR; j++) {
      const int ch = tid + j * (64 * NW);
      const int row = ch / DC, col = ch % DC;
      vr_voff[j] = (ch < BT * DC && col < cpr) ? (int)((row * a.vs[2] + col * 8) * 2) : kOutOfRange;
      vr_lds[j] = (row * LDV + col * 8) * 2;
    }
  }
  auto fetch_v = [&](int kt) {
    const int soff = __builtin_amdgcn_readfirstlane(kt * v_tile_bytes);
#pragma unroll
    for (int j = 0; j < VR; j++) vreg[j] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(v_rsrc, vr_voff[j], soff, 0));
  };
  auto post_top = [&](int slot) {
    u16x2_t all = {0, 0};
#pragma unroll
    for (int j = 0; j < VR; j++) {
      const uint32_t w[4] = {vreg[j].x, vreg[j].y, vreg[j].z, vreg[j].w};
#pragma unroll
      for (int e = 0; e < 4; e++) all = __builtin_elementwise_max(all, __builtin_bit_cast(u16x2_t, w[e] & 0x7fff7fffu));
    }
    uint32_t m = max((uint32_t)all[0], (uint32_t)all[1]);
    v_special = m >= 0x7f80u;
    if (v_special) {
      m = 0;
#pragma unroll
      for (int j = 0; j < VR; j++) {
        m = bf16x2_finite_top(vreg[j].x, m);
        m = bf16x2_finite_top(vreg[j].y, m);
        m = bf16x2_finite_top(vreg[j].z, m);
        m = bf16x2_finite_top(vreg[j].w, m);
      }
    }
    if ((m >> 7) > (top_run >> 7)) atomicMax(&v_top[slot], m);
  };
  auto rewrite_v = [&](int buf) {  // after the barrier that follows post_top(buf)
    top_run = max(top_run, v_top[buf]);
    thr_next = max((int)(top_run >> 7) - 29, 0);
    const uint32_t tb2 = ((uint32_t)thr_next << 7) * 0x00010001u;
    char *dst = reinterpret_cast<char *>(&Vs2[buf][0]);
    uint4 o[VR];
#pragma unroll
    for (int j = 0; j < VR; j++)
      o[j] = make_uint4(bf16x2_to_scaled_f16x2(vreg[j].x, tb2), bf16x2_to_scaled_f16x2(vreg[j].y, tb2),
                        bf16x2_to_scaled_f16x2(vreg[j].z, tb2), bf16x2_to_scaled_f16x2(vreg[j].w, tb2));
    if (v_special) {
#pragma unroll
      for (int j = 0; j < VR; j++)
        o[j] = make_uint4(bf16x2_to_scaled_f16x2_any(vreg[j].x, tb2), bf16x2_to_scaled_f16x2_any(vreg[j].y, tb2),
                          bf16x2_to_scaled_f16x2_any(vreg[j].z, tb2), bf16x2_to_scaled_f16x2_any(vreg[j].w, tb2));
    }
#pragma unroll
    for (int j = 0; j < VR; j++) {
      if ((BT * DC) % (64 * NW) != 0 && tid + j * (64 * NW) >= BT * DC) continue;
      *reinterpret_cast<uint4 *>(dst + vr_lds[j]) = o[j];
    }
  };

  // lane-constant pieces of the LDS addresses
  const int k_frag_off = n * LDK + 8 * g;  // + kb*32*LDK + 16*ks
  // transposing V read: within each 16-lane block, lane i supplies row (i / 4) and 4-column group
  // (i % 4) of a 4-key x 16-column patch and receives the 4 keys of column i.
  const int i16 = lane & 15;
  const int v_frag_off = (4 * g + (i16 >> 2)) * LDV + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
  // + (kb*32 + 16*t [+8]) * LDV + db*32

  if (n_kv_tiles > 0) load_tile(0, 0);
  if constexpr (CV) {
    if (tid < 2) v_top[tid] = 0;
    if (n_kv_tiles > 0) fetch_v(0);
    __syncthreads();
    if (n_kv_tiles > 0) {
      post_top(0);
      __syncthreads();
      rewrite_v(0);
      if (n_kv_tiles > 1) fetch_v(1);
    }
  }
  // (the second K buffer is not written before the loop's first barrier: room for the inv_freq table)
  if (a.q_rope) rotate_q_fragments<MT, D>(qreg, a, b, qi, g, reinterpret_cast<float *>(&Ks2[1][0]));
  // The compiler does not model the asm loads or the asm wait below. Make it wait for Q here;
  // otherwise it puts its own vmcnt(0) in front of the first MFMA inside the loop, after the
  // prefetch of the next tile has been issued.
#pragma unroll
  for (int ks = 0; ks < KS; ks++) asm volatile("" :: "v"(qreg[ks]));

  for (int kt = 0; kt < n_kv_tiles; kt++) {
    // One barrier per tile: tile kt (fetched during the previous iteration) becomes visible, and every
    // wave is done with tile kt-1, whose buffer the fetch of tile kt+1 now overwrites.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's blocks of tile kt are in LDS
    if constexpr (CV)
      if (kt + 1 < n_kv_tiles) post_top((kt + 1) & 1);  // (its registers hold V of tile kt + 1)
    __syncthreads();  // ... and everyone's; tile kt-1 has been consumed, its buffer is free
    if (kt + 1 < n_kv_tiles) load_tile(kt + 1, (kt + 1) & 1);  // in flight while tile kt is computed
    if constexpr (CV) thr_cur = thr_next;
    const uint16_t *Ks = Ks2[kt & 1] + kg * (BW * LDK);
    const uint16_t *Vs = Vs2[kt & 1] + kg * (BW * LDV);

    const int k0 = kt * BT + kg * BW;         // first key of this wave's share of the tile
    // all of it above this wave's diagonal, or past the last key (second half of the last tile)
    if ((CAUSAL && k0 > wave_q_hi) || (KSPLIT > 1 && k0 >= k_end)) {
      if constexpr (CV) {
        rewrite_v((kt + 1) & 1);
        if (kt + 2 < n_kv_tiles) fetch_v(kt + 2);
      }
      continue;
    }

    // ---- S^T = K Q^T for the wave's 32-key blocks, two at a time: their fragments are fetched first, then
    // the two accumulator chains alternate so that neither waits on LDS or on its own previous MFMA ----
    floatx16_t sacc[NKB];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int i = 0; i < 16; i++) sacc[kb][i] = 0.f;
    constexpr int KBG = NKB < 2 ? NKB : 2;  // key blocks whose fragments are fetched together
#pragma unroll
    for (int kb0 = 0; kb0 < NKB; kb0 += KBG) {
      vec8 kf[KBG][KS];
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int kb = 0; kb < KBG; kb++)
          kf[kb][ks] = *reinterpret_cast<const vec8 *>(&Ks[k_frag_off + (kb0 + kb) * 32 * LDK + 16 * ks]);
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int kb = 0; kb < KBG; kb++) {
#ifdef LMH_FOLD_SCALE
          sacc[kb0 + kb] = MT::mfma(kf[kb][ks], qreg[ks], ks == 0 ? neg_mc16 : sacc[kb0 + kb]);
#else
          sacc[kb0 + kb] = MT::mfma(kf[kb][ks], qreg[ks], sacc[kb0 + kb]);
#endif
        }
    }

    // The next V tile is rewritten here, in the shadow of the MFMAs just issued. (After the last tile this rewrites
    // stale registers into the buffer of tile kt - 1, which nobody reads any more.)
    if constexpr (CV) {
      rewrite_v((kt + 1) & 1);
      if (kt + 2 < n_kv_tiles) fetch_v(kt + 2);
    }

    // ---- masking (diagonal tiles and the ragged last tile only) ----
    const bool need_mask = (k0 + BW > n_keys) || (CAUSAL && k0 + BW - 1 > wave_q_lo);
    if (need_mask) {
#pragma unroll
      for (int kb = 0; kb < NKB; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int key = k0 + kb * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          if (key >= n_keys || (CAUSAL && key > qi)) sacc[kb][i] = -INFINITY;
        }
    }

    // ---- online softmax; all statistics are per lane (one query column) ----
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[kb][i]);
    mx = max_over_wave_halves(mx);
#ifdef LMH_FOLD_SCALE
    // the scores are c s - c m already: raise m (and re-base this tile) where a row exceeds it by 2^8, and on the first tile
    if (!have_m || __builtin_amdgcn_ballot_w64(mx > kLazyRescale) != 0) {
      const float d = have_m ? fmaxf(mx, 0.f) : mx;
      const float alpha = have_m ? __builtin_amdgcn_exp2f(-d) : 1.f;
      have_m = true;
      neg_mc -= d;
#pragma unroll
      for (int i = 0; i < 16; i++) neg_mc16[i] = neg_mc;
      l_i *= alpha;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[db][i] *= alpha;
#pragma unroll
      for (int kb = 0; kb < NKB; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[kb][i] -= d;
    }
#else
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
#endif
    const float mc = m_i * c;
    pvec8 pf[NKB][2], pf_lo[NKB][2];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
#ifdef LMH_FOLD_SCALE
          const float p = __builtin_amdgcn_exp2f(sacc[kb][8 * t + e]);
#else
          const float p = __builtin_amdgcn_exp2f(sacc[kb][8 * t + e] * c - mc);
#endif
          pf[kb][t][e] = MT::cvt_p(p);
          if (MT::kSplitP) pf_lo[kb][t][e] = MT::cvt_p(p - (float)pf[kb][t][e]);
        }
        l_i = MT::sum8(pf[kb][t], l_i);
        if (MT::kSplitP) l_i = MT::sum8(pf_lo[kb][t], l_i);
      }

    // ---- O^T += V^T P^T ----
    if constexpr (CV) {
      if (thr_cur != thr_acc) {  // this tile's V is stored against a larger value than the accumulated ones
        const int d = thr_cur - thr_acc;
        const float f = d < 127 ? __uint_as_float((uint32_t)(127 - d) << 23) : 0.f;
        thr_acc = thr_cur;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) oacc[db][i] *= f;
      }
    }
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
      for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const uint16_t *vaddr = &Vs[v_frag_off + (kb * 32 + 16 * t) * LDV + db * 32];
          const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr));
          const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr + 8 * LDV));
          const shortx8_t v8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[db] = MT::mfma_pv(__builtin_bit_cast(vec8, v8), pf[kb][t], oacc[db]);
          if (MT::kSplitP) oacc[db] = MT::mfma_pv(__builtin_bit_cast(vec8, v8), pf_lo[kb][t], oacc[db]);
        }
      }
    }
  }

#ifdef LMH_FOLD_SCALE
  m_i = have_m ? -neg_mc / c : -INFINITY;  // back to the units the merge below works in
#endif
  if constexpr (CV) {  // the accumulators hold O * 2^(112 - thr_acc)
    const float f = __uint_as_float((uint32_t)(thr_acc + 15) << 23);
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] *= f;
  }
  // ---- key groups: fold group 1's (m, l, O) into group 0's; lane for lane the same layout ----
  if (KSPLIT > 1) {
    constexpr int NF = DB * 16 + 2;  // floats per lane
    static_assert(KSPLIT == 1 || RG * NF * 64 * 4 <= (int)sizeof(Ks2), "merge buffer must fit in the K tiles");
    float *xch = reinterpret_cast<float *>(&Ks2[0][0]) + (wave % RG) * (NF * 64) + lane;  // [NF][64 lanes]
    __syncthreads();  // every wave has read its last tile
    if (kg == 1) {
      xch[0] = m_i;
      xch[64] = l_i;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) xch[(2 + db * 16 + i) * 64] = oacc[db][i];
    }
    __syncthreads();
    if (kg == 1) return;
    const float m1 = xch[0], l1 = xch[64];
    const float m_new = fmaxf(m_i, m1);
    // a group that saw no key has m = -inf, l = 0, O = 0
    const float a0 = m_i == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m_i - m_new) * c);
    const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m1 - m_new) * c);
    l_i = l_i * a0 + l1 * a1;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] = oacc[db][i] * a0 + xch[(2 + db * 16 + i) * 64] * a1;
  }

  // ---- epilogue: out[qi][d] = O^T[d][qi] / l ----
  const float l_tot = sum_over_wave_halves(l_i);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (qi < a.Sq) {
    const int64_t off = b * a.os[0] + hq * a.os[1] + (int64_t)qi * a.os[2];
    store_out_rows<MT, DB, false>(oacc, inv, a.out, off, g, a.D, a.out_f32);
  }
}

// One workgroup per CU for non-causal launches with too few query rows to go round: the workgroup owns R
// consecutive 32-row blocks of one (b, hq) and runs R x KG waves — wave (r, kg) takes row block r against the kg-th
// 32 keys of every staged tile of 32 KG keys, with its own running max / sum / output; the KG partial results of a
// row block are folded through LDS at the end. With KG chosen so that R x KG is close to a multiple of four, every
// SIMD of the CU carries the same share of the workgroup's (rows x keys) area, which equal 64-row workgroups dealt
// two or three to a CU do not achieve, and every K/V tile is staged once for all R row blocks.
// Measured against those workgroups (B=4 H=20 Sq=448 D=64 fp16, five row blocks x three key groups): 1500 keys 28.7 ->
// 25.3 us, 3000 keys 51.4 -> 43.7, 750 keys 17.0 -> 16.4, 256 keys 9.2 -> 10.5 (one prologue per CU instead of three
// that overlap). Taller tiles (two blocks per wave and tile) and a third tile buffer were 1 % and 7 % slower.
// `mixed`: with five or seven row blocks no equal number of key groups fills four SIMDs evenly (5 x 3 = 15 waves: 4, 4, 4, 3).
// Then the workgroup runs 16 waves on tiles of 128 keys, some row blocks split between two waves (two 32-key blocks of a
// tile each) and the others between four, so that every SIMD walks R / 4 of a block's keys: 1.25 against 1.33 at R = 5
// (B=4 H=20 Sq=448 Sk=1500 D=64: 23.85 -> 23.55 us; D=96 with 3000 keys 54.9 -> 53.5), 1.75 against 2 at R = 7 (Sq=672:
// 37.4 us on the 64-row workgroups -> 32.7 us here).
constexpr int kWideMaxKeyGroups = 6;  // tiles of up to 192 keys: two buffers of them fit the LDS at D = 96
template <typename MT, int D>
__global__ __launch_bounds__(1024, 4) void prefill_mfma_wide_kernel(PrefillArgs a, int wgs_per_head, int n_bh_groups, int mixed) {
  request_args(a);
  request_arg(wgs_per_head);
  request_arg(n_bh_groups);
  request_arg(mixed);
  using vec8 = typename MT::vec8;
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int LDK = D + kPadK, LDV = D + pad_v<D>();
  constexpr int KG_MAX = kWideMaxKeyGroups, BT_MAX = 32 * KG_MAX;  // keys per staged tile at most
  constexpr int NBUF = 2;  // tile kt + 1 is in flight while tile kt is computed
  constexpr int KC = LDK / 8, VC = LDV / 8;         // 16-byte chunks per LDS row
  constexpr int NW_MIN = 12;                        // the host launches 12 to 16 waves
  constexpr int KJ = (KC * BT_MAX / 64 + NW_MIN - 1) / NW_MIN, VJ = (VC * BT_MAX / 64 + NW_MIN - 1) / NW_MIN;
  constexpr int NF = DB * 16 + 2;                   // floats per lane of a partial result
  constexpr int K_BUF = BT_MAX * LDK, V_BUF = BT_MAX * LDV;  // elements per tile buffer
  constexpr int kWideMaxSlots = 12;  // (KG - 1) x R partial results at most; the host picks KG accordingly
  constexpr int kTileElems = NBUF * (K_BUF + V_BUF), kMergeElems = kWideMaxSlots * NF * 64 * 2;
  __shared__ __attribute__((aligned(16))) uint16_t lds[kTileElems > kMergeElems ? kTileElems : kMergeElems];  // tiles, then partials
  static_assert(sizeof(lds) <= 160 * 1024, "LDS of a CU");

  const int cpr = a.D / 8;
  const int bid = blockIdx.x;
  const int xcd = bid & 7, idx = bid >> 3;
  const int j_wg = idx % wgs_per_head;
  const int bh = (idx / wgs_per_head) * 8 + xcd;
  if (bh >= a.B * a.Hq) return;
  const int b = bh / a.Hq, hq = bh % a.Hq;
  const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
  // row blocks of this workgroup: the head's ceil(Sq / 32) blocks dealt evenly to its workgroups
  const int n_blocks = (a.Sq + 31) / 32;
  const int base = n_blocks / wgs_per_head, extra = n_blocks % wgs_per_head;
  const int R = base + (j_wg < extra ? 1 : 0);
  if (R == 0) return;
  const int block0 = j_wg * base + min(j_wg, extra);
  const int NW = blockDim.x >> 6;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, g = lane >> 5;
  // Which row block r of the workgroup the wave takes, as key group kg of that block's n_groups, and which 32-key blocks of
  // every staged tile: blocks kb0 .. kb0 + nkb - 1. The partial results of groups 1 .. n_groups - 1 go to LDS slots
  // slot0 + (kg - 1) * slot_step; group 0 folds them.
  int BT, r, kg, n_groups, kb0, nkb, slot0, slot_step;
  if (!mixed) {
    // the host launches R_max x KG waves; a workgroup with fewer row blocks may use more key groups or leave waves idle
    const int KG = min(min(NW / R, KG_MAX), kWideMaxSlots / R + 1);
    BT = 32 * KG;
    r = wave % R, kg = wave / R, n_groups = KG;
    kb0 = kg, nkb = 1, slot0 = r, slot_step = R;
  } else {
    // 16 waves on tiles of 128 keys: `heavy` row blocks are split between two waves (two 32-key blocks of a tile each), the
    // others between four (one block each). The heavy waves come first, so that dealt round-robin every SIMD gets the same
    // number of 32-key blocks per tile: R of them (R = 5: 2 + 1 + 1 + 1 against 4 x 1 per 96 keys with three key groups).
    BT = 128;
    const int heavy = max(2 * R - 8, 0), light = R - heavy;
    if (wave < 2 * heavy) {
      r = wave % heavy, kg = wave / heavy, n_groups = 2;
      kb0 = 2 * kg, nkb = 2, slot0 = r, slot_step = 0;
    } else {
      const int l = wave - 2 * heavy;
      r = heavy + l % light, kg = l / light, n_groups = 4;
      kb0 = kg, nkb = 1, slot0 = heavy + 3 * (l % light), slot_step = 1;
    }
  }
  const bool active = kg < n_groups;  // waves beyond the groups only help to stage
  const int qi = (block0 + r) * 32 + n;

  int n_keys = a.kv_len ? a.kv_len[b] : a.Sk;
  n_keys = min(max(n_keys, 0), a.Sk);
  const int n_kv_tiles = (n_keys + BT - 1) / BT;

  const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + b * a.qs[0] + hq * a.qs[1];
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  vec8 qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) {
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (active && qi < a.Sq && 16 * ks + 8 * g < a.D) raw = *reinterpret_cast<const uint4 *>(qp + (int64_t)qi * a.qs[2] + 16 * ks + 8 * g);
    qreg[ks] = __builtin_bit_cast(vec8, raw);
  }
  floatx16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[db][i] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;
  const float c = a.scale * kLog2e;

  // ---- staging, as in the kernel above: LDS-writing buffer loads, one tile ahead, wave w issues 1 KB blocks
  // w, w + NW, ...; the chunk -> (row, column) map does not depend on the tile height, rows past it are not fetched ----
  typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) void lds_void_t;
  const int KI = (KC * BT + 63) / 64, VI = (VC * BT + 63) / 64;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int nw_u = __builtin_amdgcn_readfirstlane(NW);
  auto make_desc = [](const uint16_t *base_ptr, int bytes) {
    const uint64_t pp = (uint64_t)base_ptr;
    i32x4_t d;
    d[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)pp);
    d[1] = __builtin_amdgcn_readfirstlane((int)((pp >> 32) & 0xffff));
    d[2] = __builtin_amdgcn_readfirstlane(bytes);
    d[3] = 0x00020000;
    return d;
  };
  const i32x4_t k_desc = make_desc(kp, (int)((int64_t)n_keys * a.ks[2] * 2));
  const i32x4_t v_desc = make_desc(vp, (int)((int64_t)n_keys * a.vs[2] * 2));
  int k_voff[KJ], v_voff[VJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    const int ch = (wave + NW * j) * 64 + lane;
    const int row = ch / KC, col = ch % KC;
    k_voff[j] = (col < cpr && row < BT) ? (int)((row * a.ks[2] + col * 8) * 2) : kOutOfRange;
  }
#pragma unroll
  for (int j = 0; j < VJ; j++) {
    const int ch = (wave + NW * j) * 64 + lane;
    const int row = ch / VC, col = ch % VC;
    v_voff[j] = (col < cpr && row < BT) ? (int)((row * a.vs[2] + col * 8) * 2) : kOutOfRange;
  }
  const int k_tile_bytes = (int)(BT * a.ks[2] * 2), v_tile_bytes = (int)(BT * a.vs[2] * 2);
  const uint32_t k_lds0 = (uint32_t)(uintptr_t)(lds_void_t *)&lds[0] + wave_u * 1024;
  const uint32_t v_lds0 = (uint32_t)(uintptr_t)(lds_void_t *)&lds[NBUF * K_BUF] + wave_u * 1024;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is a reserved register; it is only written here
  auto load_block = [](i32x4_t desc, uint32_t lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(desc), "s"(soff) : "memory", "m0");
  };
#pragma clang diagnostic pop
  auto load_tile = [&](int kt, int buf) {
#pragma unroll
    for (int j = 0; j < KJ; j++)
      if (wave_u + nw_u * j < KI)
        load_block(k_desc, k_lds0 + buf * (K_BUF * 2) + j * (nw_u * 1024), k_voff[j], kt * k_tile_bytes);
#pragma unroll
    for (int j = 0; j < VJ; j++)
      if (wave_u + nw_u * j < VI)
        load_block(v_desc, v_lds0 + buf * (V_BUF * 2) + j * (nw_u * 1024), v_voff[j], kt * v_tile_bytes);
  };

  const int k_frag_off = (kb0 * 32 + n) * LDK + 8 * g;  // + 32 LDK per further block
  const int i16 = lane & 15;
  const int v_frag_off = (kb0 * 32 + 4 * g + (i16 >> 2)) * LDV + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);

  if (n_kv_tiles > 0) load_tile(0, 0);
  if (a.q_rope) rotate_q_fragments<MT, D>(qreg, a, b, qi, g, reinterpret_cast<float *>(&lds[K_BUF]));
#pragma unroll
  for (int ks = 0; ks < KS; ks++) asm volatile("" :: "v"(qreg[ks]));

  for (int kt = 0; kt < n_kv_tiles; kt++) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's blocks of tile kt are in LDS
    __syncthreads();  // ... and everyone's; tile kt-1 has been consumed, its buffer is free
    if (kt + 1 < n_kv_tiles) load_tile(kt + 1, (kt + 1) & 1);
    for (int j = 0; j < nkb; j++) {
    const int k0 = kt * BT + (kb0 + j) * 32;  // this wave's 32 keys of the tile (nkb = 2: the second 32 follow)
    if (!active || k0 >= n_keys) break;
    const uint16_t *Ks = &lds[(kt & 1) * K_BUF + j * 32 * LDK];
    const uint16_t *Vs = &lds[NBUF * K_BUF + (kt & 1) * V_BUF + j * 32 * LDV];

    floatx16_t sacc;
#pragma unroll
    for (int i = 0; i < 16; i++) sacc[i] = 0.f;
    vec8 kf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kf[ks] = *reinterpret_cast<const vec8 *>(&Ks[k_frag_off + 16 * ks]);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) sacc = MT::mfma(kf[ks], qreg[ks], sacc);
    if (k0 + 32 > n_keys) {
#pragma unroll
      for (int i = 0; i < 16; i++)
        if (k0 + 8 * (i >> 2) + 4 * g + (i & 3) >= n_keys) sacc[i] = -INFINITY;
    }
    float mx = sacc[0];
#pragma unroll
    for (int i = 1; i < 16; i++) mx = fmaxf(mx, sacc[i]);
    mx = max_over_wave_halves(mx);
    if (__builtin_amdgcn_ballot_w64((mx - m_i) * c > kLazyRescale) != 0) {
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
    vec8 pf[2], pf_lo[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float p = __builtin_amdgcn_exp2f(sacc[8 * t + e] * c - mc);
        pf[t][e] = MT::cvt(p);
        if (MT::kSplitP) pf_lo[t][e] = MT::cvt(p - (float)pf[t][e]);
      }
      l_i = MT::sum8(pf[t], l_i);
      if (MT::kSplitP) l_i = MT::sum8(pf_lo[t], l_i);
    }
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const uint16_t *vaddr = &Vs[v_frag_off + 16 * t * LDV + db * 32];
        const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr));
        const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr + 8 * LDV));
        const shortx8_t v8 = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        oacc[db] = MT::mfma(__builtin_bit_cast(vec8, v8), pf[t], oacc[db]);
        if (MT::kSplitP) oacc[db] = MT::mfma(__builtin_bit_cast(vec8, v8), pf_lo[t], oacc[db]);
      }
    }
    }
  }

  // ---- fold the key groups of a row block: groups 1 .. KG-1 leave (m, l, O) in LDS, group 0 takes them in order ----
  float *xch = reinterpret_cast<float *>(&lds[0]) + lane;  // slot s at xch + s * NF * 64, [NF][64 lanes]
  __syncthreads();  // every wave has read its last tile
  if (active && kg > 0) {
    float *slot = xch + (slot0 + (kg - 1) * slot_step) * (NF * 64);
    slot[0] = m_i;
    slot[64] = l_i;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) slot[(2 + db * 16 + i) * 64] = oacc[db][i];
  }
  __syncthreads();
  if (!active || kg > 0) return;
  for (int k2 = 1; k2 < n_groups; k2++) {
    const float *slot = xch + (slot0 + (k2 - 1) * slot_step) * (NF * 64);
    const float m1 = slot[0], l1 = slot[64];
    const float m_new = fmaxf(m_i, m1);
    // a group that saw no key has m = -inf, l = 0, O = 0
    const float a0 = m_i == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m_i - m_new) * c);
    const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m1 - m_new) * c);
    m_i = m_new;
    l_i = l_i * a0 + l1 * a1;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[db][i] = oacc[db][i] * a0 + slot[(2 + db * 16 + i) * 64] * a1;
  }

  const float l_tot = sum_over_wave_halves(l_i);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (qi < a.Sq) {
    const int64_t off = b * a.os[0] + hq * a.os[1] + (int64_t)qi * a.os[2];
    store_out_rows<MT, DB, true>(oacc, inv, a.out, off, g, a.D, a.out_f32);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// Causal launches whose query tiles are few enough to matter one by one: a workgroup of 8 waves owns TWO 256-row query
// tiles of one (b, hq) — tile p and tile n - 1 - p — so that every workgroup of the launch walks the same number of keys
// (the short rows of the early tile plus the long rows of the late one), one workgroup per CU, no second round and no
// tail. Wave w carries rows 32 w .. of the early tile (row block 0) and rows 32 w .. of the late tile (row block 1).
// While the keys are visible to both tiles, every K and V^T fragment the wave reads from LDS feeds two MFMAs, one per
// row block (half the LDS reads per MFMA of the kernel above); past the early tile's diagonal the wave stores that
// tile's rows and goes on with the late tile alone. K/V tiles are staged once for both query tiles.
// Without a mask (CAUSAL = false) the two tiles are neighbours — a 512-row tile — and share every fragment to the end.
// ---------------------------------------------------------------------------------------------------------------
template <typename MT, int D, bool CAUSAL>
__global__ __launch_bounds__(512, 2) void prefill_mfma_pair_kernel(PrefillArgs a, int n_q_tiles, int n_bh_groups) {
  request_args(a);
  request_arg(n_q_tiles);
  request_arg(n_bh_groups);
  using vec8 = typename MT::vec8;
  static_assert(!MT::kSplitP && !MT::kConvertV, "one weight fragment per V fragment, V tiles staged as they are: fp16");
  constexpr int NW = 8, BM = 256;
  constexpr int BT = 2 * BN;        // 128 keys per staged tile
  constexpr int NKB = BT / 32;
  constexpr int KS = D / 16, DB = D / 32;
  const int cpr = a.D / 8;
  constexpr int LDK = D + kPadK, LDV = D + pad_v<D>();

  __shared__ __attribute__((aligned(16))) uint16_t Ks2[2][BT * LDK];
  __shared__ __attribute__((aligned(16))) uint16_t Vs2[2][BT * LDV];

  const int bid = blockIdx.x;
  const int xcd = bid & 7, idx = bid >> 3;
  const int pair = idx / n_bh_groups;
  const int bh = (idx % n_bh_groups) * 8 + xcd;
  if (bh >= a.B * a.Hq) return;
  const int b = bh / a.Hq, hq = bh % a.Hq;
  const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
  // tile p with tile n - 1 - p; with an odd number of tiles the middle one is alone (its workgroup has no early tile)
  // (without a mask: two neighbouring tiles; the second one, row block 0 here, is missing at an odd end)
  const int t_late = CAUSAL ? n_q_tiles - 1 - pair : 2 * pair, t_early = CAUSAL ? pair : 2 * pair + 1;
  const bool has_early = CAUSAL ? t_early < t_late : t_early < n_q_tiles;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, g = lane >> 5;
  // rows of this wave: qlo[rb] .. qlo[rb] + 31; without an early tile row block 0 lies past the last query
  int qlo[2];
  qlo[0] = has_early ? t_early * BM + 32 * wave : a.Sq + 64;
  qlo[1] = t_late * BM + 32 * wave;

  int n_keys = a.kv_len ? a.kv_len[b] : a.Sk;
  n_keys = min(max(n_keys, 0), a.Sk);
  const int k_end_early = !has_early ? 0 : CAUSAL ? min(n_keys, (t_early + 1) * BM) : n_keys;   // keys the early tile can see
  const int k_end_late = CAUSAL ? min(n_keys, (t_late + 1) * BM) : n_keys;
  const int n_tiles_early = (k_end_early + BT - 1) / BT;
  const int n_tiles_late = (k_end_late + BT - 1) / BT;

  const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + b * a.qs[0] + hq * a.qs[1];
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  vec8 qreg[2][KS];
#pragma unroll
  for (int rb = 0; rb < 2; rb++) {
    const int qi = qlo[rb] + n;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      uint4 raw = make_uint4(0, 0, 0, 0);
      if (qi < a.Sq && 16 * ks + 8 * g < a.D) raw = *reinterpret_cast<const uint4 *>(qp + (int64_t)qi * a.qs[2] + 16 * ks + 8 * g);
      qreg[rb][ks] = __builtin_bit_cast(vec8, raw);
    }
  }

  floatx16_t oacc[2][DB];
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[rb][db][i] = 0.f;
  float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.f, 0.f};
  const float c = a.scale * kLog2e;

  // ---- tile staging, as in prefill_mfma_kernel ----
  typedef int32_t i32x4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) void lds_void_t;
  constexpr int KC = LDK / 8, VC = LDV / 8;
  constexpr int KI = KC * BT / 64, VI = VC * BT / 64;
  constexpr int KJ = (KI + NW - 1) / NW, VJ = (VI + NW - 1) / NW;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  __builtin_assume(wave_u >= 0 && wave_u < NW);
  auto make_desc = [](const uint16_t *base, int bytes) {
    const uint64_t p = (uint64_t)base;
    i32x4_t d;
    d[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    d[1] = __builtin_amdgcn_readfirstlane((int)((p >> 32) & 0xffff));
    d[2] = __builtin_amdgcn_readfirstlane(bytes);
    d[3] = 0x00020000;
    return d;
  };
  const i32x4_t k_desc = make_desc(kp, (int)((int64_t)n_keys * a.ks[2] * 2));
  const i32x4_t v_desc = make_desc(vp, (int)((int64_t)n_keys * a.vs[2] * 2));
  int k_voff[KJ], v_voff[VJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    const int ch = (wave + NW * j) * 64 + lane;
    const int row = ch / KC, col = ch % KC;
    k_voff[j] = col < cpr ? (int)((row * a.ks[2] + col * 8) * 2) : kOutOfRange;
  }
#pragma unroll
  for (int j = 0; j < VJ; j++) {
    const int ch = (wave + NW * j) * 64 + lane;
    const int row = ch / VC, col = ch % VC;
    v_voff[j] = col < cpr ? (int)((row * a.vs[2] + col * 8) * 2) : kOutOfRange;
  }
  const int k_tile_bytes = (int)(BT * a.ks[2] * 2), v_tile_bytes = (int)(BT * a.vs[2] * 2);
  const uint32_t k_lds0 = (uint32_t)(uintptr_t)(lds_void_t *)&Ks2[0][0] + wave_u * 1024;
  const uint32_t v_lds0 = (uint32_t)(uintptr_t)(lds_void_t *)&Vs2[0][0] + wave_u * 1024;
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
  auto load_block = [](i32x4_t desc, uint32_t lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(desc), "s"(soff) : "memory", "m0");
  };
#pragma clang diagnostic pop
  auto load_tile = [&](int kt, int buf) {
#pragma unroll
    for (int j = 0; j < KJ; j++)
      if (wave_u + NW * j < KI)
        load_block(k_desc, k_lds0 + buf * (BT * LDK * 2) + j * (NW * 1024), k_voff[j], kt * k_tile_bytes);
#pragma unroll
    for (int j = 0; j < VJ; j++)
      if (wave_u + NW * j < VI)
        load_block(v_desc, v_lds0 + buf * (BT * LDV * 2) + j * (NW * 1024), v_voff[j], kt * v_tile_bytes);
  };

  const int k_frag_off = n * LDK + 8 * g;
  const int i16 = lane & 15;
  const int v_frag_off = (4 * g + (i16 >> 2)) * LDV + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);

  if (n_tiles_late > 0) load_tile(0, 0);
  if (a.q_rope) {
    float *table = reinterpret_cast<float *>(&Ks2[1][0]);
    if ((int)threadIdx.x < D / 2) table[threadIdx.x] = rope_inv_freq(threadIdx.x, D, a.q_log2_base);
    __syncthreads();
#pragma unroll
    for (int rb = 0; rb < 2; rb++) rotate_q_fragments_with_table<MT, D>(qreg[rb], a, b, qlo[rb] + n, g, table);
  }
#pragma unroll
  for (int rb = 0; rb < 2; rb++)
#pragma unroll
    for (int ks = 0; ks < KS; ks++) asm volatile("" :: "v"(qreg[rb][ks]));

  // One 32-key block at key k0 for row blocks RB0 .. 1 (RB0 = 0: both, every fragment read feeds two MFMAs; RB0 = 1: the
  // late tile alone). Online softmax per row block as in prefill_mfma_kernel.
  auto block = [&](auto rb0_c, auto nb_c, const uint16_t *Kb, const uint16_t *Vb, int k0) {
    constexpr int RB0 = decltype(rb0_c)::value;
    constexpr int NB = decltype(nb_c)::value;  // 32-key blocks taken together
    floatx16_t sacc[2][NB];
#pragma unroll
    for (int rb = RB0; rb < 2; rb++)
#pragma unroll
      for (int kb = 0; kb < NB; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[rb][kb][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int kb = 0; kb < NB; kb++) {
        const vec8 kf = *reinterpret_cast<const vec8 *>(&Kb[k_frag_off + kb * 32 * LDK + 16 * ks]);
#pragma unroll
        for (int rb = RB0; rb < 2; rb++) sacc[rb][kb] = MT::mfma(kf, qreg[rb][ks], sacc[rb][kb]);
      }
    vec8 pf[2][NB][2];
#pragma unroll
    for (int rb = RB0; rb < 2; rb++) {
      if (k0 + 32 * NB > n_keys || (CAUSAL && k0 + 32 * NB - 1 > qlo[rb])) {  // the ragged last block, or a block on this row block's diagonal
        const int qi = qlo[rb] + n;
#pragma unroll
        for (int kb = 0; kb < NB; kb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int key = k0 + 32 * kb + 8 * (i >> 2) + 4 * g + (i & 3);
            if (key >= n_keys || (CAUSAL && key > qi)) sacc[rb][kb][i] = -INFINITY;
          }
      }
      float mx = sacc[rb][0][0];
#pragma unroll
      for (int kb = 0; kb < NB; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[rb][kb][i]);
      mx = max_over_wave_halves(mx);
      // (key 0 is visible to every query, so m is finite after the first block)
      if (__builtin_amdgcn_ballot_w64((mx - m_i[rb]) * c > kLazyRescale) != 0) {
        const float m_new = fmaxf(m_i[rb], mx);
        const float alpha = __builtin_amdgcn_exp2f((m_i[rb] - m_new) * c);
        m_i[rb] = m_new;
        l_i[rb] *= alpha;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
          for (int i = 0; i < 16; i++) oacc[rb][db][i] *= alpha;
      }
      const float mc = m_i[rb] * c;
#pragma unroll
      for (int kb = 0; kb < NB; kb++)
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float p = __builtin_amdgcn_exp2f(sacc[rb][kb][8 * t + e] * c - mc);
            pf[rb][kb][t][e] = MT::cvt(p);
          }
          l_i[rb] = MT::sum8(pf[rb][kb][t], l_i[rb]);
        }
    }
#pragma unroll
    for (int kb = 0; kb < NB; kb++)
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const uint16_t *vaddr = &Vb[v_frag_off + (32 * kb + 16 * t) * LDV + db * 32];
          const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr));
          const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr + 8 * LDV));
          const vec8 v8 = __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
          for (int rb = RB0; rb < 2; rb++) {
            oacc[rb][db] = MT::mfma(v8, pf[rb][kb][t], oacc[rb][db]);
          }
        }
  };
  auto store_rows = [&](int rb) {
    const int qi = qlo[rb] + n;
    const float l_tot = sum_over_wave_halves(l_i[rb]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (qi < a.Sq)
      store_out_rows<MT, DB, false>(oacc[rb], inv, a.out, b * a.os[0] + hq * a.os[1] + (int64_t)qi * a.os[2], g, a.D, a.out_f32);
  };
  // A whole 128-key tile for the late row block alone: the loop body of prefill_mfma_kernel (four 32-key blocks at a
  // time, their QK^T chains alternating two by two, one softmax pass over all 64 scores of a lane).
  auto tile_late = [&](const uint16_t *Ks, const uint16_t *Vs, int k0) {
    constexpr int rb = 1;
    if (CAUSAL && k0 > qlo[rb] + 31) return;  // the whole tile lies above this wave's rows
    floatx16_t sacc[NKB];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int i = 0; i < 16; i++) sacc[kb][i] = 0.f;
#pragma unroll
    for (int kb0 = 0; kb0 < NKB; kb0 += 2) {
      vec8 kf[2][KS];
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
          kf[kb][ks] = *reinterpret_cast<const vec8 *>(&Ks[k_frag_off + (kb0 + kb) * 32 * LDK + 16 * ks]);
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int kb = 0; kb < 2; kb++) sacc[kb0 + kb] = MT::mfma(kf[kb][ks], qreg[rb][ks], sacc[kb0 + kb]);
    }
    if (k0 + BT > n_keys || (CAUSAL && k0 + BT - 1 > qlo[rb])) {
      const int qi = qlo[rb] + n;
#pragma unroll
      for (int kb = 0; kb < NKB; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int key = k0 + kb * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          if (key >= n_keys || (CAUSAL && key > qi)) sacc[kb][i] = -INFINITY;
        }
    }
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[kb][i]);
    mx = max_over_wave_halves(mx);
    if (__builtin_amdgcn_ballot_w64((mx - m_i[rb]) * c > kLazyRescale) != 0) {
      const float m_new = fmaxf(m_i[rb], mx);
      const float alpha = __builtin_amdgcn_exp2f((m_i[rb] - m_new) * c);
      m_i[rb] = m_new;
      l_i[rb] *= alpha;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[rb][db][i] *= alpha;
    }
    const float mc = m_i[rb] * c;
    vec8 pf[NKB][2];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float p = __builtin_amdgcn_exp2f(sacc[kb][8 * t + e] * c - mc);
          pf[kb][t][e] = MT::cvt(p);
        }
        l_i[rb] = MT::sum8(pf[kb][t], l_i[rb]);
      }
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const uint16_t *vaddr = &Vs[v_frag_off + (kb * 32 + 16 * t) * LDV + db * 32];
          const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr));
          const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr + 8 * LDV));
          const vec8 v8 = __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          oacc[rb][db] = MT::mfma(v8, pf[kb][t], oacc[rb][db]);
        }
  };
  const std::integral_constant<int, 0> kBoth{};
  const std::integral_constant<int, 1> kLate{};

  // ---- keys the early tile sees: both row blocks ----
  for (int kt = 0; kt < n_tiles_early; kt++) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kt + 1 < n_tiles_late) load_tile(kt + 1, (kt + 1) & 1);
    const uint16_t *Ks = Ks2[kt & 1];
    const uint16_t *Vs = Vs2[kt & 1];
    constexpr int NB = 2;  // two 32-key blocks of both row blocks at a time: four score blocks in flight (fp16, D = 96: 244 registers)
    const std::integral_constant<int, NB> kNB{};
    const std::integral_constant<int, 1> kOne{};
#pragma unroll
    for (int kb = 0; kb < NKB; kb += NB) {
      const int k0 = kt * BT + kb * 32;
      if (k0 >= k_end_late) break;
      if (CAUSAL ? (k0 + 32 * NB - 1 <= qlo[0] && k0 + 32 * NB <= k_end_early) : true) {   // the whole group below the early rows' diagonal
        block(kBoth, kNB, Ks + kb * 32 * LDK, Vs + kb * 32 * LDV, k0);
      } else {
#pragma unroll
        for (int j = 0; j < NB; j++) {
          const int kj = k0 + 32 * j;
          if (kj >= k_end_late) break;
          if (kj <= qlo[0] + 31 && kj < k_end_early)
            block(kBoth, kOne, Ks + (kb + j) * 32 * LDK, Vs + (kb + j) * 32 * LDV, kj);
          else
            block(kLate, kOne, Ks + (kb + j) * 32 * LDK, Vs + (kb + j) * 32 * LDV, kj);
        }
      }
    }
  }
  if (has_early) store_rows(0);
  // ---- the rest: the late tile alone ----
  for (int kt = n_tiles_early; kt < n_tiles_late; kt++) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kt + 1 < n_tiles_late) load_tile(kt + 1, (kt + 1) & 1);
    const uint16_t *Ks = Ks2[kt & 1];
    const uint16_t *Vs = Vs2[kt & 1];
    if (CAUSAL && kt * BT + BT - 1 > qlo[1]) {
      // a tile on the late rows' diagonal: block by block, so that blocks above the wave's rows are skipped (four at a
      // time they would be computed and masked: 109.9 -> 108.7 us on B=1 H=32 S=4096 D=96)
#pragma unroll
      for (int kb = 0; kb < NKB; kb++) {
        const int k0 = kt * BT + kb * 32;
        if (k0 > qlo[1] + 31 || k0 >= k_end_late) break;
        block(kLate, std::integral_constant<int, 1>{}, Ks + kb * 32 * LDK, Vs + kb * 32 * LDV, k0);
      }
    } else {
      tile_late(Ks, Vs, kt * BT);
    }
  }
  store_rows(1);
}

template <typename MT, int D>
int launch_pair(const PrefillArgs &a, hipStream_t stream) {
  const int n_q_tiles = (a.Sq + 255) / 256;
  const int n_pairs = (n_q_tiles + 1) / 2;
  const int n_bh_groups = (a.B * a.Hq + 7) / 8;
  dim3 grid(8 * n_bh_groups * n_pairs), block(512);
  if (plan_only("prefill_mfma_pair_kernel<%s, D=%d, %s> query tiles=%d, workgroups=%u", MT::kName, D, a.causal ? "causal" : "full", n_q_tiles, grid.x)) return LMH_OK;
  if (a.causal)
    hipLaunchKernelGGL((prefill_mfma_pair_kernel<MT, D, true>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  else
    hipLaunchKernelGGL((prefill_mfma_pair_kernel<MT, D, false>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

// The policy prefill_mfma_kernel runs a tensor type with. bf16 with V16: V rewritten as fp16 in the workgroups that own
// their query rows alone (B=1 H=32 S=4096 causal D=96 151 -> 122 us, D=128 202 -> 174, D=64 x 4 batches 443 -> 350; without
// a mask -15 ... -24 %); the small launches whose wave pairs split the keys keep head + remainder weights and LDS-direct V
// tiles (the rewrite sits on their critical path: 8 heads x 1024 rows 14.8 -> 20.6 us, 64 heads x 1024 rows 31.3 -> 35.6).
template <typename MT, bool V16, int KSPLIT> struct base_policy { using type = MT; };
template <> struct base_policy<MfmaBF16, true, 1> { using type = MfmaBF16V16; };

template <typename MT0, bool V16, int D, int KSPLIT, int NW, int WPS = default_wps<D, NW>()>
int launch_split(const PrefillArgs &a, hipStream_t stream) {
  using MT = typename base_policy<MT0, V16, KSPLIT>::type;
  constexpr int BM = 32 * NW / KSPLIT;
  const int n_q_tiles = (a.Sq + BM - 1) / BM;
  const int n_bh_groups = (a.B * a.Hq + 7) / 8;
  dim3 grid(8 * n_bh_groups * n_q_tiles), block(64 * NW);
  if (plan_only("prefill_mfma_kernel<%s, D=%d, %s, key groups=%d, waves=%d, waves per SIMD=%d> workgroups=%u%s", MT::kName, D,
                a.causal ? "causal" : "full", KSPLIT, NW, WPS, grid.x, MT::kConvertV ? ", V as fp16" : ""))
    return LMH_OK;
  if (a.causal)
    hipLaunchKernelGGL((prefill_mfma_kernel<MT, D, true, KSPLIT, NW, WPS>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  else
    hipLaunchKernelGGL((prefill_mfma_kernel<MT, D, false, KSPLIT, NW, WPS>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

// Plan for the wide kernel: workgroups per head, waves per workgroup. Returns false where it does not apply or the
// equal 64-row workgroups are expected to do as well. `load` = the share of a 32-row block's keys that the busiest SIMD
// of the busiest CU walks, the quantity the launch time follows when the chip is not full. Measured (fp16, 1500 keys,
// wide against 64-row workgroups): load 1.33 vs 1.5 -12 % (D = 64), -14 % (D = 96); 0.75 vs 1.0 -7 ... -12 %; equal loads
// +-2 %, and +7 % at 1024 keys; under about 500 keys the single prologue per CU costs more than the balance wins.
inline bool wide_plan(const PrefillArgs &a, int n_cus, int *wgs_per_head, int *n_waves, int *mixed) {
  const int heads = a.B * a.Hq, heads8 = (heads + 7) / 8 * 8;
  const int n_blocks = (a.Sq + 31) / 32;
  if (a.causal || heads8 > n_cus || n_blocks < 2 || a.Sk < 640) return false;
  const int w = max(1, min(n_cus / heads8, n_blocks / 2));
  const int r_max = (n_blocks + w - 1) / w;
  if (r_max > 8) return false;
  int best_kg = 0;
  double best = 1e30;
  for (int kg = 2; kg <= kWideMaxKeyGroups; kg++) {
    if (r_max * kg < 12 || r_max * kg > 16 || (kg - 1) * r_max > 12) continue;  // 12 to 16 waves, 12 partial results
    const double load = (double)((r_max * kg + 3) / 4) / kg;
    if (load <= best) best = load, best_kg = kg;  // on a tie, more waves
  }
  // two waves for some row blocks and four for the others (16 waves, tiles of 128 keys): every SIMD walks r_max / 4 of a
  // block's keys. Ahead of the equal key groups at five and seven row blocks (1.25 against 1.33, 1.75 against 2).
  *mixed = 0;
#ifndef LMH_NO_MIXED_KEY_GROUPS  // (a measurement build can keep equal key groups everywhere, for comparisons)
  if (r_max >= 5 && r_max <= 8 && r_max / 4.0 < best - 1e-9) best = r_max / 4.0, *mixed = 1;
#endif
  if (!best_kg && !*mixed) return false;
  // the equal 64-row workgroups, wave pairs splitting the keys: up to three resident on a CU, half a block's keys a wave
  const int64_t n64 = (int64_t)heads8 * ((a.Sq + 63) / 64);
  const double load_now = 0.5 * (double)((n64 + n_cus - 1) / n_cus);
  if (best > LMH_WIDE_MARGIN * load_now) return false;
  *wgs_per_head = w;
  *n_waves = *mixed ? 16 : r_max * best_kg;
  return true;
}

template <typename MT, int D>
int launch_wide(const PrefillArgs &a, int wgs_per_head, int n_waves, int mixed, hipStream_t stream) {
  const int n_bh_groups = (a.B * a.Hq + 7) / 8;
  dim3 grid(8 * n_bh_groups * wgs_per_head), block(64 * n_waves);
  if (plan_only("prefill_mfma_wide_kernel<%s, D=%d> workgroups per head=%d, waves=%d, workgroups=%u%s", MT::kName, D, wgs_per_head,
                n_waves, grid.x, mixed ? ", two and four key groups" : ""))
    return LMH_OK;
  hipLaunchKernelGGL((prefill_mfma_wide_kernel<MT, D>), grid, block, 0, stream, a, wgs_per_head, n_bh_groups, mixed);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

// V16 (bf16 only): the launches of one key group hand V to the matrix cores as fp16 (base_policy above).
template <typename MT, int D, bool V16>
int launch_for_d(const PrefillArgs &a, hipStream_t stream) {
  static_assert(!V16 || MT::kSplitP, "V16 is a form of the bf16 kernels");
  // With fewer than two 128-row workgroups per CU the launch is bound by how long one workgroup
  // takes to walk its keys, not by the matrix pipes: split the keys of a tile between wave pairs.
  // Measured on 256 CUs: at exactly two per CU the split still wins for causal launches (41.8 vs
  // 46.7 us at B=1 H=32 S=2048 D=96) and loses for non-causal ones (79.8 vs 66.6 us); at three per
  // CU it loses for both.
  const int n_cus = device_cu_count();
  // Causal launches that are exactly one round of paired 256-row tiles (tile p with tile n - 1 - p: equal work in every
  // workgroup, one per CU): the Phi-3 prompt, 32 heads x 16 tiles = 256 pairs. Measured against the kernels below on
  // 256 CUs, fp16: B=1 H=32 S=4096 D=96 -3.2 %, D=64 -6 %, D=80 -3 %; B=2 H=32 S=2048 -5 %; H=8 S=16384 -4.6 %;
  // S=3900 -2 %. With the chip not exactly full it loses (1.25 rounds +23 %, 1.5 rounds +10 %, half a round +30 %),
  // at exactly two rounds it ties (-1.4 ... +7 %).
  // bf16 stays on the kernels below: the fp16 rewrite of V that prefill_mfma_kernel does gains more than the pairing did
  // with bf16 weights as head + remainder (B=1 H=32 S=4096 D=64 causal: 117.7 us here, 99.8 us there), and two row blocks
  // plus the rewrite's registers do not fit; this kernel is built for fp16 only.
#ifndef LMH_NO_PAIR_KERNEL  // (measurement builds can keep these launches on the kernels below, for comparisons with them)
  if constexpr (D <= 96 && !MT::kSplitP) {
    const int64_t wgs_pair = (int64_t)((a.B * a.Hq + 7) / 8) * 8 * (((a.Sq + 255) / 256 + 1) / 2);
    if (a.causal && a.Sq > 256 && wgs_pair <= n_cus && 16 * wgs_pair >= 15 * n_cus) return launch_pair<MT, D>(a, stream);
    // Without a mask the same kernel takes two neighbouring tiles (512 rows, every fragment read shared all the way);
    // its workgroups are equal, so it wants whole rounds: B=1 H=32 S=4096 D=96 (one round) -5.9 %, S=8192 (two) -3.5 %,
    // B=4 (four) -1.1 %; D=64 one round -2.4 %, two rounds +2.5 %; 1.25 rounds +20 %.
    if (!a.causal && a.Sq > 256 && wgs_pair >= n_cus) {
      const int64_t rounds = (wgs_pair + n_cus - 1) / n_cus, last = wgs_pair - (rounds - 1) * n_cus;
      if (16 * last >= 15 * n_cus && (rounds == 1 || (D > 64 && rounds <= 2))) return launch_pair<MT, D>(a, stream);
    }
  }
#endif
  const int64_t wgs = (int64_t)((a.B * a.Hq + 7) / 8) * 8 * ((a.Sq + 127) / 128);
  const int64_t limit = a.causal ? 2 * n_cus : 2 * n_cus - 1;
  if (wgs <= limit && a.Sk >= 4 * BN) {
    if constexpr (D <= 96) {
      int wgs_per_head, n_waves, mixed;
      if (wide_plan(a, n_cus, &wgs_per_head, &n_waves, &mixed)) return launch_wide<MT, D>(a, wgs_per_head, n_waves, mixed, stream);
    }
    return launch_split<MT, V16, D, 2, 4>(a, stream);
  }
  // Large launches: 256-row workgroups of eight waves. Measured against the 128-row ones at D = 96, fp16:
  // non-causal 512 / 768 / 1024 / 1536 / 2048 workgroups +3 / +2 / +2 / +6 / +5 %, causal 512 -7 %
  // (too few to balance their unequal lengths), 1024 +3 %, 1536 +4..7 %, 2048 +5 %.
  // D = 128 does not fit the 128 registers that four waves per SIMD leave: one 256-row workgroup per CU there,
  // which turns over in rounds and balances earlier. fp16: non-causal 256 / 512 / 2048 workgroups +5 / +3 / +6 %,
  // causal 256 / 384 -8 / -5 %, 512 / 1024 / 2048 +8 / +3 / +4 %; bf16 (V rewritten as fp16) 512 workgroups causal
  // +8 %, without a mask +5 %, 2048 causal +5 %.
  const int64_t wgs256 = (int64_t)((a.B * a.Hq + 7) / 8) * 8 * ((a.Sq + 255) / 256);
  if (a.Sq <= 128) return launch_split<MT, V16, D, 1, 4>(a, stream);  // nothing for waves 4-7 to own
  if constexpr (D <= 96) {
    // Causal launches of 1.5 to 3 rounds of one 256-row workgroup per CU (the Phi-3 prompt, 32 heads x 4096 rows,
    // is exactly two): the workgroups turn over heaviest first, so every CU ends up with about the same number
    // of key tiles; K/V tiles are staged once per 256 rows, and with the CU to itself the workgroup stages 128
    // keys at a time. Against the 128-row workgroups at D = 96: 1.5 rounds +2 %, 2 rounds +6 % (120.4 -> 112 us;
    // bf16 164 -> 153 us), 2.25 / 2.5 rounds +1 %, 3 and 3.5 rounds +-0; one round -20 %; D = 64 (2 rounds) -5 %.
    // Non-causal workgroups are all equally long and a part-filled round is lost time: from two rounds on only
    // (2 rounds +1 %, bf16 +4 %; 2.5 rounds +3 %; 1.5 rounds -11 %).
    // bf16 (V rewritten as fp16 through registers) spills at four waves per SIMD and stays on this form however many
    // rounds there are: B=4 H=32 S=4096 causal 583 -> 507 us, without a mask 946 -> 892 us. At D = 64 it takes this form for
    // causal launches of 1.5 to 3 rounds (the rewrite is shared by eight waves instead of four: B=1 H=32 S=4096 100.1 -> 96.5
    // us, H=64 S=2048 60.3 -> 58.6); from three rounds on and without a mask two workgroups per CU are 6-10 % ahead there.
    if constexpr (D == 96 || V16)
      if ((D == 96 || a.causal) && ((D == 96 && V16) || wgs256 < 3 * n_cus) &&
          (a.causal ? 2 * wgs256 >= 3 * n_cus : wgs256 >= 2 * n_cus))
        return launch_split<MT, V16, D, 1, 8, 2>(a, stream);
    if constexpr (!(D == 96 && V16))  // (with V16, D = 96 never gets here with that many workgroups)
      if (wgs256 >= (a.causal ? 4 * n_cus : 2 * n_cus)) return launch_split<MT, V16, D, 1, 8>(a, stream);
  } else if constexpr (!MT::kSplitP || V16) {  // (bf16 with head + remainder weights: 0 / -2 %, stays on 128 rows)
    if (wgs256 >= (a.causal ? 2 * n_cus : n_cus)) return launch_split<MT, V16, D, 1, 8>(a, stream);
  }
  return launch_split<MT, V16, D, 1, 4>(a, stream);
}

template <typename MT>
int launch_for_type(const PrefillArgs &a, hipStream_t stream) {
  if (a.D > 128) return fail(LMH_E_UNSUPPORTED, "MFMA flash attention: head dim %d not tiled", a.D);
#ifndef LMH_BF16_SPLIT_P
  if constexpr (MT::kSplitP) {
    // bf16: V as fp16 pays from about 512 keys per query row on. Its prologue (the first V tile through registers before
    // the first barrier) and one workgroup per CU cost short rows more than the second MFMA per fragment does: 512 heads,
    // fp16 rewrite against head + remainder, causal S=128 +15 ... +35 %, S=256 +7 ... +44 %, S=512 -3 ... +18 %, S=1024
    // -13 ... 0 %; without a mask S=128 0 ... +30 %, S=256 -7 ... -1 %, S=512 -13 ... +5 %, S=1024 -5 ... -19 %. (The
    // D = 96 tiling, one workgroup per CU in this form, is the one that ties or loses at 512 keys per row: 1024 there.)
    const int64_t keys_per_row = a.causal ? (a.Sq < a.Sk ? a.Sq : a.Sk) / 2 : a.Sk;
    if (keys_per_row >= (a.D > 64 && a.D <= 96 ? 1024 : 512)) {
      if (a.D <= 64) return launch_for_d<MT, 64, true>(a, stream);
      if (a.D <= 96) return launch_for_d<MT, 96, true>(a, stream);
      return launch_for_d<MT, 128, true>(a, stream);
    }
  }
#endif
  // the smallest tiling that holds the head dim; the padding costs its share of the MFMAs
  if (a.D <= 64) return launch_for_d<MT, 64, false>(a, stream);
  if (a.D <= 96) return launch_for_d<MT, 96, false>(a, stream);
  return launch_for_d<MT, 128, false>(a, stream);
}

}  // namespace

bool prefill_mfma_supported(int dtype, int D) {
  return (dtype == LMH_F16 || dtype == LMH_BF16) && D >= 8 && D <= 128 && D % 8 == 0;
}

int launch_prefill_mfma(const PrefillArgs &a, int dtype, hipStream_t stream) {
#ifdef LMH_W64_KERNEL
  if (prefill_w64_takes(a, dtype)) return launch_prefill_w64(a, stream);
#endif
  if (dtype == LMH_F16) return launch_for_type<MfmaF16>(a, stream);
  if (dtype == LMH_BF16) return launch_for_type<MfmaBF16>(a, stream);
  return fail(LMH_E_UNSUPPORTED, "MFMA flash attention: dtype %d has no matrix-core path", dtype);
}

}  // namespace lmh
