// Measurement kernel, compiled only into measurement builds of the library (-DLMH_W64_KERNEL, which needs
// -DLMH_MEASUREMENT_BUILD): flash attention forward with 64 query columns per wave and a hand-arranged software pipeline.
// It exists to answer one question with counters: what does the launch time do when the vector and LDS instruction
// counts per MFMA of prefill_mfma_kernel are cut (each K / V^T fragment read feeds two MFMAs; no row max in the common
// path; row sums on the dot-product instruction)? It takes only what that question needs: fp16, head dim 96, no mask,
// no kv_len, no rotary embedding, Sq a multiple of 256 and Sk a multiple of 128; everything else stays with the
// shipped kernels.
#include <type_traits>

#include "prefill_mfma.hpp"

#if !defined(LMH_W64_KERNEL) || !defined(LMH_MEASUREMENT_BUILD)
#error "prefill_mfma_w64.hip belongs to measurement builds only (-DLMH_W64_KERNEL -DLMH_MEASUREMENT_BUILD)"
#endif

namespace lmh {
namespace {

// the PV MFMA with its accumulator pinned to the accumulation registers (AGPRs), so that O does not compete with the
// scores, weights and fragments for vector registers
__device__ inline void mfma_acc(MfmaF16, half8_t a, half8_t b, floatx16_t &c) {
  asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// ---------------------------------------------------------------------------------------------------------------
// 64 query columns per wave: a workgroup of 4 waves owns 256 query rows of one (b, hq), one wave per SIMD; a wave
// carries two 32-row blocks (block w and block 7 - w of the tile, so that every wave has the same work on the causal
// diagonal) and every K / V^T fragment it reads from LDS feeds two MFMAs, one per half. With a single wave on a SIMD
// the matrix and the vector work can only overlap inside that wave, so the loop is software-pipelined over 32-key
// blocks: in one step the wave issues S^T(i+1) = K Q^T (12 MFMAs), the softmax of block i (vector ALU) and
// O^T += V^T P^T of block i-1 (12 MFMAs), three independent instruction streams. S and P alternate between two
// register sets; K/V tiles of 128 keys rotate through three LDS buffers (the last stage still reads tile kt-1 while
// tile kt+1 is being fetched), one barrier per tile.
template <typename MT, int D>
__global__ __launch_bounds__(256, 1) void prefill_mfma_w64_kernel(PrefillArgs a, int n_q_tiles, int n_bh_groups) {
  using vec8 = typename MT::vec8;
  constexpr int BM = 256, BT = 128, NW = 4, NBUF = 3;
  constexpr int KS = D / 16, DB = D / 32;
  constexpr int LDK = D + kPadK, LDV = D + pad_v<D>();
  // elements per tile buffer, rounded up to the 1 KB blocks the waves fetch (4 per round): the loads of the last round
  // that fall beyond the tile land in the slack
  constexpr int K_BUF = (BT * LDK + 2047) / 2048 * 2048, V_BUF = (BT * LDV + 2047) / 2048 * 2048;
  __shared__ __attribute__((aligned(16))) uint16_t lds[NBUF * (K_BUF + V_BUF)];
  static_assert(sizeof(lds) <= 160 * 1024, "LDS of a CU");

  const int bid = blockIdx.x;
  const int xcd = bid & 7, idx = bid >> 3;
  const int tile_rank = idx / n_bh_groups;
  const int bh = (idx % n_bh_groups) * 8 + xcd;
  if (bh >= a.B * a.Hq) return;
  const int b = bh / a.Hq, hq = bh % a.Hq;
  const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
  const int q_tile = tile_rank;
  const int q0 = q_tile * BM;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n = lane & 31, g = lane >> 5;
  int qi[2];
  qi[0] = q0 + 32 * wave + n;
  qi[1] = q0 + 32 * (7 - wave) + n;

  const int n_keys = a.Sk;
  const int n_kv_tiles = n_keys / BT;

  const uint16_t *qp = reinterpret_cast<const uint16_t *>(a.q) + b * a.qs[0] + hq * a.qs[1];
  const uint16_t *kp = reinterpret_cast<const uint16_t *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const uint16_t *vp = reinterpret_cast<const uint16_t *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  const int cpr = a.D / 8;
  vec8 qreg[2][KS];
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      uint4 raw = make_uint4(0, 0, 0, 0);
      if (qi[h] < a.Sq && 16 * ks + 8 * g < a.D) raw = *reinterpret_cast<const uint4 *>(qp + (int64_t)qi[h] * a.qs[2] + 16 * ks + 8 * g);
      qreg[h][ks] = __builtin_bit_cast(vec8, raw);
    }

  floatx16_t oacc[2][DB];
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[h][db][i] = 0.f;
  // The running max starts at a finite value far below any score, not at -inf: a block of all -inf scores (the
  // pipeline's fill, a fully masked block) then gives exp2(-inf) = 0 instead of exp2(-inf + inf) = NaN.
  float m_i[2] = {-1e30f, -1e30f};
  float l_i[2] = {0.f, 0.f};
  const float c = a.scale * kLog2e;

  // ---- staging: LDS-writing buffer loads as in the kernel above, wave w issues 1 KB blocks w, w + 4, ... ----
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
#pragma clang diagnostic ignored "-Winline-asm"
  auto load_block = [](i32x4_t desc, uint32_t lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_addr), "v"(voff), "s"(desc), "s"(soff) : "memory", "m0");
  };
#pragma clang diagnostic pop
  static_assert(KJ * NW * 512 <= K_BUF && VJ * NW * 512 <= V_BUF, "every round of loads lands inside the buffer");
  // piece p of a tile: one 1 KB block per wave (K rounds first, then V rounds); no conditions, so that the pieces can
  // be dropped one by one into the compute groups (a block beyond the tile fetches out of range into the slack)
  constexpr int NPIECE = KJ + VJ;
  uint32_t ld_k_lds = 0, ld_v_lds = 0;
  int ld_k_soff = 0, ld_v_soff = 0;
  auto load_target = [&](int kt, int buf) {
    ld_k_lds = k_lds0 + buf * (K_BUF * 2);
    ld_v_lds = v_lds0 + buf * (V_BUF * 2);
    ld_k_soff = kt * k_tile_bytes;
    ld_v_soff = kt * v_tile_bytes;
  };
  auto load_piece = [&](int p) {
    if (p < KJ) load_block(k_desc, ld_k_lds + p * (NW * 1024), k_voff[p], ld_k_soff);
    else if (p < NPIECE) load_block(v_desc, ld_v_lds + (p - KJ) * (NW * 1024), v_voff[p - KJ], ld_v_soff);
  };
  auto load_tile = [&](int kt, int buf) {
    load_target(kt, buf);
#pragma unroll
    for (int p = 0; p < NPIECE; p++) load_piece(p);
  };

  const int k_frag_off = n * LDK + 8 * g;
  const int i16 = lane & 15;
  const int v_frag_off = (4 * g + (i16 >> 2)) * LDV + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);

  // ---- one pipeline step: QK of block i+1 (at Kb), softmax of block i (S -> Pn), PV of block i-1 (at Vb, weights Pp) ----
  // O lives in the accumulation registers (the PV MFMAs are written as asm with an "a" constraint), so the vector
  // registers hold Q, two sets of scores, two sets of weights and the fragments in flight. The compiler does not know
  // that these asm statements are MFMAs: before any other instruction reads O, settle() waits for the last of them.
  auto settle = [&]() {
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7"
                 : "+a"(oacc[0][0]), "+a"(oacc[0][1]), "+a"(oacc[0][DB - 1]), "+a"(oacc[1][0]), "+a"(oacc[1][1]), "+a"(oacc[1][DB - 1]));
  };
  auto k_frag = [&](const uint16_t *Kb, int ks) {
    return *reinterpret_cast<const vec8 *>(&Kb[k_frag_off + 16 * ks]);
  };
  auto v_frag = [&](const uint16_t *Vb, int f) {
    const int t = f / DB, db = f % DB;
    const uint16_t *vaddr = &Vb[v_frag_off + 16 * t * LDV + db * 32];
    const shortx4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr));
    const shortx4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t *)(vaddr + 8 * LDV));
    return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  auto pv = [&](const uint16_t *Vb, int f, vec8 (&P)[2][2]) {
    const vec8 v8 = v_frag(Vb, f);
#pragma unroll
    for (int h = 0; h < 2; h++) mfma_acc(MT{}, v8, P[h][f / DB], oacc[h][f % DB]);
  };
  // weights of elements [e0, e1) (an even range) of half h: P = exp2(c s - c m) rounded to the element type, and
  // their sum (in fp32, before rounding) added to sg[h]
  auto weights = [&](int h, int e0, int e1, floatx16_t (&S)[2], vec8 (&Pn)[2][2], const float (&mc)[2], float (&sg)[2][2]) {
#ifndef LMH_W64_SUM_F32
#pragma unroll
    for (int e = e0; e < e1; e += 2) {
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      const h2 one = {(_Float16)1.f, (_Float16)1.f};
      h2 pp;
      pp[0] = (_Float16)__builtin_amdgcn_exp2f(S[h][e] * c - mc[h]);
      pp[1] = (_Float16)__builtin_amdgcn_exp2f(S[h][e + 1] * c - mc[h]);
      Pn[h][e >> 3][e & 7] = pp[0];
      Pn[h][e >> 3][(e & 7) + 1] = pp[1];
      sg[h][0] = __builtin_amdgcn_fdot2(pp, one, sg[h][0], false);
    }
#else
#pragma unroll
    for (int e = e0; e < e1; e++) {
      const float pe = __builtin_amdgcn_exp2f(S[h][e] * c - mc[h]);
      Pn[h][e >> 3][e & 7] = MT::cvt(pe);
      sg[h][e & 1] += pe;
    }
#endif
  };
  constexpr int NF = 2 * DB;  // V^T fragments of a block
  static_assert(KS == NF, "the step below pairs K and V^T fragments one to one");
  // The weights of a block are computed against the running max as it stands, without looking at the block's own max
  // first: if the sum of a lane's 16 weights stays below kSumLimit, each of them is a finite half-precision number and
  // the block is done; otherwise (the first block of a row, or scores that outgrew the running max by more than 11
  // powers of two) the wave takes the slow path: row max, rescale of O and l, weights again. The quotient O / l does
  // not depend on the reference max, so the result is the same either way.
  constexpr float kSumLimit = 2048.f;
  // A step is written as six groups fenced against each other (the compiler orders instructions inside a group only):
  //   groups 0-2: four QK MFMAs each (two K fragments x two halves); groups 3-5: four PV MFMAs each (two V^T fragments
  //   x two halves); beside them a third of a half's weights per group. Every fragment is read from LDS one group
  //   before its MFMAs. kfA / kfB carry the first two K fragments of the next step.
  auto step = [&](auto load_phase, auto do_qk, auto do_sm, auto do_pv, auto prefetch_next, const uint16_t *Kb, const uint16_t *Vb,
                  const uint16_t *Kb_next, floatx16_t (&S)[2], floatx16_t (&Sn)[2], vec8 (&Pp)[2][2], vec8 (&Pn)[2][2],
                  vec8 &kfA, vec8 &kfB) {
    constexpr bool QK = decltype(do_qk)::value, SM = decltype(do_sm)::value, PV = decltype(do_pv)::value;
    constexpr bool NEXT = decltype(prefetch_next)::value;
    constexpr int LP = decltype(load_phase)::value;  // this step issues pieces 6 LP .. 6 LP + 5 of the next tile (-1: none)
    float mc[2] = {m_i[0] * c, m_i[1] * c};
    float sg[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
    vec8 kf2, kf3, kf4, kf5, vf0, vf1, vf2, vf3, vf4, vf5;
    auto qk2 = [&](vec8 fa, int ka, vec8 fb, int kb) {
#pragma unroll
      for (int h = 0; h < 2; h++) {
        if (ka == 0) {
          floatx16_t z;
#pragma unroll
          for (int i = 0; i < 16; i++) z[i] = 0.f;
          Sn[h] = MT::mfma(fa, qreg[h][ka], z);
        } else {
          Sn[h] = MT::mfma(fa, qreg[h][ka], Sn[h]);
        }
      }
#pragma unroll
      for (int h = 0; h < 2; h++) Sn[h] = MT::mfma(fb, qreg[h][kb], Sn[h]);
    };
    auto pv2 = [&](vec8 fa, int f_a, vec8 fb, int f_b) {
#pragma unroll
      for (int h = 0; h < 2; h++) mfma_acc(MT{}, fa, Pp[h][f_a / DB], oacc[h][f_a % DB]);
#pragma unroll
      for (int h = 0; h < 2; h++) mfma_acc(MT{}, fb, Pp[h][f_b / DB], oacc[h][f_b % DB]);
    };
    // ---- group 0 ----
    if (LP >= 0) load_piece(6 * LP + 0);
    if (QK) {
      kf2 = k_frag(Kb, 2);
      kf3 = k_frag(Kb, 3);
      qk2(kfA, 0, kfB, 1);
    }
    if (SM) weights(0, 0, 6, S, Pn, mc, sg);
    __builtin_amdgcn_sched_barrier(0);
    // ---- group 1 ----
    if (LP >= 0) load_piece(6 * LP + 1);
    if (QK) {
      kf4 = k_frag(Kb, 4);
      kf5 = k_frag(Kb, 5);
      qk2(kf2, 2, kf3, 3);
    }
    if (SM) weights(0, 6, 10, S, Pn, mc, sg);
    __builtin_amdgcn_sched_barrier(0);
    // ---- group 2 ----
    if (LP >= 0) load_piece(6 * LP + 2);
    if (PV) {
      vf0 = v_frag(Vb, 0);
      vf1 = v_frag(Vb, 1);
    }
    if (QK) qk2(kf4, 4, kf5, 5);
    if (SM) weights(0, 10, 16, S, Pn, mc, sg);
    __builtin_amdgcn_sched_barrier(0);
    // ---- group 3 ----
    if (LP >= 0) load_piece(6 * LP + 3);
    if (PV) {
      vf2 = v_frag(Vb, 2);
      vf3 = v_frag(Vb, 3);
      pv2(vf0, 0, vf1, 1);
    }
    if (SM) weights(1, 0, 6, S, Pn, mc, sg);
    __builtin_amdgcn_sched_barrier(0);
    // ---- group 4 ----
    if (LP >= 0) load_piece(6 * LP + 4);
    if (PV) {
      vf4 = v_frag(Vb, 4);
      vf5 = v_frag(Vb, 5);
      pv2(vf2, 2, vf3, 3);
    }
    if (SM) weights(1, 6, 10, S, Pn, mc, sg);
    __builtin_amdgcn_sched_barrier(0);
    // ---- group 5 ----
    if (LP >= 0) load_piece(6 * LP + 5);
    if (NEXT) {
      kfA = k_frag(Kb_next, 0);
      kfB = k_frag(Kb_next, 1);
    }
    if (PV) pv2(vf4, 4, vf5, 5);
    if (SM) {
      weights(1, 10, 16, S, Pn, mc, sg);
      float sum[2] = {sg[0][0] + sg[0][1], sg[1][0] + sg[1][1]};
      // (written so that a NaN sum takes the slow path too)
      if (__builtin_expect(__builtin_amdgcn_ballot_w64(!(fmaxf(sum[0], sum[1]) <= kSumLimit)) != 0, 0)) {
        settle();  // the PV MFMAs of this step have landed in O: everything in O is relative to the old max
#pragma unroll
        for (int h = 0; h < 2; h++) {
          float mx = S[h][0];
#pragma unroll
          for (int i = 1; i < 16; i++) mx = fmaxf(mx, S[h][i]);
          mx = max_over_wave_halves(mx);
          const float m_new = fmaxf(m_i[h], mx);
          const float alpha = __builtin_amdgcn_exp2f((m_i[h] - m_new) * c);
          m_i[h] = m_new;
          l_i[h] *= alpha;
#pragma unroll
          for (int db = 0; db < DB; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) oacc[h][db][i] *= alpha;
          const float mcn = m_new * c;
          float sa = 0.f;
#pragma unroll
          for (int e = 0; e < 16; e++) {
            const float pe = __builtin_amdgcn_exp2f(S[h][e] * c - mcn);
            Pn[h][e >> 3][e & 7] = MT::cvt(pe);
            sa += pe;
          }
          sum[h] = sa;
        }
        settle();
      }
      l_i[0] += sum[0];
      l_i[1] += sum[1];
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  using std::true_type;
  using std::false_type;
  const true_type T{};
  const false_type F{};
  static_assert(NPIECE <= 18, "three steps issue the pieces of a tile");
  const std::integral_constant<int, 0> L0{};
  const std::integral_constant<int, 1> L1{};
  const std::integral_constant<int, 2> L2{};
  const std::integral_constant<int, -1> LN{};

  floatx16_t S0[2], S1[2];
  vec8 P0[2][2], P1[2][2];
  vec8 kfA, kfB;
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int e = 0; e < 8; e++) P0[h][t][e] = P1[h][t][e] = MT::cvt(0.f);

  if (n_kv_tiles > 0) load_tile(0, 0);
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int ks = 0; ks < KS; ks++) asm volatile("" :: "v"(qreg[h][ks]));

  // Block i = 4 kt + j. Step (kt, j) runs QK of block 4 kt + j, softmax of block 4 kt + j - 1 and PV of block
  // 4 kt + j - 2; the S and P sets alternate with the block's parity.
  // The first tile fills the pipeline; it is peeled so that the loop body has a single path.
  if (n_kv_tiles > 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    load_target(1, 1);  // (a tile past the last key fetches out of range: zeros into a buffer nobody reads)
    const uint16_t *Kt = &lds[0];
    const uint16_t *Vt = &lds[NBUF * K_BUF];
    kfA = k_frag(Kt, 0);
    kfB = k_frag(Kt, 1);
    step(L0, T, F, F, T, Kt, Vt, Kt + 32 * LDK, S1, S0, P0, P1, kfA, kfB);
    step(L1, T, T, F, T, Kt + 32 * LDK, Vt, Kt + 64 * LDK, S0, S1, P1, P0, kfA, kfB);
    step(L2, T, T, T, T, Kt + 64 * LDK, Vt, Kt + 96 * LDK, S1, S0, P0, P1, kfA, kfB);
    step(LN, T, T, T, F, Kt + 96 * LDK, Vt + 32 * LDV, Kt, S0, S1, P1, P0, kfA, kfB);
  }
  int buf = 1, buf_prev = 0;  // LDS buffer of tile kt and of tile kt - 1
  for (int kt = 1; kt < n_kv_tiles; kt++) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's blocks of tile kt are in LDS
    __syncthreads();  // ... and everyone's; every wave is done with tile kt-2, whose buffer the next fetch overwrites
    const int buf_next = buf == NBUF - 1 ? 0 : buf + 1;
    load_target(kt + 1, buf_next);
    const uint16_t *Kt = &lds[buf * K_BUF];
    const uint16_t *Vt = &lds[NBUF * K_BUF + buf * V_BUF];
    const uint16_t *Vp = &lds[NBUF * K_BUF + buf_prev * V_BUF];
    kfA = k_frag(Kt, 0);
    kfB = k_frag(Kt, 1);
    step(L0, T, T, T, T, Kt, Vp + 64 * LDV, Kt + 32 * LDK, S1, S0, P0, P1, kfA, kfB);
    step(L1, T, T, T, T, Kt + 32 * LDK, Vp + 96 * LDV, Kt + 64 * LDK, S0, S1, P1, P0, kfA, kfB);
    step(L2, T, T, T, T, Kt + 64 * LDK, Vt, Kt + 96 * LDK, S1, S0, P0, P1, kfA, kfB);
    step(LN, T, T, T, F, Kt + 96 * LDK, Vt + 32 * LDV, Kt, S0, S1, P1, P0, kfA, kfB);
    buf_prev = buf;
    buf = buf_next;
  }
  // drain: softmax of the last block, PV of the last two (they are in tile n_kv_tiles - 1, buffer buf_prev)
  if (n_kv_tiles > 0) {
    const uint16_t *Vp = &lds[NBUF * K_BUF + buf_prev * V_BUF];
    step(LN, F, T, T, F, Vp, Vp + 64 * LDV, Vp, S1, S0, P0, P1, kfA, kfB);
    step(LN, F, F, T, F, Vp, Vp + 96 * LDV, Vp, S0, S1, P1, P0, kfA, kfB);
  }
  settle();

  // ---- epilogue: out[qi][d] = O^T[d][qi] / l ----
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const float l_tot = sum_over_wave_halves(l_i[h]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (qi[h] < a.Sq) {
      const int64_t off = b * a.os[0] + hq * a.os[1] + (int64_t)qi[h] * a.os[2];
      uint16_t *op = reinterpret_cast<uint16_t *>(a.out) + off;
      float *op32 = reinterpret_cast<float *>(a.out) + off;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const int d = db * 32 + 8 * i4 + 4 * g;
          if (d >= a.D) continue;
          if (a.out_f32) {
            *reinterpret_cast<float4 *>(op32 + d) =
                make_float4(oacc[h][db][4 * i4 + 0] * inv, oacc[h][db][4 * i4 + 1] * inv, oacc[h][db][4 * i4 + 2] * inv,
                            oacc[h][db][4 * i4 + 3] * inv);
            continue;
          }
          uint2 packed;
          packed.x = (uint32_t)MT::cvt_bits(oacc[h][db][4 * i4 + 0] * inv) |
                     ((uint32_t)MT::cvt_bits(oacc[h][db][4 * i4 + 1] * inv) << 16);
          packed.y = (uint32_t)MT::cvt_bits(oacc[h][db][4 * i4 + 2] * inv) |
                     ((uint32_t)MT::cvt_bits(oacc[h][db][4 * i4 + 3] * inv) << 16);
          *reinterpret_cast<uint2 *>(op + d) = packed;
        }
    }
  }
}

template <typename MT, int D>
int launch_w64(const PrefillArgs &a, hipStream_t stream) {
  const int n_q_tiles = a.Sq / 256;
  const int n_bh_groups = (a.B * a.Hq + 7) / 8;
  dim3 grid(8 * n_bh_groups * n_q_tiles), block(256);
  if (plan_only("prefill_mfma_w64_kernel<%s, D=%d> workgroups=%u", MT::kName, D, grid.x)) return LMH_OK;
  hipLaunchKernelGGL((prefill_mfma_w64_kernel<MT, D>), grid, block, 0, stream, a, n_q_tiles, n_bh_groups);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

}  // namespace

bool prefill_w64_takes(const PrefillArgs &a, int dtype) {
  return dtype == LMH_F16 && a.D == 96 && !a.causal && !a.kv_len && !a.q_rope && a.Sq > 0 && a.Sq % 256 == 0 && a.Sk >= 256 &&
         a.Sk % 128 == 0;
}

int launch_prefill_w64(const PrefillArgs &a, hipStream_t stream) { return launch_w64<MfmaF16, 96>(a, stream); }

}  // namespace lmh
