// Pieces shared by the matrix-core flash attention kernels (fp16 / bf16 in, fp32 accumulate): tile constants, LDS
// paddings and the two element-type policies (MFMA instruction, conversions, row sums).
#pragma once

#include "common.hpp"
#include "dtypes.hpp"

namespace lmh {
namespace {

constexpr int BN = 64;   // keys per staged tile (twice that in one instantiation, see BT)
// LDS row paddings in elements. K rows are read 16 bytes per lane, one row per lane: a stride of
// D + 8 elements spreads 16 consecutive rows over all banks (5 cycles per 1 KB fragment per CU,
// against 16 unpadded). V rows go through the transposing read (4 rows x 32 bytes per 16 lanes); in
// a microbenchmark its cost depends on the stride (5.6 cycles per fragment at 96 elements modulo
// 128, 8 at D + 8, 16 at a multiple of 128 bytes), in the kernel D = 64 measures the same with 0, 8,
// 16 or 32 elements of padding, and 0 lets a fourth workgroup fit on a CU.
constexpr int kPadK = 8;
template <int D> constexpr int pad_v() { return D == 128 ? 32 : 0; }
constexpr float kLog2e = 1.4426950408889634f;
// The running max is only raised (and the output rescaled) when a row's scores outgrow it by more
// than this many powers of two; until then P is computed against the stale max and may reach
// 2^kLazyRescale, which fp16/bf16/fp32 all hold. The quotient O / l does not depend on the reference
// max, so the result is unchanged while most tiles skip the D-wide rescale.
constexpr float kLazyRescale = 8.0f;
// Byte offset no K/V slice reaches (the host routes larger ones elsewhere): a buffer load there
// is out of range and returns zeros.
constexpr int kOutOfRange = 0x7ffffff0;

typedef short shortx8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) shortx4_t lds_shortx4_t;

struct MfmaF16 {
  static constexpr const char *kName = "f16";
  using vec8 = half8_t;
  static constexpr bool kSplitP = false;  // 11 significant bits in P are within the 2e-3 budget
  static constexpr bool kConvertV = false;
  using pvec8 = vec8;  // the softmax weights, as the matrix cores take them
  __device__ static floatx16_t mfma(vec8 a, vec8 b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static uint16_t cvt_bits(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }
  __device__ static _Float16 cvt(float x) { return (_Float16)x; }
  __device__ static _Float16 cvt_p(float x) { return (_Float16)x; }
  __device__ static floatx16_t mfma_pv(vec8 v, pvec8 p, floatx16_t c) { return mfma(v, p, c); }
  // acc + sum of the 8 (already rounded) elements: 4 x v_dot2_f32_f16 against (1, 1)
  __device__ static float sum8(vec8 p, float acc) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 one = {(_Float16)1.f, (_Float16)1.f};
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(p, p, 0, 1), one, acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(p, p, 2, 3), one, acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(p, p, 4, 5), one, acc, false);
    acc = __builtin_amdgcn_fdot2(__builtin_shufflevector(p, p, 6, 7), one, acc, false);
    return acc;
  }
};
struct MfmaBF16 {
  static constexpr const char *kName = "bf16";
  using vec8 = bf16x8_t;
  // A bf16 P has 8 significant bits; on short or peaked rows that alone is ~2.5e-3 of the output
  // range. P is therefore fed to the matrix cores as head + remainder (two MFMAs per V fragment).
  static constexpr bool kSplitP = true;
  static constexpr bool kConvertV = false;
  using pvec8 = vec8;
  __device__ static floatx16_t mfma(vec8 a, vec8 b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static uint16_t cvt_bits(float x) { return f32_to_bf16_bits(x); }
  __device__ static __bf16 cvt(float x) { return (__bf16)x; }
  __device__ static __bf16 cvt_p(float x) { return (__bf16)x; }
  __device__ static floatx16_t mfma_pv(vec8 v, pvec8 p, floatx16_t c) { return mfma(v, p, c); }
  __device__ static float sum8(vec8 p, float acc) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    const b2 one = {(__bf16)1.f, (__bf16)1.f};
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(p, p, 0, 1), one, acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(p, p, 2, 3), one, acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(p, p, 4, 5), one, acc, false);
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(p, p, 6, 7), one, acc, false);
    return acc;
  }
};


// bf16 tensors with the second product in fp16: S^T = K Q^T runs on the bf16 MFMA (its operands are exact), the
// softmax weights are rounded to fp16 (11 significant bits, one MFMA per V fragment instead of head + remainder) and
// the V tiles are rewritten as fp16 on their way into LDS. A bf16 value has 8 significant bits, so the rewrite is exact
// once the exponent fits: every tile is stored relative to the largest finite |v| the workgroup has met so far (that
// value lands at 2^14), values more than 2^29 below it go to zero, and the accumulators carry the power of two.
struct MfmaBF16V16 : MfmaBF16 {
  static constexpr bool kSplitP = false;
  static constexpr bool kConvertV = true;
  using pvec8 = half8_t;
  __device__ static _Float16 cvt_p(float x) { return (_Float16)x; }
  __device__ static floatx16_t mfma_pv(vec8 v, pvec8 p, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, v), p, c, 0, 0, 0);
  }
  __device__ static float sum8(pvec8 p, float acc) { return MfmaF16::sum8(p, acc); }
};

// One 32-bit word = two bf16 values -> two fp16 values holding v * 2^(112 - thr) (thr = the biased bf16 exponent that
// maps to the fp16 exponent field 0): exponent and mantissa bits shifted into place with 16-bit packed integer
// instructions, no float arithmetic. Finite inputs whose exponent is at most thr come out as zero or as an fp16
// subnormal (|result| < 2^-14); the caller guarantees exponent - thr <= 29 for every finite input.
typedef uint16_t u16x2_t __attribute__((ext_vector_type(2)));
__device__ inline uint32_t bf16x2_to_scaled_f16x2(uint32_t w, uint32_t thr_bits2) {
  const u16x2_t t = __builtin_bit_cast(u16x2_t, w & 0x7fff7fffu);
  const u16x2_t e = __builtin_elementwise_sub_sat(t, __builtin_bit_cast(u16x2_t, thr_bits2));
  const u16x2_t three = {3, 3};
  return (w & 0x80008000u) | __builtin_bit_cast(uint32_t, (u16x2_t)(e << three));
}
// the same for a word that may hold infinities or NaNs (kept as such)
__device__ inline uint32_t bf16x2_to_scaled_f16x2_any(uint32_t w, uint32_t thr_bits2) {
  uint32_t r = bf16x2_to_scaled_f16x2(w, thr_bits2);
  if ((w & 0x7f80u) == 0x7f80u) r = (r & 0xffff0000u) | (w & 0x8000u) | 0x7c00u | ((w & 0x7fu) ? 0x200u : 0u);
  if ((w & 0x7f800000u) == 0x7f800000u) r = (r & 0x0000ffffu) | (w & 0x80000000u) | 0x7c000000u | ((w & 0x7f0000u) ? 0x2000000u : 0u);
  return r;
}
// largest |bits| (exponent and mantissa, 15 bits) over the finite halves of a word, folded into m
__device__ inline uint32_t bf16x2_finite_top(uint32_t w, uint32_t m) {
  const uint32_t lo = w & 0x7fffu, hi = (w >> 16) & 0x7fffu;
  if (lo < 0x7f80u) m = max(m, lo);
  if (hi < 0x7f80u) m = max(m, hi);
  return m;
}

// Epilogue of the matrix-core flash attention kernels: out[qi][d] = O^T[d][qi] * inv for the wave's 32 query rows.
// In the accumulator layout lane (n, g) holds, per 32-row block db of O^T, four groups of four consecutive head dims:
// d = 32 db + 8 i4 + 4 g + (0..3). Written as they lie (WIDE16 = false), a 16-bit output takes one 8-byte store per
// group, each a separate partial-line request. With WIDE16 one v_permlane32_swap per packed register hands the lower
// half-wave both halves of the even groups and the upper half-wave both halves of the odd ones: 16 contiguous bytes
// per lane and store, half the store instructions and requests. That pays where the epilogue is a visible share of
// the launch (B=4 H=20 Sq=448 Sk=1500 D=64 fp16 through prefill_mfma_wide_kernel: 25.24 -> 24.75 us, and 7.3 -> 6.7 us
// with no keys at all); in the long causal launches of prefill_mfma_kernel and prefill_mfma_pair_kernel it measured
// no gain (B=1 H=32 S=4096 D=96: fp16 109.9 -> 110.3 us, bf16 153.2 -> 155.9 us), so those keep the plain form.
template <typename MT, int DB, bool WIDE16>
__device__ inline void store_out_rows(const floatx16_t (&oacc)[DB], float inv, void *out, int64_t row_off, int g, int d_valid,
                                      bool out_f32) {
  if (out_f32) {
    float *op32 = reinterpret_cast<float *>(out) + row_off;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int d = db * 32 + 8 * i4 + 4 * g;
        if (d >= d_valid) continue;
        *reinterpret_cast<float4 *>(op32 + d) = make_float4(oacc[db][4 * i4 + 0] * inv, oacc[db][4 * i4 + 1] * inv,
                                                            oacc[db][4 * i4 + 2] * inv, oacc[db][4 * i4 + 3] * inv);
      }
    return;
  }
  uint16_t *op = reinterpret_cast<uint16_t *>(out) + row_off;
  auto pack2 = [&](int db, int i) {
    return (uint32_t)MT::cvt_bits(oacc[db][i] * inv) | ((uint32_t)MT::cvt_bits(oacc[db][i + 1] * inv) << 16);
  };
#pragma unroll
  for (int db = 0; db < DB; db++) {
    if constexpr (WIDE16) {
#pragma unroll
      for (int pr = 0; pr < 2; pr++) {
        // w[0..1] = the even group (i4 = 2 pr), w[2..3] = the odd group (i4 = 2 pr + 1)
        float w[4];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
          for (int j = 0; j < 2; j++) w[2 * h + j] = __uint_as_float(pack2(db, 4 * (2 * pr + h) + 2 * j));
        // afterwards the lower lanes hold (their even dims 0..3, the upper lanes' even dims 4..7) and the upper lanes
        // (the lower lanes' odd dims 0..3, their own odd dims 4..7)
        swap_wave_halves(w[0], w[2]);
        swap_wave_halves(w[1], w[3]);
        const int d = db * 32 + 8 * (2 * pr + g);
        if (d >= d_valid) continue;
        *reinterpret_cast<uint4 *>(op + d) =
            make_uint4(__float_as_uint(w[0]), __float_as_uint(w[1]), __float_as_uint(w[2]), __float_as_uint(w[3]));
      }
    } else {
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int d = db * 32 + 8 * i4 + 4 * g;
        if (d >= d_valid) continue;
        *reinterpret_cast<uint2 *>(op + d) = make_uint2(pack2(db, 4 * i4), pack2(db, 4 * i4 + 2));
      }
    }
  }
}

}  // namespace
}  // namespace lmh
