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
  __device__ static floatx16_t mfma(vec8 a, vec8 b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static uint16_t cvt_bits(float x) { return __builtin_bit_cast(uint16_t, (_Float16)x); }
  __device__ static _Float16 cvt(float x) { return (_Float16)x; }
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
  __device__ static floatx16_t mfma(vec8 a, vec8 b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  __device__ static uint16_t cvt_bits(float x) { return f32_to_bf16_bits(x); }
  __device__ static __bf16 cvt(float x) { return (__bf16)x; }
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


}  // namespace
}  // namespace lmh
