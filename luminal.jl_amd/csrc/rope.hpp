// Rotary position embedding arithmetic shared by the standalone kernels (cache_ops.hip) and by the flash attention
// kernels that rotate their query rows on the way in: apply_rotary_embeddings, reference src/NN.jl:253-303.
// inv_freq[j] = 1 / base^(2j/D), angle = position * inv_freq[j], (x0, x1) -> (x0 cos - x1 sin, x0 sin + x1 cos);
// the pair of j is (j, j + D/2) in the reference (its reshape to (D/2, 2) runs on a column-major array), or
// (2j, 2j + 1) in the interleaved convention. Every kernel goes through these functions, so a fused rotation gives the
// bits the standalone kernel would have stored.
#pragma once

#include <hip/hip_runtime.h>

namespace lmh {

// sin and cos of an fp32 angle (radians, any magnitude an fp32 position reaches) on the hardware's
// v_sin_f32 / v_cos_f32, which take revolutions. The library sincosf costs ~100 instructions per angle (its
// large-argument path alone is a table walk) and made the rotary kernels compute-bound at 46 % of the
// memory roofline. Here the angle is reduced by whole turns with 2 pi split into its fp32 head and the
// remainder (two fused multiply-adds: the first is exact up to the rounding of a result no larger than
// ~pi, whatever the number of turns), so |r| <= pi to ~3e-7 rad, and r / 2 pi goes to the hardware.
__device__ inline void sincos_angle(float angle, float *sn, float *cs) {
  constexpr float kInv2Pi = 0.15915493667125702f;
  constexpr float k2PiHead = 6.2831854820251465f;      // fp32(2 pi)
  constexpr float k2PiTail = -1.7484555314695172e-07f;  // 2 pi - fp32(2 pi)
  const float turns = rintf(angle * kInv2Pi);
  float r = fmaf(-turns, k2PiHead, angle);
  r = fmaf(-turns, k2PiTail, r);
  const float x = r * kInv2Pi;
  *sn = __builtin_amdgcn_sinf(x);
  *cs = __builtin_amdgcn_cosf(x);
}

// inv_freq = 1 / exp2((2j/D) * log2(base)), evaluated as the reference does (src/NN.jl:262-263)
__device__ inline float rope_inv_freq(int j, int D, float log2_base) {
  const float freq = (float)j * 2.0f / (float)D;
  return 1.0f / exp2f(freq * log2_base);
}

// The result is the fp32 value, as the reference computes it; a caller that stores half precision rounds that value.
// Two things are pinned so that every kernel that shares this function produces the same bits: the fused multiply-adds
// are written out (left to the compiler, which product it fuses depends on the surrounding code), and the results pass
// through an empty asm statement, which keeps the compiler from merging the last fused multiply-add with the caller's
// conversion into one mixed-precision instruction that rounds once instead of twice.
__device__ inline void rope_rotate(float x0, float x1, float sn, float cs, float *o0, float *o1) {
  float r0 = fmaf(x0, cs, -(x1 * sn));
  float r1 = fmaf(x0, sn, x1 * cs);
  asm("" : "+v"(r0), "+v"(r1));
  *o0 = r0;
  *o1 = r1;
}

__device__ inline void rope_pair(float x0, float x1, float pos, int j, int D, float log2_base, float *o0, float *o1) {
  float sn, cs;
  sincos_angle(pos * rope_inv_freq(j, D, log2_base), &sn, &cs);
  rope_rotate(x0, x1, sn, cs, o0, o1);
}

// Element d of a row after the rotation at `pos`, for kernels that hold one element at a time; `row` points at the
// row's D elements, ld converts a stored element to fp32. The result is not yet rounded to the element type.
template <typename Raw, typename Ld>
__device__ inline float rope_element(const Raw *row, int d, int D, float pos, float log2_base, bool interleaved, Ld ld) {
  const int half = D / 2;
  const bool first = interleaved ? (d % 2 == 0) : (d < half);
  const int j = interleaved ? d / 2 : (d < half ? d : d - half);
  const int dp = interleaved ? (first ? d + 1 : d - 1) : (first ? d + half : d - half);
  const float x0 = ld(first ? row[d] : row[dp]);
  const float x1 = ld(first ? row[dp] : row[d]);
  float o0, o1;
  rope_pair(x0, x1, pos, j, D, log2_base, &o0, &o1);
  return first ? o0 : o1;
}

}  // namespace lmh
