// Element types of the attention tensors and their conversion to/from the fp32 the kernels
// accumulate in.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lmh {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));
typedef short shortx4_t __attribute__((ext_vector_type(4)));

// Reductions over lane l and lane l ^ 32 (the two halves of a wave) with v_permlane32_swap_b32: one vector instruction
// exchanges the upper half of one register with the lower half of another, where __shfl_xor(x, 32) is a round trip
// through the LDS crossbar (ds_bpermute_b32) plus its index arithmetic. Written as asm: given the same value for both
// operands the builtin's two results are treated as one. The s_nop covers the instruction's wait after a vector write
// of its operands.
__device__ inline void swap_wave_halves(float &a, float &b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32_e32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ inline float max_over_wave_halves(float x) {
  float a = x, b = x;
  swap_wave_halves(a, b);  // a = the lower half's x on all lanes, b = the upper half's
  return fmaxf(a, b);
}
__device__ inline float sum_over_wave_halves(float x) {
  float a = x, b = x;
  swap_wave_halves(a, b);
  return a + b;  // lower + upper on every lane: both halves get the same bits
}

__device__ inline float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round-to-nearest-even, NaN kept quiet
__device__ inline uint16_t f32_to_bf16_bits(float x) {
  uint32_t u = __float_as_uint(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

struct F32 {
  static constexpr const char *kName = "f32";
  using raw = float;
  static constexpr int kVec = 4;  // elements per 128-bit access
  __device__ static float ld(raw x) { return x; }
  __device__ static raw st(float x) { return x; }
};
struct F16 {
  static constexpr const char *kName = "f16";
  using raw = _Float16;
  static constexpr int kVec = 8;
  __device__ static float ld(raw x) { return (float)x; }
  __device__ static raw st(float x) { return (_Float16)x; }
};
struct BF16 {
  static constexpr const char *kName = "bf16";
  using raw = uint16_t;
  static constexpr int kVec = 8;
  __device__ static float ld(raw x) { return bf16_bits_to_f32(x); }
  __device__ static raw st(float x) { return f32_to_bf16_bits(x); }
};

// 128-bit load of data that is read exactly once by the whole launch (a KV cache streamed by decode
// attention, the rows an append moves): non-temporal, so the stream neither waits on nor displaces
// lines in L2 and the last-level cache. On C5 this alone takes decode from 6.0 to 6.7 TB/s.
typedef unsigned int u32x4_stream_t __attribute__((ext_vector_type(4)));
__device__ inline uint4 load_stream_128(const void *p) {
  const u32x4_stream_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_stream_t *>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

// Unpack one 128-bit global load into fp32 lanes.
template <typename E>
struct Vec128;

template <>
struct Vec128<F32> {
  float4 r;
  __device__ void load(const void *p) { r = *reinterpret_cast<const float4 *>(p); }
  __device__ void load_stream(const void *p) {
    const uint4 u = load_stream_128(p);
    r = make_float4(__uint_as_float(u.x), __uint_as_float(u.y), __uint_as_float(u.z), __uint_as_float(u.w));
  }
  __device__ void zero() { r = make_float4(0.f, 0.f, 0.f, 0.f); }
  __device__ void unpack(float *f) const { f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w; }
};
template <>
struct Vec128<F16> {
  uint4 r;
  __device__ void load(const void *p) { r = *reinterpret_cast<const uint4 *>(p); }
  __device__ void load_stream(const void *p) { r = load_stream_128(p); }
  __device__ void zero() { r = make_uint4(0, 0, 0, 0); }
  __device__ void unpack(float *f) const {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      typedef _Float16 h2 __attribute__((ext_vector_type(2)));
      h2 h = __builtin_bit_cast(h2, w[i]);
      f[2 * i] = (float)h[0];
      f[2 * i + 1] = (float)h[1];
    }
  }
};
template <>
struct Vec128<BF16> {
  uint4 r;
  __device__ void load(const void *p) { r = *reinterpret_cast<const uint4 *>(p); }
  __device__ void load_stream(const void *p) { r = load_stream_128(p); }
  __device__ void zero() { r = make_uint4(0, 0, 0, 0); }
  __device__ void unpack(float *f) const {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

}  // namespace lmh
