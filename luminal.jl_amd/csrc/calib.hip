// A plain device-to-device copy kernel of known size. It exists so that hardware traffic counters
// (FETCH_SIZE / WRITE_SIZE) can be scaled: profile this kernel on N bytes, read what the counter
// reports, and apply the same factor to the attention kernels' readings.
//
// A bare MFMA loop on caller-supplied operands. The published matrix-core peak assumes the boost clock;
// under a full-chip MFMA load the clock is power-managed and depends on how many operand bits toggle
// (all-zero operands sustain a much higher rate than random ones). Timing this kernel on the same
// kind of data as the attention inputs gives the rate the matrix cores can actually sustain, the
// ceiling an attention kernel is measured against besides the published figure.
//
// These kernels are measurement aids, not part of the attention backend: they are built into their own library,
// libluminal_hip_calib.so (include/luminal_hip_calib.h), which only the benchmark and its test load.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/luminal_hip_calib.h"

namespace lmh {
namespace {
thread_local char g_calib_error[256] = "";
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_calib_error, sizeof(g_calib_error), fmt, ap);
  va_end(ap);
  return code;
}
#define LMH_HIP_TRY(expr)                                                                                    \
  do {                                                                                                       \
    hipError_t lmh_e_ = (expr);                                                                              \
    if (lmh_e_ != hipSuccess) return fail(LMH_E_HIP, "HIP error %d (%s) in %s", (int)lmh_e_, hipGetErrorString(lmh_e_), #expr); \
  } while (0)

typedef _Float16 calib_half8_t __attribute__((ext_vector_type(8)));
typedef float calib_floatx16_t __attribute__((ext_vector_type(16)));
constexpr int kCalibMfmaGrid = 512;    // two workgroups per CU
constexpr int kCalibMfmaPerIter = 8;   // MFMAs per wave per loop iteration

// active_xcds < 8: workgroups that land on XCD `active_xcds` or above (the hardware's own XCC_ID) leave at once and
// mark their first sink slot with -1, so the loop runs on part of the chip while the rest idles.
__global__ __launch_bounds__(256, 2) void calib_mfma_kernel(float *__restrict__ sink, const calib_half8_t *__restrict__ operands,
                                                            int n_operands, int iters, int active_xcds) {
  if (active_xcds < 8) {
    const int xcc = __builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15;  // HW_REG_XCC_ID, bits 3:0
    if (xcc >= active_xcds) {
      if (threadIdx.x == 0) sink[blockIdx.x * 256] = -1.f;
      return;
    }
  }
  calib_half8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = operands[(threadIdx.x * 4 + i) % n_operands];
    b[i] = operands[(threadIdx.x * 4 + i + n_operands / 2) % n_operands];
  }
  calib_floatx16_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; c++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[c][i] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int m = 0; m < kCalibMfmaPerIter; m++) {
      acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m & 3], b[(m >> 1) & 3], acc[m & 3], 0, 0, 0);
      // Several waves of a SIMD running MFMAs with nothing in between settle into one of two rates, the full one or two
      // thirds of it, depending on how far apart they started; one scalar instruction between the MFMAs keeps the full rate.
      asm volatile("s_nop 0");
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; c++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[c][i];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void calib_copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = src[i];
}
// An interleaved stream with a chosen instruction mix per MFMA: NV vector instructions (NE of them v_exp_f32, the
// rest fused multiply-adds) and one 16-byte-per-lane LDS read every LDS_EVERY MFMAs (0 = none; the fragment read
// feeds the A operand of the next LDS_EVERY MFMAs). Two or four waves per SIMD, operands from caller-supplied values. This
// is the best case of a kernel with that mix — no barriers, no staging, no dependencies between the MFMA and the
// vector work — so its rate on the whole chip is the ceiling for an attention kernel of the same mix.
// AGPR_ACC = true keeps the MFMA accumulators in accumulation registers (AGPRs) instead of the vector registers the
// compiler picks for a kernel of this size: does it matter to the vector work beside the MFMAs which file they are in?
template <bool AGPR_ACC>
__device__ inline void calib_mfma(calib_floatx16_t &acc, calib_half8_t a, calib_half8_t b) {
  if constexpr (AGPR_ACC) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  else acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
}
template <int NV, int NE, int LDS_EVERY, bool AGPR_ACC = false>
__global__ __launch_bounds__(512) void calib_mix_kernel(float *__restrict__ sink, const calib_half8_t *__restrict__ operands,
                                                        int n_operands, int iters) {
  __shared__ calib_half8_t lds[4096];
  for (int i = threadIdx.x; i < 4096; i += 512) lds[i] = operands[i % n_operands];
  __syncthreads();
  calib_half8_t a[8], b[4];
#pragma unroll
  for (int i = 0; i < 8; i++) a[i] = operands[(threadIdx.x * 4 + i) % n_operands];
#pragma unroll
  for (int i = 0; i < 4; i++) b[i] = operands[(threadIdx.x * 4 + i + n_operands / 2) % n_operands];
  calib_floatx16_t acc[4];
#pragma unroll
  for (int c = 0; c < 4; c++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[c][i] = 0.f;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = (float)a[0][i];
  int idx = threadIdx.x;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int m = 0; m < 8; m++) {
      const int frag = LDS_EVERY > 1 ? (m / LDS_EVERY) * LDS_EVERY : m;
      calib_mfma<AGPR_ACC>(acc[m & 3], a[frag & 7], b[m & 3]);
      if (NV == 0 && LDS_EVERY == 0) {  // nothing between the MFMAs otherwise: see calib_mfma_kernel
        asm volatile("s_nop 0");
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int j = 0; j < NV; j++) {
        if (j < NE) v[j & 7] = __builtin_amdgcn_exp2f(v[j & 7] * 0.001f);
        else v[j & 7] = __builtin_fmaf(v[j & 7], 0.999f, 0.25f);
      }
      if (LDS_EVERY > 0 && m % LDS_EVERY == 0) {  // the fragment MFMAs m + 4 .. use
        a[(m + 4) & 7] = lds[idx & 4095];
        idx += 517;
      }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; c++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[c][i];
#pragma unroll
  for (int i = 0; i < 8; i++) s += v[i];
  sink[blockIdx.x * 512 + threadIdx.x] = s;
}

// Read-only stream with non-temporal 16-byte loads, 8 in flight per lane: what the memory system delivers to a
// kernel that does nothing else (256 workgroups of 256 threads, one slab each).
typedef unsigned calib_u4_t __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void calib_read_kernel(const calib_u4_t *__restrict__ src, size_t n_per_wg, unsigned *__restrict__ sink) {
  const calib_u4_t *p = src + (size_t)blockIdx.x * n_per_wg;
  unsigned acc = 0;
  size_t i = threadIdx.x;
  for (; i + 7 * 256 < n_per_wg; i += 8 * 256) {
    calib_u4_t v[8];
#pragma unroll
    for (int u = 0; u < 8; u++) v[u] = __builtin_nontemporal_load(p + i + u * 256);
    __builtin_amdgcn_sched_barrier(0);  // all eight loads are issued before the first is consumed
#pragma unroll
    for (int u = 0; u < 8; u++) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n_per_wg; i += 256) {
    const calib_u4_t v = __builtin_nontemporal_load(p + i);
    acc += v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) *sink = acc;  // keeps the loads alive; practically never taken
}
}  // namespace
}  // namespace lmh

extern "C" const char *lmh_calib_last_error(void) { return lmh::g_calib_error; }

extern "C" int lmh_calib_read(const void *src, size_t bytes, void *sink4, void *stream) {
  using namespace lmh;
  if (!src || !sink4) return fail(LMH_E_NULL, "lmh_calib_read: null pointer");
  if (bytes % (16 * 256) != 0 || (reinterpret_cast<uintptr_t>(src) & 15u))
    return fail(LMH_E_SHAPE, "lmh_calib_read: size must be a multiple of 4096 bytes and the pointer 16-byte aligned");
  if (bytes == 0) return LMH_OK;
  hipLaunchKernelGGL(calib_read_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<const calib_u4_t *>(src),
                     bytes / 16 / 256, reinterpret_cast<unsigned *>(sink4));
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

extern "C" int lmh_calib_copy(void *dst, const void *src, size_t bytes, void *stream) {
  using namespace lmh;
  if (!dst || !src) return fail(LMH_E_NULL, "lmh_calib_copy: null pointer");
  if (bytes % 16 != 0 || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u))
    return fail(LMH_E_SHAPE, "lmh_calib_copy: size and pointers must be multiples of 16 bytes");
  if (bytes == 0) return LMH_OK;
  hipLaunchKernelGGL(calib_copy_kernel, dim3(8192), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<uint4 *>(dst),
                     reinterpret_cast<const uint4 *>(src), bytes / 16);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

extern "C" int lmh_calib_mfma_xcds(void *sink, const void *operands, size_t operand_bytes, int iters, int active_xcds,
                                   double *flops_per_workgroup, void *stream) {
  using namespace lmh;
  if (!sink || !operands) return fail(LMH_E_NULL, "lmh_calib_mfma: null pointer");
  if (operand_bytes < 32 || operand_bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(operands) & 15u) || iters < 1)
    return fail(LMH_E_SHAPE, "lmh_calib_mfma: operands must be >= 32 bytes, a multiple of 16, 16-byte aligned; iters >= 1");
  if (active_xcds < 1 || active_xcds > 8) return fail(LMH_E_SHAPE, "lmh_calib_mfma_xcds: active_xcds must be 1..8");
  hipLaunchKernelGGL(calib_mfma_kernel, dim3(kCalibMfmaGrid), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<float *>(sink),
                     reinterpret_cast<const calib_half8_t *>(operands), (int)(operand_bytes / 16), iters, active_xcds);
  LMH_HIP_TRY(hipGetLastError());
  if (flops_per_workgroup) *flops_per_workgroup = 4.0 * iters * kCalibMfmaPerIter * (2.0 * 32 * 32 * 16);
  return LMH_OK;
}

extern "C" int lmh_calib_mix(void *sink, const void *operands, size_t operand_bytes, int iters, int mix, int waves_per_simd,
                             double *flops, void *stream) {
  using namespace lmh;
  if (!sink || !operands) return fail(LMH_E_NULL, "lmh_calib_mix: null pointer");
  if (operand_bytes < 32 || operand_bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(operands) & 15u) || iters < 1)
    return fail(LMH_E_SHAPE, "lmh_calib_mix: operands must be >= 32 bytes, a multiple of 16, 16-byte aligned; iters >= 1");
  if (waves_per_simd != 2 && waves_per_simd != 4)
    return fail(LMH_E_UNSUPPORTED, "lmh_calib_mix: waves_per_simd must be 2 or 4, got %d", waves_per_simd);
  const dim3 grid(128 * waves_per_simd), block(512);  // one or two workgroups of 8 waves per CU
  float *snk = reinterpret_cast<float *>(sink);
  const calib_half8_t *ops = reinterpret_cast<const calib_half8_t *>(operands);
  const int n_ops = (int)(operand_bytes / 16);
  const hipStream_t st = (hipStream_t)stream;
  switch (mix) {
    case 0: hipLaunchKernelGGL((calib_mix_kernel<0, 0, 0>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 1: hipLaunchKernelGGL((calib_mix_kernel<6, 1, 0>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 2: hipLaunchKernelGGL((calib_mix_kernel<6, 1, 1>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 3: hipLaunchKernelGGL((calib_mix_kernel<6, 1, 2>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 4: hipLaunchKernelGGL((calib_mix_kernel<4, 1, 1>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 5: hipLaunchKernelGGL((calib_mix_kernel<4, 1, 2>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 6: hipLaunchKernelGGL((calib_mix_kernel<11, 0, 1>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 7: hipLaunchKernelGGL((calib_mix_kernel<6, 1, 1, true>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    case 8: hipLaunchKernelGGL((calib_mix_kernel<4, 1, 2, true>), grid, block, 0, st, snk, ops, n_ops, iters); break;
    default: return fail(LMH_E_UNSUPPORTED, "lmh_calib_mix: mix %d is not one of 0..8", mix);
  }
  LMH_HIP_TRY(hipGetLastError());
  if (flops) *flops = (double)grid.x * 8.0 * iters * 8.0 * (2.0 * 32 * 32 * 16);
  return LMH_OK;
}

extern "C" int lmh_calib_mfma(void *sink, const void *operands, size_t operand_bytes, int iters, double *flops, void *stream) {
  double per_wg = 0.0;
  const int rc = lmh_calib_mfma_xcds(sink, operands, operand_bytes, iters, 8, &per_wg, stream);
  if (rc == LMH_OK && flops) *flops = per_wg * lmh::kCalibMfmaGrid;
  return rc;
}
