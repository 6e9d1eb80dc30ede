// A plain device-to-device copy kernel of known size. It exists so that hardware traffic counters
// (FETCH_SIZE / WRITE_SIZE) can be scaled: profile this kernel on N bytes, read what the counter
// reports, and apply the same factor to the attention kernels' readings.
#include "common.hpp"

namespace lmh {
namespace {
__global__ __launch_bounds__(256) void calib_copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = src[i];
}
}  // namespace
}  // namespace lmh

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
