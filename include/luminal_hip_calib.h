/*
 * luminal_hip_calib.h — C ABI of libluminal_hip_calib.so: measurement kernels for the MI355X (gfx950) attention
 * backend. None of them has a counterpart in the reference and none is part of the attention path; they exist so
 * that a benchmark can scale hardware traffic counters against a transfer of known size and time the rates the
 * chip sustains on its own (a bare MFMA loop, synthetic instruction mixes, a read-only stream). The library is
 * separate from libluminal_hip.so: a host that only runs attention never loads it.
 *
 * Same conventions as luminal_hip.h: `extern "C"`, plain pointers and sizes, LMH_OK or a negative LMH_E_* code,
 * lmh_calib_last_error() holds the message of the last failure on the calling thread.
 */
#ifndef LUMINAL_HIP_CALIB_H
#define LUMINAL_HIP_CALIB_H

#include <stddef.h>
#include <stdint.h>

#include "luminal_hip.h" /* status codes */

#ifdef __cplusplus
extern "C" {
#endif

const char *lmh_calib_last_error(void);

/* A plain copy kernel (reads `bytes`, writes `bytes`; both pointers and the size multiples of 16) used to
 * calibrate HBM traffic counters against a known transfer. */
int lmh_calib_copy(void *dst_dev, const void *src_dev, size_t bytes, void *stream);
/* ... and a read-only stream over `bytes` (a multiple of 4096) with non-temporal 16-byte loads, 8 in flight per lane:
 * the rate the memory system delivers to a kernel that does nothing else, the practical ceiling of the decode
 * kernels at a given size. `sink4_dev` is 4 bytes of device memory (never written in practice). */
int lmh_calib_read(const void *src_dev, size_t bytes, void *sink4_dev, void *stream);

/* A bare loop of fp16 MFMAs (512 workgroups, 4 waves each, 8 v_mfma_f32_32x32x16_f16 per iteration) on operands
 * read from `operands_dev` (`operand_bytes` >= 32, a multiple of 16). The sustained matrix-core rate depends on the operand
 * values (clock management under load), so time it on data like the attention inputs. `sink_dev`
 * receives 512*256 floats; `*flops` (host, optional) the flops of one launch. */
int lmh_calib_mfma(void *sink_dev, const void *operands_dev, size_t operand_bytes, int iters, double *flops, void *stream);
/* The same loop on part of the chip: workgroups that land on XCD number `active_xcds` (1..8) or above exit at once
 * and set their first sink slot (sink[256 * workgroup]) to -1, the others run the loop, so the host can count
 * them. `*flops_per_workgroup` (host, optional) is what one running workgroup computes. Shows how the rate a CU
 * sustains depends on how much of the chip is busy (clock and power management). */
int lmh_calib_mfma_xcds(void *sink_dev, const void *operands_dev, size_t operand_bytes, int iters, int active_xcds,
                        double *flops_per_workgroup, void *stream);

/* An interleaved instruction stream with the mix of an attention inner loop, `waves_per_simd` (2 or 4) waves per SIMD on the whole chip, no barriers and no dependencies between the
 * matrix and the vector work: the best case for a kernel of that mix. Per v_mfma_f32_32x32x16_f16:
 *   mix 0: nothing else            mix 1: 6 vector instructions, one of them v_exp_f32
 *   mix 2: mix 1 + one 16-byte-per-lane LDS fragment read      mix 3: mix 1 + one such read per two MFMAs
 *   mix 4: 4 vector instructions (1 exp) + one read            mix 5: 4 vector instructions (1 exp) + one read per two
 *   mix 6: 11 vector instructions, none of them exp (the exp of mix 2 as a six-instruction polynomial) + one read
 *   mix 7: mix 2, mix 8: mix 5, with the MFMA accumulators in accumulation registers (AGPRs) instead of vector registers
 * `sink_dev` receives 512*512 floats, operands as for lmh_calib_mfma; `*flops` (host, optional) the flops of the launch. */
int lmh_calib_mix(void *sink_dev, const void *operands_dev, size_t operand_bytes, int iters, int mix, int waves_per_simd,
                  double *flops, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LUMINAL_HIP_CALIB_H */
