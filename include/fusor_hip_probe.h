/* fusor_hip_probe.h - measurement probes of libfusor_hip.so.
 *
 * These entry points have no counterpart in the reference and are not part of the operator boundary
 * (include/fusor_hip.h): they are what a benchmark prices the kernels against on the device it runs on - the cost of a
 * launch, of a plain streaming read, and the rates of the matrix cores, the LDS and the L2.  A binding of the boundary
 * does not need them. */
#ifndef FUSOR_HIP_PROBE_H
#define FUSOR_HIP_PROBE_H

#include "fusor_hip.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* An empty kernel of `workgroups` x `threads`,
 * and a plain streaming read of `bytes` (a multiple of 16384) from src_dev.  A benchmark prices the matvec kernels
 * against what these cost on the same device in the same launch pattern. */
fh_status fh_probe_empty(fh_device *dev, int32_t workgroups, int32_t threads);
fh_status fh_probe_read(fh_device *dev, const void *src_dev, size_t bytes);
/* What the device sustains under three patterns the kernels are built from; blocking, every call measures itself.
 *   kind 0: dense v_mfma_f32_32x32x16_f16, a = wavefronts per SIMD (1, 2), b = iterations of four MFMAs:
 *           out4[0] = TFLOP/s, out4[1] = microseconds.
 *   kind 1: ds_read_b128, eight reads in flight per wavefront, a = wavefronts per compute unit (4, 8, 16),
 *           b = address pattern (0 linear; MFMA operand addressing with 1 no swizzle, 2 row & 7, 3 the tile kernels'):
 *           out4[0] = bytes per ns and compute unit, out4[1] = bytes per shader clock and compute unit.
 *   kind 2: 16 wavefronts per compute unit, a = 0 all read a shared 256 KB region (L2 hits), 1 all stream 512 KB each,
 *           2 even ones the first and odd ones the second; src_dev = 256 KB + compute units x 16 x 512 KB:
 *           out4[0] / out4[1] = bytes per ns and compute unit from the L2 / from memory. */
fh_status fh_probe_device(fh_device *dev, int32_t kind, int32_t a, int32_t b, const void *src_dev, size_t src_bytes,
                          double *out4);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif

#endif /* FUSOR_HIP_PROBE_H */
