/*
 * tsx_aids.h -- entry points of the MEASUREMENT build of the library (libtsx_hip_aids.so, compiled with
 * -DTSX_MEASUREMENT_AIDS by `python -m tennis_amd.build --aids`).  They have no counterpart in the reference and
 * are not part of the product ABI (include/tsx_hip.h): the product library carries neither them nor the phase
 * stamps inside its kernels.
 */
#ifndef TSX_AIDS_H
#define TSX_AIDS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Launches `blocks` workgroups of 4 wavefronts, each issuing iters * 8 register-only v_mfma_i32_32x32x32_i8
 * (65536 ops each) on operands read once from operands_dev (32 KiB).  Timed by the caller, it gives the int8 MFMA
 * rate this part sustains for the given operand data -- the practical ceiling of the contraction kernels (clocks
 * drop under the power of random operands, so it is well below the nominal peak).
 * ops = blocks * 4 * iters * 8 * 65536. */
int tsx_probe_mfma_i8(const void *operands_dev, int32_t iters, int32_t blocks, int32_t *sink_dev, void *stream);

/* While a buffer is set (NULL switches it off; process-wide), every wavefront of the weight-stationary int8
 * convolution kernel writes (wall clock at 100 MHz, shader clock) pairs at its phase boundaries, at
 * buffer[((workgroup * 8 + wavefront) * 24 + k) * 2 ...]:
 *   multiplying wavefronts 0-3: k = 0 kernel entry, 1 weights in registers and first rows in LDS, 2 last fragment done;
 *   serving wavefronts 4-7:     k = 0 kernel entry, 1 ring filled, 2 last round done, 3 stores issued, 4 stores left.
 * (Compiled with -DTSX_MEASUREMENT_AIDS=2 the kernel also stamps every fragment / round, between k = 1 and the
 * phase behind it; those stamps slow the loop by a quarter.)  Wavefronts whose slot lies beyond `bytes` write nothing. */
int tsx_debug_phase_stamps(void *buffer_dev, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif
