/*
 * ferrum_hip_probe.h -- measurement kernels of the MI355X (gfx950) backend.
 *
 * None of these has a counterpart in Ferrum: they are launched by the benchmark only, to show
 * what the device delivers with no operator attached, and are kept out of ferrum_hip.h so that
 * the operator surface a `src/hip` backend binds stays the reference's.  They live in the same
 * shared library and follow the conventions of ferrum_hip.h (fh_status, the device's stream).
 */
#ifndef FERRUM_HIP_PROBE_H
#define FERRUM_HIP_PROBE_H

#include "ferrum_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Reads every byte of a resident matrix with 128-bit loads and writes nothing: the HBM rate
 * a streaming kernel is compared with.  The tuning key `probe_read_form` picks the launch shape:
 * 100 x threads per workgroup + loads per lane (25604, 25608, 25616, 51204, 51208, 102404,
 * 102408), + 1000000 for LDS-direct loads (1025608, 1025616, 1051208); 0 = 256 threads x 8. */
fh_status fh_probe_read(fh_device* device, const fh_qmatrix* weight);

/* `groups` workgroups of four waves, each wave issuing `iterations` rounds of eight independent
 * matrix instructions from registers; *flops receives the floating-point operations of the
 * launch.  shape 0: v_mfma_f32_16x16x32_f16, shape 1: v_mfma_f32_32x32x16_f16, both on small
 * integer operands; shape 2: v_mfma_f32_32x32x16_f16 on pseudo-random f16 operands of
 * magnitude 0.5 .. 2 (different per lane), which is what a GEMM on random data feeds the
 * matrix cores and what sets their clock when the whole chip multiplies. */
fh_status fh_probe_mfma(fh_device* device, uint32_t shape, uint32_t groups, uint32_t iterations,
                        double* flops);

/* `groups` workgroups of eight waves, two per SIMD: waves 0..3 issue `iterations` x 8
 * v_mfma_f32_32x32x16_f16 when `mfma` is set, waves 4..7 `iterations` x `valu_rounds` x 8
 * v_fma_f32 when `valu_rounds` is not zero; timing the three combinations shows whether the
 * two kinds of arithmetic overlap on a SIMD. */
fh_status fh_probe_coissue(fh_device* device, uint32_t groups, uint32_t iterations, uint32_t mfma,
                           uint32_t valu_rounds);

#ifdef __cplusplus
}
#endif
#endif /* FERRUM_HIP_PROBE_H */
