/*
 * cahel_probe.h -- C-ABI of libcahel_probe.so: micro-benchmarks of instruction issue rates on the GPU.
 *
 * Measurement support for bench.py (the VALU side of the roofline is priced against these rates); not part of the
 * engine's interface (include/cahel_hip.h) and not needed to use it.  Nothing here has a counterpart in the
 * reference.  Return values: 0 on success, a positive hipError_t value when the HIP runtime failed, -1 for invalid
 * arguments.  `stream` is a hipStream_t passed as void* (NULL = the null stream).
 */
#ifndef CAHEL_PROBE_H
#define CAHEL_PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HE_OK 0
#define HE_E_INVALID_ARGUMENT (-1)

/* Measures the issue rate of full-rate FP64 vector instructions on this GPU (lane-operations per second, 8
 * independent fused multiply-add chains per lane over `blocks` workgroups of 256 lanes, `iters` x 64 operations per
 * lane): the peak that the VALU roofline of the FP64 back end is priced against.  Measurement support; allocates a
 * 64-byte buffer and two events for the duration of the call. */
int he_probe_fp64_issue_rate(uint32_t blocks, uint32_t iters, double *lane_ops_per_second, void *stream);

/* The same measurement for the other instruction kinds that the kernels' bounds are argued with (`kind` below): 8
 * independent chains per lane, `iters` x 64 operations per lane; the result counts lane-operations (multiply-adds for
 * the matrix kinds: one v_mfma_f64_16x16x4_f64 is 1,024 of them per wave, i.e. 16 per lane; HE_PROBE_MFMA_F64_WITH_FMA
 * issues as many multiply-adds on the matrix instruction as on v_fma_f64 and reports their sum, so a result equal to
 * either kind alone means that the two do not run side by side).  Measurement support, as above. */
enum {
    HE_PROBE_FMA_F64 = 0,           /* v_fma_f64 */
    HE_PROBE_MAD_U64_U32 = 1,       /* v_mad_u64_u32: 32 x 32 + 64 -> 64 */
    HE_PROBE_MUL_LO_U32 = 2,        /* v_mul_lo_u32 */
    HE_PROBE_ADD_U32 = 3,           /* v_add_u32 */
    HE_PROBE_MFMA_F64 = 4,          /* v_mfma_f64_16x16x4_f64 alone */
    HE_PROBE_MFMA_F64_WITH_FMA = 5  /* the matrix instruction interleaved with v_fma_f64, equal work on each */
};
int he_probe_issue_rate(uint32_t kind, uint32_t blocks, uint32_t iters, double *lane_ops_per_second, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CAHEL_PROBE_H */
