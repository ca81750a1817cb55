/* arcq_probe.h -- MEASUREMENT ONLY: the C ABI of libarcq_probe.so, a handful of plain copy kernels.
 *
 * Not part of the drop-in boundary (include/arcq.h) and not loaded by the operators: bench.py times these
 * kernels on the bytes of the headline quantizer launch to report what any single launch of that size reaches
 * on the box, and the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are calibrated on them.  No counterpart in
 * the reference.
 */
#ifndef ARCQ_PROBE_H_
#define ARCQ_PROBE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes (the values of include/arcq.h's arcq_status for the same conditions) */
enum { ARCQ_PROBE_OK = 0, ARCQ_PROBE_ERR_NULL = 1, ARCQ_PROBE_ERR_SHAPE = 2, ARCQ_PROBE_ERR_ALIGN = 4, ARCQ_PROBE_ERR_LAUNCH = 5 };

/*
 * Reads bytes_in from src and writes the first bytes_out of them to dst (multiples of 16, bytes_out <=
 * bytes_in, 16-byte aligned pointers): one 16-byte load in flight per thread (variant 0 below).
 */
int arcq_stream_probe(const void *src, void *dst, size_t bytes_in, size_t bytes_out, void *stream);

/*
 * The same copy with other launch shapes: 2, 4 or 8 independent loads in flight per thread, non-temporal
 * loads and stores, as many workgroups as the chip holds or exactly one round of threads, or LDS-direct
 * loads.  arcq_stream_probe_variants() is their number; an unknown variant is ARCQ_PROBE_ERR_SHAPE.
 */
int arcq_stream_probe_variant(const void *src, void *dst, size_t bytes_in, size_t bytes_out, int variant, void *stream);
int arcq_stream_probe_variants(void);

/*
 * Register-only matrix-pipe loop on all 256 CUs (one workgroup per CU, waves_per_simd = 1 or 2 waves on every
 * SIMD): what the MFMA units sustain on given operand bits without loads, LDS traffic or barriers.
 *   kind  0: v_mfma_scale_f32_32x32x64_f8f6f4 on FP4 operands with E8M0 block scales (the MXFP4 GEMM's instruction)
 *         1: v_mfma_f32_32x32x16_f16 (what NVFP4 decodes to), 2: v_mfma_f32_32x32x16_bf16 (the bf16 baseline)
 *   src   4096 32-bit words on the device that fill the operand registers: the sustained rate depends on them
 *         (zeros, random bits, fp16 values with three mantissa bits ...), the chip lowers its clock under load
 *   out   256 * 512 floats on the device (keeps the arithmetic alive)
 * arcq_mfma_rate_probe_flops: floating-point operations one such launch performs.
 */
int arcq_mfma_rate_probe(int kind, int waves_per_simd, int iters, const void *src, void *out, void *stream);
double arcq_mfma_rate_probe_flops(int kind, int waves_per_simd, int iters);

#ifdef __cplusplus
}
#endif
#endif /* ARCQ_PROBE_H_ */
