/*
 * mnb_probe.h -- C entry points of libmnb_probe.so: diagnostics for the benchmark, NOT part of the operator's C ABI
 * (that is include/mnb_mi355x.h).  They have no counterpart in the reference: they measure what the device sustains
 * with the plainest kernels, so that the throughput of the real kernels can be read against it.  Every call
 * allocates device memory, runs for a few milliseconds and synchronises the device.  Return 0 on success, 1 on a HIP
 * error, 2 on an invalid argument.
 */
#ifndef MNB_PROBE_H_
#define MNB_PROBE_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MNB_PROBE_API __attribute__((visibility("default")))

/* GB/s of `launches` back-to-back kernels (one HIP graph) that each only read their own `bytes_per_launch` bytes of
 * device memory once: workgroups of `threads` threads (multiple of 64, at most 1024), every thread issuing
 * `loads_in_flight` (2, 4, 8, 16 or 32) independent 16-byte loads `batches` times; the grid covers the buffer.
 * The buffers are kept between calls with the same sizes (a sweep allocates once); MnbProbeRelease frees them. */
MNB_PROBE_API int MnbProbeReadBandwidth(size_t bytes_per_launch, int launches, int threads, int loads_in_flight,
                                        int batches, double* gb_per_s);
/* The same with every launch reading the SAME buffer: what a kernel of that size reaches when its data waits in the
 * Infinity Cache (bytes_per_launch well below 256 MB) instead of HBM. */
MNB_PROBE_API int MnbProbeReadBandwidthResident(size_t bytes_per_launch, int launches, int threads,
                                                int loads_in_flight, int batches, double* gb_per_s);
MNB_PROBE_API void MnbProbeRelease(void);

/* TFLOP/s of a loop of nothing but v_mfma_f32_32x32x16_f16 on every CU, with constant operands
 * (random_operands = 0) or random fp16 operands (1): the sustained matrix-core clock depends on operand toggling. */
MNB_PROBE_API int MnbProbeMfmaRate(int random_operands, double* tflops);
/* The same loop with the value class of each operand chosen (A = the first, B = the second source of the matrix
 * instruction): 0 the constant 1, 1 uniform in (-1, 1), 2 zero, 3 bell-shaped with variance 1 (activations),
 * 4 dequantised 4-bit weights (q - 8) * scale with a scale per column (what the prefill kernel feeds as B),
 * 5 the integers q - 8, 6 the raw halves 1024 + q (what the decode kernel feeds), 7 a 4-bit grid under one scale.
 * The instruction stream is the same for every class; only the operands' significant bits differ. */
MNB_PROBE_API int MnbProbeMfmaRateOperands(int a_class, int b_class, double* tflops);

/* Nanoseconds per "slot" of a loop that every wavefront of the chip runs (waves_per_simd = 1 or 2 wavefronts on each
 * SIMD): a slot is one v_mfma_f32_32x32x16_f16 (when with_mfma) followed by valu_per_mfma (0, 1, 2, 4, 8) independent
 * packed-fp16 multiply-adds; with lds_reads_per_two_mfma = 1 or 2 the matrix instruction's A operand comes from a
 * 16-byte-per-lane LDS read issued two slots earlier (one read per matrix instruction, or one per two).  Comparing (mfma only), (vector only) and (both) tells whether the two kinds of
 * instruction overlap on a SIMD or take turns. */
MNB_PROBE_API int MnbProbeIssueOverlap(int valu_per_mfma, int with_mfma, int waves_per_simd,
                                       int lds_reads_per_two_mfma, double* ns_per_slot);

/* Nanoseconds per step of the streaming kernel's instruction mix, run by waves_per_simd (1 or 2) wavefronts on every
 * SIMD: a step is 13 vector instructions that dequantise one 32-bit word of eight 4-bit weights into a matrix-core
 * operand and four v_mfma_f32_16x16x32_f16 that use it.  mode 0: the matrix instructions alone; 1: the vector
 * instructions alone; 2: the operand made right in front of its matrix instructions; 3: the next step's operand made
 * between the matrix instructions of the current one. */
MNB_PROBE_API int MnbProbeDequantMfma16(int mode, int waves_per_simd, double* ns_per_step);

/* The clock the shader engines run at while other work is on the chip: Start launches a single wavefront on a stream
 * of its own that watches the shader clock's cycle counter against the constant 100 MHz counter for sample_ms
 * milliseconds and returns at once; Finish waits for it and gives the ratio in GHz and the time actually sampled.
 * Launch the kernels to be observed between the two calls. */
MNB_PROBE_API int MnbProbeShaderClockStart(double sample_ms);
MNB_PROBE_API int MnbProbeShaderClockFinish(double* ghz, double* sampled_ms);

#ifdef __cplusplus
}
#endif
#endif /* MNB_PROBE_H_ */
