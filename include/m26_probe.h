/* Measurement aids of the gfx950 expert-FFN library. No counterpart in the reference: its benchmark
 * prices kernels against measured device rates as well as nominal ones
 * (crates/mimo26-expert/docs/expert-gemm.md:444-451); these two entries measure, on the GPU the
 * library runs on, the two rates the FFN is priced against. Both allocate their own buffers, run on
 * `stream` (NULL = the default stream), time with events and return 0, or 1 for a bad argument and
 * 2 for a runtime error with a message in `err`. */
#ifndef M26_PROBE_H
#define M26_PROBE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Streams `bytes` (a multiple of 1 MiB, at least 64 MiB, far beyond the caches) `reps` times with
 * 16-byte streaming loads, the access the decode schedule makes for weights; *gbps = bytes read per
 * second / 1e9 of the best repetition over three launch shapes. */
int m26p_read_bandwidth(uint64_t bytes, int reps, void* stream, double* gbps, char* err, size_t errlen);

/* Issues nothing but the block-scaled MFMA the GEMMs use (v_mfma_scale_f32_16x16x128_f8f6f4, FP4
 * weights x FP8 activations, 32 independent accumulators per wave, operands in registers, varied
 * bits) from two waves per SIMD; *tflops = 2 * 16 * 16 * 128 flops per instruction per second / 1e12
 * of the best repetition. */
int m26p_mfma_rate(int iters, int reps, void* stream, double* tflops, char* err, size_t errlen);

#ifdef __cplusplus
}
#endif
#endif
