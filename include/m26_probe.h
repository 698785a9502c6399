/* Measurement aids of the gfx950 expert-FFN library. No counterpart in the reference: its benchmark
 * prices kernels against measured device rates as well as nominal ones
 * (crates/mimo26-expert/docs/expert-gemm.md:444-451); these entries measure, on the GPU the
 * library runs on, the two rates the FFN is priced against. All allocate their own buffers, run on
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

/* The same kernel `launches` times back to back (2..1000), nothing between the launches but an event: the rate of the
 * first and of the last launch, and the shader clock each of them ran at (GHz: a workgroup in the middle of the grid
 * reads the shader-clock counter and the fixed 100 MHz counter around its loop). What the part holds when the load
 * lasts, and the clock that goes with it: the power management lowers the clock under load, by an amount that
 * depends on what the load is. */
int m26p_mfma_sustained(int iters, int launches, void* stream, double* tflops_first, double* tflops_last,
                        double* ghz_first, double* ghz_last, char* err, size_t errlen);

#ifdef __cplusplus
}
#endif
#endif
