/* C ABI of the coordinator-side kernels that sit directly upstream and downstream of the routed-expert
 * FFN: routing, the wire quantizer, the request-frame fill, the rank sum and the residual add.
 * Plain pointers and sizes; every pointer is a device pointer; `stream` is a hipStream_t (or null).
 * Return value: 0 on success, otherwise the hipError_t of the failed launch or 1 for a bad argument
 * (the reference returns cudaError_t, where cudaErrorInvalidValue is 1 as well).
 *
 * Each entry names the reference interface it replaces (paths relative to the reference repository;
 * the Rust side binds them in crates/mimo26-coordinator/src/dforward.rs:33-101 and
 * crates/mimo26-attn/src/lib.rs).
 */
#ifndef M26C_GLUE_H
#define M26C_GLUE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* crates/mimo26-coordinator/kernels/glue.cu:76-124,252-261 (CPU: src/router.rs:41-80).
 * Per row: FP64 sigmoid of the FP32 logits, selection of top_k by (score + bias) descending with ties
 * to the lower expert id, weights = unbiased scores over their sum (FP64, summed in selection order),
 * rounded to FP32. n_experts <= 1024 and a multiple of 32, 1 <= top_k <= min(n_experts, 64). */
int m26c_router_topk(const float* logits, const float* bias, int rows, int n_experts, int top_k, int* idx_out,
                     float* w_out, void* stream);

/* crates/mimo26-coordinator/kernels/glue.cu:126-143,263-268 (CPU: src/wire.rs:83-108).
 * Per 32 values: s = 0 for an all-zero block else clamp(ceil(log2(amax / 448)) + 127, 0, 254);
 * scale_inv = 2^(127 - s). */
int m26c_quant_scales(const float* x, long n_blocks, unsigned char* scales, float* scale_inv, void* stream);

/* crates/mimo26-attn/kernels/kv_cache_fp8.cu:161-178 (CPU: crates/mimo26-coordinator/src/wire.rs:53-78,
 * crates/mimo26-load/src/e4m3.rs:50-81). payload[i] = E4M3 of x[i] * scale_inv[i / 32], nearest with
 * ties to the larger magnitude, saturating at 448, NaN -> 0. */
int m26_quantize_hidden_fp8(const float* x, const float* scale_inv, uint8_t* payload, int64_t n_elem, void* stream);

/* No counterpart as one call in the reference: the two entries above fused, one pass over x, rows of
 * `cols` values (a multiple of 32), payload and scale rows written at their own pitches (4224 / 4224
 * with scales = payload + cols writes request-frame rows in place). Same bytes as the pair. */
int m26c_quantize_hidden(const float* x, long rows, int cols, uint8_t* payload, size_t payload_pitch, uint8_t* scales,
                         size_t scales_pitch, void* stream);

/* crates/mimo26-coordinator/kernels/glue.cu:309-348. Writes the request frame's route entries
 * (12 bytes each: row u32, expert u32, weight f32 bits; t * topk of them) and its hidden rows (hid
 * payload bytes then hid / 32 scale bytes, at `pitch`). hid must be a multiple of 256; payload 16-byte,
 * scales and hidden 8-byte and routes 4-byte aligned, pitch a multiple of 8 (a request frame's hidden rows
 * start on 8-byte boundaries only); anything else returns 1. */
int m26c_frame_fill(const int* idx, const float* wts, const uint8_t* payload, const uint8_t* scales, int t, int topk,
                    int hid, uint8_t* routes, uint8_t* hidden, int pitch, void* stream);

/* crates/mimo26-coordinator/kernels/glue.cu:198-213,270-276 (CPU: crates/mimo26-wire/src/l4.rs
 * CoordinatorSum). out = ((((0 + p0) + p1) + p2) + p3) on the BF16 rows of the four ranks, FP32,
 * no fused operations. */
int m26c_rank_sum_bf16(const uint16_t* p0, const uint16_t* p1, const uint16_t* p2, const uint16_t* p3, float* out,
                       long n, void* stream);

/* crates/mimo26-coordinator/kernels/glue.cu:240-245. h[i] += a[i] (the residual add). */
int m26c_add_inplace(float* h, const float* a, long n, void* stream);

/* crates/mimo26-coordinator/kernels/glue.cu:215-221,277-282. FP32 -> BF16, round to nearest even. */
int m26c_f32_to_bf16(const float* x, uint16_t* y, long n, void* stream);

#ifdef __cplusplus
}
#endif
#endif
