/* C ABI of the gfx950 routed-expert FFN (B1, numerical mode E-W4A8-v1).
 *
 * The first six entry points are the ones the reference's Rust expert-rank daemon binds
 * (crates/mimo26-spark/src/b1.rs:21-49) and its CUDA unit defines
 * (crates/mimo26-spark/kernels/b1_serve.cu:214-574): same names, argument order and meaning,
 * same return codes. The rest are extensions for one-GPU operation (full intermediate,
 * device-resident inputs, 8,192-row calls) and for stage-level parity tests.
 *
 * Return codes (b1_serve.cu:315-317, 365-368, 551-562): 0 ok; 1 bad handles / rows / pitch;
 * 2 HIP runtime error; 3 invalid routes (id, residency, weight, duplicate expert in a token);
 * 4 device numerical or metadata fault. `err` receives a NUL-terminated message (truncated to
 * errlen). Outputs are invalid on a nonzero return. No exceptions, no aborts.
 *
 * Threading: one scratch = one call in flight; handles may move between threads but are not
 * shared (b1.rs:59-61,97-98).
 */
#ifndef M26S_B1_H
#define M26S_B1_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct m26s_b1_layer m26s_b1_layer;
typedef struct m26s_b1_scratch m26s_b1_scratch;

/* ---- the reference's expert-rank ABI ------------------------------------------------------ */

/* b1_serve.cu:218-265. canonical_dev: DEVICE buffer of exactly 256 * 3,342,336 bytes, one
 * quarter-slice image v2 per expert in expert-id order, for TP4 rank `rank` (0..3). The layer
 * keeps its own permuted copy; the caller may free canonical_dev on return. */
int m26s_b1_layer_new(const uint8_t* canonical_dev, uint64_t canonical_bytes, uint32_t rank,
                      m26s_b1_layer** out, char* err, size_t errlen);
/* b1_serve.cu:268. 1 when every weight scale byte lies in [2, 252]. A layer for which this is 0 is
 * served all the same: its calls take the conforming arm (each weight decoded by the format's rule,
 * min(s, 254) and saturation at +-FLT_MAX included, then multiplied; the counterpart of the reference's
 * decode-then-fmaf arm, crates/mimo26-expert/kernels/b1/grouped.cu:42-67), far slower than the matrix
 * pipe. Real checkpoints hold scale bytes 118..125 and never take it. */
int m26s_b1_layer_all_normal(const m26s_b1_layer* layer);
/* b1_serve.cu:270-276. */
void m26s_b1_layer_free(m26s_b1_layer* layer);
/* b1_serve.cu:278-291. Owns one stream, its events and grow-only device buffers. */
int m26s_b1_scratch_new(m26s_b1_scratch** out, char* err, size_t errlen);
/* b1_serve.cu:293-302. */
void m26s_b1_scratch_free(m26s_b1_scratch* scratch);
/* b1_serve.cu:312-572. HOST pointers. payload: `rows` rows of 4096 E4M3 bytes at payload_pitch;
 * scales: rows of 128 UE8M0 bytes at scales_pitch (4096 / 128 for separate arrays, 4224 for both
 * when read in place from a request frame); ids / weights: [rows*8] token-major top-8;
 * bf16_out: [rows*4096] BF16 bits. ms (8 floats or NULL): [0] upload + plan, [1] GPU compute,
 * [2] download + checks, [3] group count, [4..7] FC1 (with the fused intermediate quantizer),
 * 0, FC2, reduce. Synchronous. rows in 1..8192 (the reference stops at 4096). */
int m26s_b1_ffn(const m26s_b1_layer* layer, m26s_b1_scratch* scratch, const uint8_t* payload,
                size_t payload_pitch, const uint8_t* scales, size_t scales_pitch, const int32_t* ids,
                const float* weights, uint32_t rows, uint16_t* bf16_out, float* ms, char* err,
                size_t errlen);

/* ---- extensions: one GPU holds the whole intermediate -------------------------------------- */

/* The four TP4 rank pools of one layer (each exactly what m26s_b1_layer_new takes for its rank)
 * fused into one layer with intermediate 2048: gate/up rows 512*r.. and the matching K columns
 * of down come from rank_images_dev[r]. The FFN then returns the BF16 rounding of the complete
 * FP32 sum (one rounding) instead of four per-rank roundings added afterwards. */
int m26s_b1_layer_new_full(const uint8_t* const rank_images_dev[4], uint64_t bytes_each,
                           m26s_b1_layer** out, char* err, size_t errlen);
/* Intermediate columns the layer holds: 512 (one rank) or 2048 (full). */
uint32_t m26s_b1_layer_intermediate(const m26s_b1_layer* layer);

/* The prepared pool of a layer, for persisting it or checking it: 256 images of *image_bytes each
 * (3,342,336 for one rank's share, four times that for a full layer) in expert-id order, device
 * memory owned by the layer. *layout_tag names the byte order (the counterpart of the reference's
 * prepared tag, crates/mimo26-expert/kernels/b1/prepared.cuh:16-31): M26S_B1_LAYOUT_G950_V2 is
 * the operand order of gfx950's v_mfma_scale_f32_16x16x128_f8f6f4 this library writes; a persisted
 * pool carrying any other tag must be prepared again from the canonical images. Returns 0, or 1
 * for a null argument. */
#define M26S_B1_LAYOUT_G950_V2 0x47393502u /* "G95" 0x02 */
int m26s_b1_layer_view(const m26s_b1_layer* layer, const uint8_t** prepared_dev, uint64_t* image_bytes,
                       uint32_t* layout_tag);

/* A scratch that launches on the caller's HIP stream (hipStream_t passed as void*; NULL is the
 * default stream) instead of creating its own, so the caller can bracket calls with its own
 * events. The stream is not owned. */
int m26s_b1_scratch_new_on(void* hip_stream, m26s_b1_scratch** out, char* err, size_t errlen);
/* The hipStream_t (as void*) the scratch launches on, its own or the caller's: whoever writes the
 * inputs of an enqueued call on the device has to order those writes before the call, which work on
 * this stream is and work on another stream is not. */
void* m26s_b1_scratch_stream(const m26s_b1_scratch* scratch);

/* m26s_b1_ffn with DEVICE pointers for every array: no PCIe in the call. payload_dev must be
 * 16-byte aligned with payload_pitch % 16 == 0; scales_dev 4-byte aligned with
 * scales_pitch % 4 == 0. partial_dev (optional) receives the FP32 sum before the BF16 rounding
 * (the reference keeps it internally, kernels/b1/route_reduce.cuh:11-16). Synchronous. */
int m26s_b1_ffn_dev(const m26s_b1_layer* layer, m26s_b1_scratch* scratch, const uint8_t* payload_dev,
                    size_t payload_pitch, const uint8_t* scales_dev, size_t scales_pitch,
                    const int32_t* ids_dev, const float* weights_dev, uint32_t rows,
                    uint16_t* bf16_out_dev, float* partial_dev, float* ms, char* err, size_t errlen);
/* Same work, enqueued only: returns after the launches. Faults of every call since the last
 * m26s_b1_scratch_sync accumulate and are reported there as the OR of the calls' fault words, routes
 * before numerics (3 before 4). What a fault stops: a rejected plan stops every stage of its own call and
 * of every later call enqueued before that sync; a fault of FC1 or of the quantizer stops FC2 and the
 * combine of its own and of later calls, but not their plan or FC1; an FC2 or combine fault stops
 * nothing that follows. After a nonzero sync every output written since the previous sync is invalid. The
 * call puts its kernels on the stream and nothing else (no events: the synchronous entries record theirs
 * only when ms is given). */
int m26s_b1_ffn_enqueue(const m26s_b1_layer* layer, m26s_b1_scratch* scratch, const uint8_t* payload_dev,
                        size_t payload_pitch, const uint8_t* scales_dev, size_t scales_pitch,
                        const int32_t* ids_dev, const float* weights_dev, uint32_t rows,
                        uint16_t* bf16_out_dev, float* partial_dev, char* err, size_t errlen);
/* Waits for the scratch's stream and decodes the fault words (return codes as above). */
int m26s_b1_scratch_sync(m26s_b1_scratch* scratch, char* err, size_t errlen);

/* No counterpart in the reference. For callers that cannot allocate: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc. m26s_b1_ffn_enqueue without a scratch handle: every
 * per-call array (plan, intermediate, per-route rows, count and fault words) lies in a fixed array of 32 MiB
 * inside the library's device image, which each GPU the library runs on holds until the process ends, and
 * the call makes no allocation of any kind. Limits: rows in 1..128 (the decode / verify batch); more rows
 * return 1 with a message. Launches on `hip_stream` (hipStream_t as void*, NULL = the default stream) and
 * returns without waiting: 0, 1 for bad arguments, 2 for a runtime error. status_dev (8 uint32 of device
 * memory, or NULL) receives the call's words {group count, plan fault, chunk count, fc1 fault, quantizer
 * fault, lowest faulting block, fc2 fault, reduce fault} behind its last kernel: read them after the
 * stream has run; bf16_out_dev is valid when words 1, 3, 4, 6 and 7 are zero (decoded as m26s_b1_ffn's
 * return codes 3 and 4). All calls on one GPU share the one array, which keeps the last call's contents
 * (each call's first kernel clears the words it needs at zero and rewrites the constants the array holds,
 * so there is no initialising call that a graph capture could swallow: the first call on a GPU may be
 * captured, and may come on any stream): calls that overlap in time on one GPU race, also from different
 * streams or threads. Pointers, pitches and alignments as m26s_b1_ffn_enqueue. */
int m26s_b1_ffn_static(const m26s_b1_layer* layer, const uint8_t* payload_dev, size_t payload_pitch,
                       const uint8_t* scales_dev, size_t scales_pitch, const int32_t* ids_dev,
                       const float* weights_dev, uint32_t rows, uint16_t* bf16_out_dev, uint32_t* status_dev,
                       void* hip_stream, char* err, size_t errlen);

/* ---- stage-level entry points (parity tests and diagnostics) ------------------------------- */

/* Stage 1 alone, on DEVICE arrays: the reference planner's outputs
 * (kernels/b1/group_plan.cuh:10-26). capacity is 256, 2048, 4096 or 8192 rows; the arrays hold
 * capacity*8 entries (groups: capacity*8 records of 76 bytes) and every slot is rewritten as
 * the serial planner does; on invalid routes only *fault_dev (the planner's Status) is set.
 * resident_dev: 256 bytes of 0/1. Synchronous; returns 0, 1 or 2 (never 3: read the fault). */
int m26s_b1_plan_dev(const int32_t* ids_dev, const float* weights_dev, uint32_t rows, uint32_t capacity,
                     const uint8_t* resident_dev, int32_t* inverse_dev, int32_t* original_routes_dev,
                     float* grouped_weights_dev, void* groups_dev, uint32_t* group_count_dev,
                     uint32_t* fault_dev, char* err, size_t errlen);
/* Quantizer v1 alone (kernels/b1/quant_v1.cuh:84-100): consecutive K32 blocks of FP32 ->
 * E4M3FN bytes + one scale byte + one fault word per block (0 ok, 1 nonfinite, 2 reconstruction
 * overflow; a faulting block's bytes are left untouched). Synchronous. */
int m26s_b1_quantize_dev(const float* h_dev, uint64_t elements, uint8_t* payload_dev, uint8_t* scales_dev,
                         uint32_t* faults_dev, char* err, size_t errlen);
/* Combine alone (kernels/b1/route_reduce.cu:61-124): y [rows][8][4096] FP32 unweighted, weights
 * [rows][8] -> FP32 sum (optional) and BF16 bits; *fault_dev nonzero on a numerical fault. */
int m26s_b1_reduce_dev(const float* y_dev, const float* weights_dev, uint32_t rows, float* partial_dev,
                       uint16_t* bf16_dev, uint32_t* fault_dev, char* err, size_t errlen);

/* With taps on, the next FFN calls also keep FP32 gate / up / h of every grouped row. */
void m26s_b1_scratch_set_taps(m26s_b1_scratch* scratch, int on);
/* Switches of a scratch, for the calls made on it afterwards. Returns 0, 1 for a bad handle or option, 2 for
 * a runtime error.
 *   TAPS              as m26s_b1_scratch_set_taps.
 *   FUSED_COMBINE     the router-weighted combine runs inside FC2 instead of as a launch of its own behind it
 *                     (crates/mimo26-spark/kernels/b1_serve.cu:502-515 launches it): the wave that writes a
 *                     token's eighth per-route row sums the eight, in slot order, so both forms give the same
 *                     bits (tested). Off by default: measured on MI355X it is never the faster form (level at
 *                     16 tokens of one rank's share, 2 % behind at 128 tokens, 5 % at 8192: a wave's waits for
 *                     its stores, its count and the rows it sums are paid with nothing else to run). Layers on
 *                     the conforming arm always combine separately.
 *   BF16_ROUTE_ROWS   the reference's opt-in MIMO26_B1_Y=bf16 (b1_serve.cu:98-143,400-405; the store rule of
 *                     crates/mimo26-expert/kernels/b1/connected.cu:41-44): FC2 keeps its per-route rows as
 *                     BF16 bits instead of FP32 and the combine widens them. A numerical-mode change, never
 *                     the default; a scratch is created with it on when the environment holds MIMO26_B1_Y=bf16.
 *                     View 7 then holds uint16 rows.
 *   SCOPE_TIMING      the timed entries record one interval over FC1 + SwiGLU + quantizer + FC2 with no event between
 *                     the stages, the scope the reference's bandwidth gate times between its two events
 *                     (crates/mimo26-expert/tests/b1_core/bench_connected.cuh:66-81): ms[4] is then that interval
 *                     and ms[6] is 0. An event is one more packet between two dependent kernels, about 3 us.
 *   GUARDS            test aid (the counterpart of crates/mimo26-expert/tests/b1_core/primitive.cu:23-40):
 *                     every internal array is followed, and the first preceded, by at least 256 bytes of 0xa5,
 *                     written before each call and read back by m26s_b1_scratch_check_guards. */
enum { M26S_B1_OPT_TAPS = 0, M26S_B1_OPT_FUSED_COMBINE = 1, M26S_B1_OPT_BF16_ROUTE_ROWS = 2, M26S_B1_OPT_GUARDS = 3,
       M26S_B1_OPT_SCOPE_TIMING = 4 };
int m26s_b1_scratch_set_option(m26s_b1_scratch* scratch, int option, int value);
/* Waits for the scratch's stream and reads every red zone back: 0 intact, 1 guards not enabled or no call made,
 * 2 runtime error, 4 a zone holds a byte other than 0xa5 (err names the zone and the offset). */
int m26s_b1_scratch_check_guards(m26s_b1_scratch* scratch, char* err, size_t errlen);
/* Device address and byte size of an internal buffer after a call. which: 0 inverse, 1 original
 * routes, 2 grouped weights, 3 groups, 4 meta words {group count, plan fault, chunk count, fc1
 * fault, quantizer fault, lowest faulting block, fc2 fault, reduce fault}, 5 intermediate payload
 * [groups*16][I], 6 its scales [groups*16][I/32], 7 y [rows*8][4096], 8/9/10 gate/up/h taps,
 * 11 chunks (16 bytes each: first group, groups, expert, zero), 12 the clock record of the last call that ran
 * the prefill-size schedule: four 64-bit words {shader-clock ticks, ticks of the fixed 100 MHz counter} over one
 * work item in the middle of the gate/up launch, then the same of the down launch (the ratio x 0.1 is the clock
 * in GHz the launch ran at; zeros before the first such call). Returns 0, or 1 for an unknown or unallocated buffer. */
int m26s_b1_scratch_view(const m26s_b1_scratch* scratch, int which, void** dev_ptr, size_t* bytes);
/* Plain copies for callers without a HIP binding of their own (synchronous). */
int m26s_b1_copy_to_host(void* dst_host, const void* src_dev, size_t bytes);
int m26s_b1_copy_to_device(void* dst_dev, const void* src_host, size_t bytes);
void* m26s_b1_device_alloc(size_t bytes);
void m26s_b1_device_free(void* dev_ptr);
/* Free and total bytes of the current GPU's memory (hipMemGetInfo): 0, 1 for a null argument, 2 for a runtime error. */
int m26s_b1_device_memory(size_t* free_bytes, size_t* total_bytes);

#ifdef __cplusplus
}
#endif
#endif
