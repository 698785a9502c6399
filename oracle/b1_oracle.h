/* CPU restatement of the reference's routed-expert FFN ("B1", lattice E-W4A8-v1).
 *
 * TEST INFRASTRUCTURE ONLY. This library is the checker for the HIP path; nothing the
 * product ships may link, import or call it. Only tests, the smoke check and the
 * benchmark's cpu_baseline leg use it.
 *
 * Every function cites the reference text it restates (paths relative to the reference
 * repository root). Parity pins per function are listed in b1_oracle.c's header.
 */
#ifndef B1_ORACLE_H
#define B1_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum {
    ORC_HIDDEN = 4096,
    ORC_EXPERTS = 256,
    ORC_TOPK = 8,
    ORC_RANK_I = 512,          /* one TP4 rank's share of the intermediate */
    ORC_IMAGE_BYTES = 3342336, /* quarter-slice image v2 */
    ORC_GATE_PAYLOAD = 0,
    ORC_GATE_SCALES = 1048576,
    ORC_UP_PAYLOAD = 1114112,
    ORC_UP_SCALES = 2162688,
    ORC_DOWN_PAYLOAD = 2228224,
    ORC_DOWN_SCALES = 3276800
};

/* Planner status codes, numbered as the reference's Status enum. */
enum { ORC_OK = 0, ORC_VERSION, ORC_GEOMETRY, ORC_SIZE, ORC_POINTER, ORC_OVERLAP, ORC_BOUNDS,
       ORC_METADATA, ORC_NONFINITE };

/* --- codecs ---------------------------------------------------------------------- */
/* MXFP4 element -> IEEE-754 binary32 bits. */
uint32_t orc_mxfp4_bits(uint32_t nibble, uint32_t scale_byte);
/* Whole row: payload [k/2] bytes (low nibble = even k), scales [k/32]. */
void orc_mxfp4_row(const uint8_t* payload, const uint8_t* scales, size_t k, float* out);
/* E4M3FN byte -> value (NaN for 0x7f / 0xff). */
float orc_e4m3_value(uint8_t code);
/* Activation rows: payload [rows][cols] at pitch, scales [rows][cols/32] at pitch -> f32.
 * Returns the number of elements that are NaN codes or carry a scale outside [105,247]
 * (those decode to NaN, as the reference's load path does). */
size_t orc_activation_decode(const uint8_t* payload, size_t payload_pitch, const uint8_t* scales,
                             size_t scales_pitch, size_t rows, size_t cols, float* out);
/* FP32 -> BF16 bits, round to nearest even (no NaN special-casing: callers fault first). */
uint16_t orc_bf16_rne(float v);

/* Wire input quantizer ("Q0"): f32 rows -> E4M3 payload + UE8M0 K32 scales. */
void orc_q0_quantize(const float* x, size_t rows, size_t cols, uint8_t* payload, uint8_t* scales);
/* The single-value encoder Q0 uses (nearest E4M3, ties to the larger magnitude). */
uint8_t orc_e4m3_encode_half_up(double v);

/* Intermediate quantizer v1 over consecutive K32 blocks. faults[b]: 0 ok, 1 nonfinite input,
 * 2 reconstruction overflow; a faulting block leaves its payload/scale bytes untouched.
 * Returns the number of faulting blocks. */
size_t orc_quant_v1(const float* h, size_t elements, uint8_t* payload, uint8_t* scales,
                    uint32_t* faults);

/* --- planner ----------------------------------------------------------------------- */
typedef struct {
    int32_t expert, rows, route_base;
    int32_t input_rows[16];
} orc_group; /* 76 bytes, the reference's Group */

/* Stable expert-major route plan. ids/weights are [rows*8] token-major; resident is 256 bytes
 * of 0/1. Output arrays hold capacity*8 entries each and are fully rewritten on success; on a
 * value fault only *fault is written. Returns the status, also stored in *fault. */
uint32_t orc_plan(uint32_t capacity, uint32_t rows, const int32_t* ids, const float* weights,
                  const uint8_t* resident, int32_t* inverse, int32_t* original_routes,
                  float* grouped_weights, orc_group* groups, uint32_t* group_count,
                  uint32_t* fault);

/* --- activation and combine --------------------------------------------------------- */
/* SwiGLU with the CPU reference's exp (binary64 exp rounded once to binary32). */
float orc_silu_up(float gate, float up);
/* Weight-once, slot-ordered FP32 combine + BF16. y is [rows][8][cols], w is [rows][8].
 * Returns 0, or ORC_NONFINITE on the first element that violates the finite/sign rules
 * (outputs then hold what was written before it). partial and bf16 may each be NULL. */
uint32_t orc_reduce(const float* y, const float* w, size_t rows, size_t cols, float* partial,
                    uint16_t* bf16);

/* The opt-in BF16 per-route mode: FC2's store rule (FP32 -> BF16 bits, round to nearest even by the integer
 * formula) and the combine over such rows [rows][8][cols] (no FP32 sum is kept). Returns 0 or 5. */
void orc_bf16_store_rows(const float* y, size_t n, uint16_t* out);
uint32_t orc_reduce_bf16y(const uint16_t* y16, const float* w, size_t rows, size_t cols, uint16_t* bf16);

/* --- expert FFN ---------------------------------------------------------------------- */
/* A layer's weights: `ranks` pools (1 = one TP4 rank's share, I = 512; 4 = all four rank
 * images, I = 2048), each 256 quarter-slice images back to back in expert-id order. */
typedef struct {
    const uint8_t* pool[4];
    uint32_t ranks;
} orc_layer;

/* W4A8 lattice FFN of one expert over `rows` activation rows (already gathered):
 * FP64 dots, FP32 at gate/up/h/y, v1 requantisation of h per K32 block, unweighted y.
 * Any of gate/up/h/mid_payload/mid_scales may be NULL. y is [rows][4096].
 * Returns 0, or a nonzero fault: 1 nonfinite at an FP32 boundary, 2 quantizer fault. */
uint32_t orc_expert_ffn(const orc_layer* layer, uint32_t expert, const uint8_t* x_payload,
                        size_t x_pitch, const uint8_t* x_scales, size_t xs_pitch, size_t rows,
                        float* gate, float* up, float* h, uint8_t* mid_payload,
                        uint8_t* mid_scales, float* y);

/* Whole layer, W4A8: plan, per-expert FFN, combine. Token t's row is x_payload + t*x_pitch.
 * y_routes (optional) receives the unweighted per-route outputs [rows*8][4096].
 * threads <= 0 means all hardware threads. Returns 0 or: 3 invalid routes, 4 numerical fault. */
uint32_t orc_layer_ffn(const orc_layer* layer, const uint8_t* x_payload, size_t x_pitch,
                       const uint8_t* x_scales, size_t xs_pitch, const int32_t* ids,
                       const float* weights, size_t rows, float* y_routes, float* partial,
                       uint16_t* bf16, int threads);

/* Whole layer, E-FP32: the reference's CPU merge-gate path (decoded f32 activations, per-MAC
 * weight decode, f32 accumulation in k order, silu(g)*u, no intermediate requantisation,
 * weighted slot-ordered f32 sum, BF16 RNE). */
uint32_t orc_layer_ffn_efp32(const orc_layer* layer, const uint8_t* x_payload, size_t x_pitch,
                             const uint8_t* x_scales, size_t xs_pitch, const int32_t* ids,
                             const float* weights, size_t rows, float* partial, uint16_t* bf16,
                             int threads);

int orc_hardware_threads(void);

/* ---- coordinator-side steps around the path ------------------------------------------------- */

/* Router selection over FP32 logits [rows][n_experts]: FP64 sigmoid, top_k by (score + bias)
 * descending with ties to the lower expert id, weights = unbiased scores over their sum taken in
 * selection order (FP64), rounded to FP32. */
void orc_router_topk(const float* logits, const float* bias, size_t rows, size_t n_experts, size_t top_k,
                     int32_t* idx, float* weights);
/* Q0's scale half: scale byte and 2^(127 - s) per K32 block. */
void orc_q0_scales(const float* x, size_t n_blocks, uint8_t* scales, float* scale_inv);
/* out = ((((0 + p0) + p1) + p2) + p3) over BF16 values, FP32 additions in that order. */
void orc_rank_sum_bf16(const uint16_t* p0, const uint16_t* p1, const uint16_t* p2, const uint16_t* p3,
                       float* out, size_t n);
/* FP32 -> BF16 round to nearest even, NaN -> 0x7fff (the conversion the reference's GEMM input cast uses). */
uint16_t orc_bf16_rne_nan(float v);

#ifdef __cplusplus
}
#endif
#endif
