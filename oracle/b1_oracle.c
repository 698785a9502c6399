/* CPU restatement of the reference's routed-expert FFN ("B1", lattice E-W4A8-v1).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path. Nothing shipped may call it.
 *
 * What pins each function (all checks live in tests/, CPU-only):
 *   orc_mxfp4_bits      - the reference's 64x64 pack/unpack golden file, its hand vector
 *                         (byte 0x71, scales 127/128), the closed form over all 16x256
 *                         pairs, and the compiled reference decoder where it builds.
 *   orc_e4m3_value      - the reference's 256-entry decode table.
 *   orc_q0_quantize     - brute force over every bf16 input against a direct
 *                         nearest-with-ties-to-larger search of the decode table, the
 *                         reference's stated vectors (codes encode to themselves,
 *                         7.5/512 -> 0x08, 2^-6 -> 0x08), and the ceil(log2) scale formula
 *                         evaluated on boundary neighbours.
 *   orc_quant_v1        - the compiled reference quantize_host (differential) where it
 *                         builds, the committed vectors it produced, the reference's edge
 *                         vectors, and an exact-rational referee.
 *   orc_plan            - the compiled reference plan_host where it builds, committed
 *                         vectors, and an independent stable sort.
 *   orc_reduce          - the compiled reference reduce_host where it builds, committed
 *                         vectors, and the reference's closed-form order / non-fused /
 *                         subnormal / BF16-midpoint vectors.
 *   orc_reduce_bf16y,
 *   orc_bf16_store_rows - identity with orc_reduce on the widened rows (a function pinned above, other
 *                         code), hand-worked sums with BF16 midpoints at the store and at the output, the
 *                         order witness (a sum that differs in any other slot order) and the fault cases.
 *   orc_silu_up         - the reference's four retained (g,u)->h witnesses and specials.
 *   orc_expert_ffn,
 *   orc_layer_ffn       - composition of the above; closed-form synthetic projections with
 *                         an exact integer dot, brute force on tiny shapes, rank-split
 *                         identity, M-prefix identity and mutation detectors.
 *   orc_layer_ffn_efp32 - structure check only against the W4A8 path (same routing, looser
 *                         numerics); it is a reported baseline, not a parity oracle.
 *   orc_router_topk     - the reference holds no vectors for it: a stable argsort of library
 *                         sigmoids (scipy expit), the tie rule on equal logits, bias selecting but
 *                         not weighting, a closed-form two-expert weight.
 *   orc_q0_scales       - closed form on amax = 448 * 2^e and its neighbours over the whole
 *                         exponent range, identity with orc_q0_quantize's scale bytes.
 *   orc_rank_sum_bf16   - sequential binary32 additions in numpy, data where another order
 *                         differs, and the 1 + 2^-24 + 2^-24 - 1 case a fused sum gets wrong.
 *   orc_bf16_rne_nan    - midpoint, signed-zero, infinity, NaN and subnormal vectors.
 *   prepared_g950       - (numpy, in b1_oracle.py) the prepared byte order of the gfx950 library as
 *                         a forward map; pinned by hand-worked coordinates of every region, by
 *                         being a bijection that keeps the byte multiset, and by the measured
 *                         operand order of the MFMA itself: the closed-form projections only
 *                         come out exact on the GPU if every byte sits where the instruction
 *                         reads it.
 */
#include "b1_oracle.h"
#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------------
 * Codecs
 * ---------------------------------------------------------------------------------------- */

static uint32_t f32_bits(float v) { uint32_t b; memcpy(&b, &v, 4); return b; }
static float bits_f32(uint32_t b) { float v; memcpy(&v, &b, 4); return v; }

/* crates/mimo26-expert/kernels/include/mimo26_expert_bits.h:29-40, spike/mxfp4.py:44-84:
 * value = codebook[nibble] * 2^(min(scale,254) - 127), saturated to +-FLT_MAX, zero keeps
 * its sign. Twice the codebook magnitudes are the integers below, so the value is
 * twice_mag * 2^(s - 128), which ldexpf forms exactly down to the subnormals. */
uint32_t orc_mxfp4_bits(uint32_t nibble, uint32_t scale_byte) {
    static const float twice_mag[8] = {0.f, 1.f, 2.f, 3.f, 4.f, 6.f, 8.f, 12.f};
    const uint32_t sign = (nibble & 8u) ? 0x80000000u : 0u;
    const float m = twice_mag[nibble & 7u];
    if (m == 0.f) return sign;
    const int s = scale_byte > 254u ? 254 : (int)scale_byte;
    float v = ldexpf(m, s - 128);
    if (!(v <= FLT_MAX)) v = FLT_MAX;
    return sign | f32_bits(v);
}

void orc_mxfp4_row(const uint8_t* payload, const uint8_t* scales, size_t k, float* out) {
    for (size_t i = 0; i < k; ++i) {
        const uint32_t byte = payload[i >> 1];
        const uint32_t nib = (i & 1) ? byte >> 4 : byte & 15u; /* low nibble = even k */
        out[i] = bits_f32(orc_mxfp4_bits(nib, scales[i >> 5]));
    }
}

/* oracle/lattice/quant_v1.py:37-45, crates/mimo26-load/src/e4m3.rs:19-32. */
float orc_e4m3_value(uint8_t code) {
    const int e = (code >> 3) & 15, m = code & 7;
    if ((code & 0x7f) == 0x7f) return NAN;
    const float mag = e ? ldexpf((float)(8 + m), e - 10) : ldexpf((float)m, -9);
    return (code & 0x80) ? -mag : mag;
}

/* crates/mimo26-expert/kernels/b1/grouped.cu:23-41 (scale accepted only in [105,247], NaN
 * codes propagate), oracle/lattice/quant_v1.py:93-100 (value * 2^(scale-127) in FP32). */
size_t orc_activation_decode(const uint8_t* payload, size_t payload_pitch, const uint8_t* scales,
                             size_t scales_pitch, size_t rows, size_t cols, float* out) {
    size_t bad = 0;
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < cols; ++c) {
            const uint8_t code = payload[r * payload_pitch + c];
            const int s = scales[r * scales_pitch + c / 32];
            float v;
            if ((code & 0x7f) == 0x7f || s < 105 || s > 247) { v = NAN; ++bad; }
            else v = ldexpf(orc_e4m3_value(code), s - 127);
            out[r * cols + c] = v;
        }
    return bad;
}

/* crates/mimo26-expert/kernels/b1/route_reduce.cu:52-59. */
uint16_t orc_bf16_rne(float v) {
    const uint32_t b = f32_bits(v);
    return (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}

/* crates/mimo26-load/src/e4m3.rs:50-81: nearest representable magnitude, ties to the larger
 * magnitude; NaN -> 0; saturate at 448; the sign bit is "v < 0" (so -0.0 encodes to 0x00 and
 * a negative value that rounds to zero keeps 0x80). */
uint8_t orc_e4m3_encode_half_up(double v) {
    if (isnan(v)) v = 0.0;
    double mag = fabs(v);
    if (mag > 448.0) mag = 448.0;
    const uint8_t sign = v < 0.0 ? 0x80 : 0;
    if (mag == 0.0) return sign;
    if (mag < 0.015625) { /* below 2^-6: quantum 2^-9 */
        const int m = (int)floor(mag * 512.0 + 0.5);
        return (uint8_t)(sign | (m >= 8 ? 8 : m));
    }
    int g;
    const double f = frexp(mag, &g); /* mag = f * 2^g, f in [0.5,1) */
    int e = g - 1 + 7;               /* biased exponent of 1.xxx * 2^(g-1) */
    int m = (int)floor((2.0 * f - 1.0) * 8.0 + 0.5);
    if (m >= 8) { m = 0; ++e; }
    if (e < 1) e = 1;
    if (e > 15) e = 15;
    if (m > 7) m = 7;
    return (uint8_t)(sign | (e << 3) | m);
}

/* crates/mimo26-coordinator/src/wire.rs:53-78: per 32 values, s = 0 for an all-zero block else
 * clamp(ceil(log2(amax/448)) + 127, 0, 254); payload = encode(v * 2^(127-s)).
 * ceil(log2(amax/448)) is the smallest integer e with amax <= 448*2^e; with amax = m*2^x,
 * m in [0.5,1), and 448 = 0.875*2^9, that is x-9 when m <= 0.875 and x-8 otherwise. */
void orc_q0_quantize(const float* x, size_t rows, size_t cols, uint8_t* payload, uint8_t* scales) {
    const size_t blocks = cols / 32;
    for (size_t r = 0; r < rows; ++r)
        for (size_t b = 0; b < blocks; ++b) {
            const float* blk = x + r * cols + b * 32;
            double amax = 0.0;
            for (int i = 0; i < 32; ++i) {
                const double a = fabs((double)blk[i]);
                if (a > amax) amax = a; /* NaN never wins, as f64::max ignores it */
            }
            int s = 0;
            if (amax > 0.0) {
                int xexp;
                const double m = frexp(amax, &xexp);
                s = (m <= 0.875 ? xexp - 9 : xexp - 8) + 127;
                if (isinf(amax)) s = 254;
                if (s < 0) s = 0;
                if (s > 254) s = 254;
            }
            scales[r * blocks + b] = (uint8_t)s;
            for (int i = 0; i < 32; ++i)
                payload[r * cols + b * 32 + i] =
                    orc_e4m3_encode_half_up(ldexp((double)blk[i], 127 - s));
        }
}

/* oracle/lattice/quant_v1.py:48-87 (codec of record) and the rule list in
 * crates/mimo26-expert/kernels/b1/quant_v1.cuh:84-100: a = max(max|h|, f32(1e-4)); k from
 * frexp (m <= 0.875 ? e-9 : e-8); payload = round-half-even of h*2^-k onto E4M3FN with -0
 * kept; fault 1 on nonfinite input, fault 2 when a code times 2^k leaves the FP32 range. */
static uint8_t e4m3_encode_rne(double y, int negative) {
    const double ay = fabs(y);
    int code;
    if (ay < 0.015625) {
        code = (int)nearbyint(ay * 512.0); /* 8 is the first normal code by construction */
    } else {
        int g;
        (void)frexp(ay, &g);
        int e = g - 1;
        int r = (int)nearbyint(ldexp(ay, 3 - e)); /* 8..16 */
        if (r == 16) { r = 8; ++e; }
        if (e > 8 || (e == 8 && r > 14)) code = 0x7e;
        else code = ((e + 7) << 3) | (r - 8);
    }
    return (uint8_t)(code | (negative ? 0x80 : 0));
}

size_t orc_quant_v1(const float* h, size_t elements, uint8_t* payload, uint8_t* scales,
                    uint32_t* faults) {
    size_t failed = 0;
    for (size_t b = 0; b < elements / 32; ++b) {
        const float* blk = h + b * 32;
        float a = 1e-4f;
        int finite = 1;
        for (int i = 0; i < 32; ++i) {
            if (!(fabsf(blk[i]) <= FLT_MAX)) finite = 0;
            if (fabsf(blk[i]) > a) a = fabsf(blk[i]);
        }
        if (!finite) { if (faults) faults[b] = 1; ++failed; continue; }
        int e;
        const float m = frexpf(a, &e);
        const int k = m <= 0.875f ? e - 9 : e - 8;
        uint8_t codes[32];
        int overflow = 0;
        for (int i = 0; i < 32; ++i) {
            codes[i] = e4m3_encode_rne(ldexp((double)blk[i], -k), signbit(blk[i]) != 0);
            const double back = ldexp((double)fabsf(orc_e4m3_value(codes[i])), k);
            if (back > (double)FLT_MAX) overflow = 1;
        }
        if (overflow) { if (faults) faults[b] = 2; ++failed; continue; }
        memcpy(payload + b * 32, codes, 32);
        scales[b] = (uint8_t)(k + 127);
        if (faults) faults[b] = 0;
    }
    return failed;
}

/* ------------------------------------------------------------------------------------------
 * Planner: crates/mimo26-expert/kernels/b1/group_plan.cu:32-79 (values only; pointer and
 * extent validation belongs to the caller here).
 * ---------------------------------------------------------------------------------------- */
uint32_t orc_plan(uint32_t capacity, uint32_t rows, const int32_t* ids, const float* weights,
                  const uint8_t* resident, int32_t* inverse, int32_t* original_routes,
                  float* grouped_weights, orc_group* groups, uint32_t* group_count,
                  uint32_t* fault) {
    const uint32_t routes = rows * 8, cap = capacity * 8;
    uint32_t count[256] = {0}, start[256], cursor[256];
    uint32_t status = ORC_OK;
    if (rows > capacity) status = ORC_GEOMETRY;
    for (int e = 0; e < 256 && status == ORC_OK; ++e)
        if (resident[e] > 1) status = ORC_METADATA;
    for (uint32_t i = 0; i < routes && status == ORC_OK; ++i) {
        const int32_t e = ids[i];
        if (e < 0 || e > 255 || !resident[e]) { status = ORC_METADATA; break; }
        if (!(weights[i] >= 0.0f && weights[i] <= FLT_MAX)) { status = ORC_NONFINITE; break; }
        for (uint32_t j = i & ~7u; j < i; ++j)
            if (ids[j] == e) status = ORC_METADATA;
        ++count[e];
    }
    *fault = status;
    if (status != ORC_OK) return status;
    uint32_t running = 0;
    for (int e = 0; e < 256; ++e) { start[e] = cursor[e] = running; running += count[e]; }
    for (uint32_t i = 0; i < cap; ++i) {
        inverse[i] = -1;
        original_routes[i] = -1;
        grouped_weights[i] = 0.0f;
        groups[i].expert = -1;
        groups[i].rows = 0;
        groups[i].route_base = -1;
        for (int j = 0; j < 16; ++j) groups[i].input_rows[j] = -1;
    }
    for (uint32_t i = 0; i < routes; ++i) { /* ascending i keeps the order stable */
        const uint32_t slot = cursor[ids[i]]++;
        inverse[i] = (int32_t)slot;
        original_routes[slot] = (int32_t)i;
        grouped_weights[slot] = weights[i];
    }
    uint32_t ng = 0;
    for (int e = 0; e < 256; ++e)
        for (uint32_t off = 0; off < count[e]; off += 16) {
            orc_group* g = &groups[ng++];
            const uint32_t left = count[e] - off;
            g->expert = e;
            g->route_base = (int32_t)(start[e] + off);
            g->rows = (int32_t)(left < 16 ? left : 16);
            for (int32_t j = 0; j < g->rows; ++j)
                g->input_rows[j] = original_routes[g->route_base + j] / 8;
        }
    *group_count = ng;
    return ORC_OK;
}

/* ------------------------------------------------------------------------------------------
 * Activation and combine
 * ---------------------------------------------------------------------------------------- */

/* crates/mimo26-repack/tests/lattice_oracle.py:32-53 (exp in binary64, rounded once to
 * binary32, then ordered FP32 ops; same form as kernels/b1/grouped.cu:89-93). */
float orc_silu_up(float gate, float up) {
    const float t = gate >= 0.0f ? -gate : gate;
    const float e = (float)exp((double)t);
    volatile float d = 1.0f + e;
    volatile float s;
    if (gate >= 0.0f) s = gate / d;
    else { volatile float n = gate * e; s = n / d; }
    volatile float h = s * up;
    return h;
}

/* crates/mimo26-expert/kernels/b1/route_reduce.cu:61-74: v = 0; for slot 0..7:
 * v = RN(v + RN(w*z)), each weight finite and >= 0, each z and running v finite; BF16 RNE
 * whose exponent must not be all ones. */
uint32_t orc_reduce(const float* y, const float* w, size_t rows, size_t cols, float* partial,
                    uint16_t* bf16) {
    for (size_t t = 0; t < rows; ++t)
        for (size_t c = 0; c < cols; ++c) {
            volatile float v = 0.0f;
            for (int s = 0; s < 8; ++s) {
                const float wt = w[t * 8 + s], z = y[(t * 8 + s) * cols + c];
                if (!(wt >= 0.0f && wt <= FLT_MAX) || !(fabsf(z) <= FLT_MAX)) return ORC_NONFINITE;
                volatile float p = wt * z;
                v = v + p;
                if (!(fabsf(v) <= FLT_MAX)) return ORC_NONFINITE;
            }
            const uint16_t code = orc_bf16_rne(v);
            if ((code & 0x7f80u) == 0x7f80u) return ORC_NONFINITE;
            if (partial) partial[t * cols + c] = v;
            if (bf16) bf16[t * cols + c] = code;
        }
    return ORC_OK;
}

/* The opt-in BF16 per-route mode (MIMO26_B1_Y=bf16). FC2's store rule, crates/mimo26-expert/kernels/b1/
 * connected.cu:41-44: BF16 bits by the integer round-to-nearest-even, no special cases. */
void orc_bf16_store_rows(const float* y, size_t n, uint16_t* out) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_rne(y[i]);
}

/* crates/mimo26-spark/kernels/b1_serve.cu:98-143 (reduce_bf16y): route_reduce's sum on the widened BF16
 * rows, same slot order, separately rounded multiply and add, same finite / sign rules, BF16 RNE out, no
 * FP32 sum kept. Returns 0, or 5 (the value that kernel's fault word takes) at the first violating element. */
uint32_t orc_reduce_bf16y(const uint16_t* y16, const float* w, size_t rows, size_t cols, uint16_t* bf16) {
    for (size_t t = 0; t < rows; ++t)
        for (size_t c = 0; c < cols; ++c) {
            volatile float v = 0.0f;
            for (int s = 0; s < 8; ++s) {
                const float wt = w[t * 8 + s], z = bits_f32((uint32_t)y16[(t * 8 + s) * cols + c] << 16);
                if (!(wt >= 0.0f && wt <= FLT_MAX) || !(z >= -FLT_MAX && z <= FLT_MAX)) return 5;
                volatile float p = wt * z;
                v = v + p;
                if (!(v >= -FLT_MAX && v <= FLT_MAX)) return 5;
            }
            const uint32_t b = f32_bits(v);
            const uint16_t code = (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
            if ((code & 0x7f80u) == 0x7f80u) return 5;
            bf16[t * cols + c] = code;
        }
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Expert FFN (W4A8 lattice): crates/mimo26-repack/tests/lattice_oracle.py:56-91.
 * Layout: crates/mimo26-expert/src/slice.rs:33-53.
 * ---------------------------------------------------------------------------------------- */

/* Dots of one weight row against a block of up to 8 activation rows held k-major
 * (xt[k*8 + j]); every row's sum runs in ascending k, in binary64. */
static void dot8(const double* xt, const float* w, size_t k, double acc[8]) {
    double a0 = 0, a1 = 0, a2 = 0, a3 = 0, a4 = 0, a5 = 0, a6 = 0, a7 = 0;
    for (size_t i = 0; i < k; ++i) {
        const double wv = (double)w[i];
        const double* x = xt + i * 8;
        a0 += x[0] * wv; a1 += x[1] * wv; a2 += x[2] * wv; a3 += x[3] * wv;
        a4 += x[4] * wv; a5 += x[5] * wv; a6 += x[6] * wv; a7 += x[7] * wv;
    }
    acc[0] = a0; acc[1] = a1; acc[2] = a2; acc[3] = a3;
    acc[4] = a4; acc[5] = a5; acc[6] = a6; acc[7] = a7;
}

static int finite32(float v) { return fabsf(v) <= FLT_MAX; }

/* rows are given as pointers so a caller can pass gathered tokens without copying */
static uint32_t expert_ffn_rows(const orc_layer* layer, uint32_t expert,
                                const uint8_t* const* xp, const uint8_t* const* xs, size_t rows,
                                float* gate, float* up, float* h, uint8_t* mid_payload,
                                uint8_t* mid_scales, float* y) {
    const size_t H = ORC_HIDDEN, I = (size_t)ORC_RANK_I * layer->ranks;
    const size_t blocks = (rows + 7) / 8;
    uint32_t fault = 0;
    double* xt = (double*)calloc(blocks * H * 8, sizeof(double));
    float* xrow = (float*)malloc(H * sizeof(float));
    float* wrow = (float*)malloc((H > I ? H : I) * sizeof(float));
    float* g_ = gate ? gate : (float*)malloc(rows * I * sizeof(float));
    float* u_ = up ? up : (float*)malloc(rows * I * sizeof(float));
    float* h_ = h ? h : (float*)malloc(rows * I * sizeof(float));
    uint8_t* mp = mid_payload ? mid_payload : (uint8_t*)malloc(rows * I);
    uint8_t* ms = mid_scales ? mid_scales : (uint8_t*)malloc(rows * I / 32);
    uint32_t* qf = (uint32_t*)malloc(rows * I / 32 * sizeof(uint32_t));
    double* mt = (double*)calloc(blocks * I * 8, sizeof(double));
    float* mrow = (float*)malloc(I * sizeof(float));

    for (size_t t = 0; t < rows; ++t) {
        if (orc_activation_decode(xp[t], 0, xs[t], 0, 1, H, xrow)) fault = 1;
        for (size_t k = 0; k < H; ++k) xt[((t / 8) * H + k) * 8 + t % 8] = (double)xrow[k];
    }
    for (int proj = 0; proj < 2 && !fault; ++proj) {
        float* dst = proj ? u_ : g_;
        const size_t poff = proj ? ORC_UP_PAYLOAD : ORC_GATE_PAYLOAD;
        const size_t soff = proj ? ORC_UP_SCALES : ORC_GATE_SCALES;
        for (size_t n = 0; n < I; ++n) {
            const uint8_t* img = layer->pool[n / ORC_RANK_I] + (size_t)expert * ORC_IMAGE_BYTES;
            const size_t local = n % ORC_RANK_I;
            orc_mxfp4_row(img + poff + local * (H / 2), img + soff + local * (H / 32), H, wrow);
            for (size_t b = 0; b < blocks; ++b) {
                double acc[8];
                dot8(xt + b * H * 8, wrow, H, acc);
                for (size_t j = 0; j < 8 && b * 8 + j < rows; ++j) {
                    const float v = (float)acc[j];
                    if (!finite32(v)) fault = 1;
                    dst[(b * 8 + j) * I + n] = v;
                }
            }
        }
    }
    if (!fault) {
        for (size_t i = 0; i < rows * I; ++i) {
            h_[i] = orc_silu_up(g_[i], u_[i]);
            if (!finite32(h_[i])) fault = 1;
        }
    }
    if (!fault && orc_quant_v1(h_, rows * I, mp, ms, qf)) fault = 2;
    if (!fault) {
        for (size_t t = 0; t < rows; ++t) {
            orc_activation_decode(mp + t * I, 0, ms + t * (I / 32), 0, 1, I, mrow);
            for (size_t k = 0; k < I; ++k) mt[((t / 8) * I + k) * 8 + t % 8] = (double)mrow[k];
        }
        for (size_t c = 0; c < H; ++c) {
            for (uint32_t r = 0; r < layer->ranks; ++r) {
                const uint8_t* img = layer->pool[r] + (size_t)expert * ORC_IMAGE_BYTES;
                orc_mxfp4_row(img + ORC_DOWN_PAYLOAD + c * (ORC_RANK_I / 2),
                              img + ORC_DOWN_SCALES + c * (ORC_RANK_I / 32), ORC_RANK_I,
                              wrow + (size_t)r * ORC_RANK_I);
            }
            for (size_t b = 0; b < blocks; ++b) {
                double acc[8];
                dot8(mt + b * I * 8, wrow, I, acc);
                for (size_t j = 0; j < 8 && b * 8 + j < rows; ++j) {
                    const float v = (float)acc[j];
                    if (!finite32(v)) fault = 1;
                    y[(b * 8 + j) * H + c] = v;
                }
            }
        }
    }
    free(xt); free(xrow); free(wrow); free(qf); free(mt); free(mrow);
    if (!gate) free(g_);
    if (!up) free(u_);
    if (!h) free(h_);
    if (!mid_payload) free(mp);
    if (!mid_scales) free(ms);
    return fault;
}

uint32_t orc_expert_ffn(const orc_layer* layer, uint32_t expert, const uint8_t* x_payload,
                        size_t x_pitch, const uint8_t* x_scales, size_t xs_pitch, size_t rows,
                        float* gate, float* up, float* h, uint8_t* mid_payload,
                        uint8_t* mid_scales, float* y) {
    const uint8_t** xp = (const uint8_t**)malloc(rows * sizeof(*xp));
    const uint8_t** xs = (const uint8_t**)malloc(rows * sizeof(*xs));
    for (size_t t = 0; t < rows; ++t) { xp[t] = x_payload + t * x_pitch; xs[t] = x_scales + t * xs_pitch; }
    const uint32_t f = expert_ffn_rows(layer, expert, xp, xs, rows, gate, up, h, mid_payload,
                                       mid_scales, y);
    free(xp); free(xs);
    return f;
}

int orc_hardware_threads(void) {
#ifdef _OPENMP
    return omp_get_num_procs();
#else
    return 1;
#endif
}

/* Routing shared by both layer variants: validate and bucket, then hand each expert its
 * rows in stable route order. */
typedef struct {
    int32_t *inverse, *original;
    float* gw;
    orc_group* groups;
    uint32_t group_count, start[257];
} layer_plan;

static uint32_t make_plan(const int32_t* ids, const float* weights, size_t rows, layer_plan* p) {
    uint8_t resident[256];
    uint32_t fault = 0;
    memset(resident, 1, sizeof resident);
    const size_t cap = rows ? rows * 8 : 8;
    p->inverse = (int32_t*)malloc(cap * 4);
    p->original = (int32_t*)malloc(cap * 4);
    p->gw = (float*)malloc(cap * 4);
    p->groups = (orc_group*)malloc(cap * sizeof(orc_group));
    orc_plan((uint32_t)rows, (uint32_t)rows, ids, weights, resident, p->inverse, p->original,
             p->gw, p->groups, &p->group_count, &fault);
    if (fault) return fault;
    uint32_t count[256] = {0};
    for (size_t i = 0; i < rows * 8; ++i) ++count[ids[i]];
    p->start[0] = 0;
    for (int e = 0; e < 256; ++e) p->start[e + 1] = p->start[e] + count[e];
    return 0;
}
static void free_plan(layer_plan* p) { free(p->inverse); free(p->original); free(p->gw); free(p->groups); }

uint32_t orc_layer_ffn(const orc_layer* layer, const uint8_t* x_payload, size_t x_pitch,
                       const uint8_t* x_scales, size_t xs_pitch, const int32_t* ids,
                       const float* weights, size_t rows, float* y_routes, float* partial,
                       uint16_t* bf16, int threads) {
    layer_plan p;
    if (make_plan(ids, weights, rows, &p)) { free_plan(&p); return 3; }
    float* y = y_routes ? y_routes : (float*)malloc(rows * 8 * ORC_HIDDEN * sizeof(float));
    uint32_t fault = 0;
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_num_procs();
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads) reduction(| : fault)
#endif
    for (int e = 0; e < 256; ++e) {
        const size_t n = p.start[e + 1] - p.start[e];
        if (!n) continue;
        const uint8_t** xp = (const uint8_t**)malloc(n * sizeof(*xp));
        const uint8_t** xs = (const uint8_t**)malloc(n * sizeof(*xs));
        float* ye = (float*)malloc(n * ORC_HIDDEN * sizeof(float));
        for (size_t j = 0; j < n; ++j) {
            const size_t token = (size_t)p.original[p.start[e] + j] / 8;
            xp[j] = x_payload + token * x_pitch;
            xs[j] = x_scales + token * xs_pitch;
        }
        const uint32_t f = expert_ffn_rows(layer, (uint32_t)e, xp, xs, n, NULL, NULL, NULL, NULL, NULL, ye);
        if (f) fault |= f;
        else
            for (size_t j = 0; j < n; ++j)
                memcpy(y + (size_t)p.original[p.start[e] + j] * ORC_HIDDEN, ye + j * ORC_HIDDEN,
                       ORC_HIDDEN * sizeof(float));
        free(xp); free(xs); free(ye);
    }
    if (!fault && orc_reduce(y, weights, rows, ORC_HIDDEN, partial, bf16)) fault = 1;
    if (!y_routes) free(y);
    free_plan(&p);
    (void)threads;
    return fault ? 4 : 0;
}

/* crates/mimo26-spark/src/main.rs:75-95 -> crates/mimo26-spark/src/serve.rs:33-61 (decode the
 * wire rows to f32), crates/mimo26-expert/src/grouped.rs:291-336 (per output: f32 acc over k of
 * unpack_element(w)*x), :352-366 (silu(g) = g/(1+exp(-g)) in f32, times up), :385-393 (down on
 * the f32 intermediate), crates/mimo26-spark/src/decode.rs:777-792 (out += y*w in route order,
 * then BF16 RNE). The activation decode there clamps instead of faulting. */
static float efp32_dot(const uint8_t* payload, const uint8_t* scales, const float* x, size_t k) {
    volatile float acc = 0.0f;
    for (size_t i = 0; i < k; ++i) {
        const uint32_t byte = payload[i >> 1];
        const float w = bits_f32(orc_mxfp4_bits((i & 1) ? byte >> 4 : byte & 15u, scales[i >> 5]));
        volatile float p = w * x[i];
        acc = acc + p;
    }
    return acc;
}

uint32_t orc_layer_ffn_efp32(const orc_layer* layer, const uint8_t* x_payload, size_t x_pitch,
                             const uint8_t* x_scales, size_t xs_pitch, const int32_t* ids,
                             const float* weights, size_t rows, float* partial, uint16_t* bf16,
                             int threads) {
    const size_t H = ORC_HIDDEN, I = (size_t)ORC_RANK_I * layer->ranks;
    layer_plan p;
    if (make_plan(ids, weights, rows, &p)) { free_plan(&p); return 3; }
    float* y = (float*)malloc(rows * 8 * H * sizeof(float));
#ifdef _OPENMP
    if (threads <= 0) threads = omp_get_num_procs();
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
#endif
    for (int e = 0; e < 256; ++e) {
        const size_t n = p.start[e + 1] - p.start[e];
        if (!n) continue;
        float* x = (float*)malloc(H * sizeof(float));
        float* hbuf = (float*)malloc(I * sizeof(float));
        float* seg = (float*)malloc(ORC_RANK_I * sizeof(float));
        for (size_t j = 0; j < n; ++j) {
            const size_t route = (size_t)p.original[p.start[e] + j], token = route / 8;
            for (size_t k = 0; k < H; ++k) {
                const uint8_t code = x_payload[token * x_pitch + k];
                const int s = x_scales[token * xs_pitch + k / 32];
                double v = (double)orc_e4m3_value(code) * ldexp(1.0, (s > 254 ? 254 : s) - 127);
                if (v > FLT_MAX) v = FLT_MAX;
                if (v < -FLT_MAX) v = -FLT_MAX;
                x[k] = (float)v;
            }
            for (size_t c = 0; c < I; ++c) {
                const uint8_t* img = layer->pool[c / ORC_RANK_I] + (size_t)e * ORC_IMAGE_BYTES;
                const size_t local = c % ORC_RANK_I;
                const float g = efp32_dot(img + ORC_GATE_PAYLOAD + local * (H / 2),
                                          img + ORC_GATE_SCALES + local * (H / 32), x, H);
                const float u = efp32_dot(img + ORC_UP_PAYLOAD + local * (H / 2),
                                          img + ORC_UP_SCALES + local * (H / 32), x, H);
                volatile float d = 1.0f + expf(-g);
                volatile float s = g / d;
                hbuf[c] = s * u;
            }
            /* Each rank's 512-wide down partial accumulates from zero in f32. With one pool
             * this is the reference's rank-local path exactly; with four pools the partials
             * add in rank order before the combine (the four-rank system instead rounds each
             * rank's combined row to BF16 first), which keeps this a baseline only. */
            for (size_t c = 0; c < H; ++c) {
                volatile float total = 0.0f;
                for (uint32_t r = 0; r < layer->ranks; ++r) {
                    const uint8_t* img = layer->pool[r] + (size_t)e * ORC_IMAGE_BYTES;
                    const float part = efp32_dot(img + ORC_DOWN_PAYLOAD + c * (ORC_RANK_I / 2),
                                                 img + ORC_DOWN_SCALES + c * (ORC_RANK_I / 32),
                                                 hbuf + (size_t)r * ORC_RANK_I, ORC_RANK_I);
                    total = layer->ranks == 1 ? part : total + part;
                }
                y[route * H + c] = total;
            }
        }
        free(x); free(hbuf); free(seg);
    }
    for (size_t t = 0; t < rows; ++t)
        for (size_t c = 0; c < H; ++c) {
            volatile float v = 0.0f;
            for (int s = 0; s < 8; ++s) {
                volatile float term = y[(t * 8 + s) * H + c] * weights[t * 8 + s];
                v = v + term;
            }
            if (partial) partial[t * H + c] = v;
            if (bf16) bf16[t * H + c] = orc_bf16_rne(v);
        }
    free(y);
    free_plan(&p);
    (void)threads;
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Coordinator-side steps around the path
 * ---------------------------------------------------------------------------------------- */

/* crates/mimo26-coordinator/src/router.rs:41-80: scores = 1 / (1 + exp(-logit)) in FP64; order by
 * score + bias descending, stable over ascending ids; weights from the unbiased scores. */
void orc_router_topk(const float* logits, const float* bias, size_t rows, size_t n_experts, size_t top_k,
                     int32_t* idx, float* weights) {
    double* score = (double*)malloc(n_experts * sizeof(double));
    double* sel = (double*)malloc(n_experts * sizeof(double));
    for (size_t r = 0; r < rows; ++r) {
        for (size_t e = 0; e < n_experts; ++e) {
            score[e] = 1.0 / (1.0 + exp(-(double)logits[r * n_experts + e]));
            sel[e] = score[e] + (double)bias[e];
        }
        double wsum = 0.0;
        for (size_t k = 0; k < top_k; ++k) { /* k passes of "largest remaining, lowest id first" = stable sort prefix */
            size_t best = n_experts;
            for (size_t e = 0; e < n_experts; ++e)
                if (!isnan(sel[e]) && (best == n_experts || sel[e] > sel[best])) best = e;
            idx[r * top_k + k] = (int32_t)best;
            wsum += score[best];
            sel[best] = NAN; /* taken */
        }
        for (size_t k = 0; k < top_k; ++k) weights[r * top_k + k] = (float)(score[idx[r * top_k + k]] / wsum);
    }
    free(score);
    free(sel);
}

/* crates/mimo26-coordinator/src/wire.rs:83-108: the scale half of orc_q0_quantize and the power of
 * two the payload half multiplies by. */
void orc_q0_scales(const float* x, size_t n_blocks, uint8_t* scales, float* scale_inv) {
    for (size_t b = 0; b < n_blocks; ++b) {
        uint8_t s;
        uint8_t scratch[32];
        orc_q0_quantize(x + b * 32, 1, 32, scratch, &s);
        scales[b] = s;
        scale_inv[b] = ldexpf(1.0f, 127 - (int)s);
    }
}

/* crates/mimo26-wire/src/l4.rs (CoordinatorSum), crates/mimo26-coordinator/kernels/glue.cu:198-213. */
void orc_rank_sum_bf16(const uint16_t* p0, const uint16_t* p1, const uint16_t* p2, const uint16_t* p3,
                       float* out, size_t n) {
    const uint16_t* p[4] = {p0, p1, p2, p3};
    for (size_t i = 0; i < n; ++i) {
        volatile float s = 0.0f; /* one rounding per addition, no contraction */
        for (int r = 0; r < 4; ++r) s = s + bits_f32((uint32_t)p[r][i] << 16);
        out[i] = s;
    }
}

uint16_t orc_bf16_rne_nan(float v) { return isnan(v) ? (uint16_t)0x7fff : orc_bf16_rne(v); }

