// gfx950 kernels of the coordinator-side steps around the routed-expert FFN: routing, the wire
// quantizer (Q0), the request-frame fill, the rank sum and the residual add. All of them move a few
// bytes per value once; they are written for coalesced 16-byte traffic and nothing else.
//
// Reference counterparts: crates/mimo26-coordinator/kernels/glue.cu (router_topk_kernel :76-124,
// quant_scales_kernel :126-143, rank_sum_bf16_kernel :198-213, f32_to_bf16_kernel :215-221,
// frame_fill_kernel :309-339), crates/mimo26-attn/kernels/kv_cache_fp8.cu:161-170 and
// crates/mimo26-attn/kernels/include/mimo26_attn_device.cuh:33-55 (e4m3_encode).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace m26g {

// ---- routing ------------------------------------------------------------------------------------
// One wave per row; lane l holds experts l, l+64, ... (PER of them, n_experts <= 64 * PER <= 1024).
// Scores and the selection run in binary64 like the reference; the k selections are k wave-wide
// arg-max rounds on (score + bias, lower id wins ties). Weights: unbiased score / sum, the sum taken
// in selection order, rounded to binary32.
//
// The rounds are a chain of dependent steps, so the wave-wide arg-max stays inside the vector unit: DPP moves
// within a row of sixteen lanes (neighbours in a quad, the mirrored half-row, the mirrored row), then the last
// lane of a row handed to the next row and the last lane of the second row to the upper two, after which lane
// 63 holds the winner and a lane read makes it uniform. Through the LDS crossbar (the shuffle intrinsics) the
// same eight rounds took three times as long.
constexpr int kRouterPerLane = 16;

struct Best {
    double v;
    int i;
};
__device__ __forceinline__ Best better(Best a, Best b) { return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a; }
template <int CTRL, int ROWS>
__device__ __forceinline__ Best best_from(Best a) {  // lanes of rows outside ROWS get their own value back
    const int lo = __double2loint(a.v), hi = __double2hiint(a.v);
    return Best{__hiloint2double(__builtin_amdgcn_update_dpp(hi, hi, CTRL, ROWS, 0xf, false), __builtin_amdgcn_update_dpp(lo, lo, CTRL, ROWS, 0xf, false)),
                __builtin_amdgcn_update_dpp(a.i, a.i, CTRL, ROWS, 0xf, false)};
}
__device__ __forceinline__ Best wave_best(Best a) {
    a = better(a, best_from<0xB1, 0xf>(a));   // quad_perm [1,0,3,2]
    a = better(a, best_from<0x4E, 0xf>(a));   // quad_perm [2,3,0,1]
    a = better(a, best_from<0x141, 0xf>(a));  // row_half_mirror
    a = better(a, best_from<0x140, 0xf>(a));  // row_mirror: every lane of a row holds the row's best
    a = better(a, best_from<0x142, 0xa>(a));  // row_bcast15 into rows 1 and 3
    a = better(a, best_from<0x143, 0xc>(a));  // row_bcast31 into rows 2 and 3: lane 63 holds the wave's best
    return Best{__hiloint2double(__builtin_amdgcn_readlane(__double2hiint(a.v), 63), __builtin_amdgcn_readlane(__double2loint(a.v), 63)),
                __builtin_amdgcn_readlane(a.i, 63)};
}

template <int PER>
__global__ void __launch_bounds__(256) router_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                          int rows, int n_experts, int top_k, int* __restrict__ idx_out,
                                                          float* __restrict__ w_out) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* lrow = logits + size_t(row) * n_experts;
    double score[PER], sel[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = lane + 64 * j;
        if (e < n_experts) {
            score[j] = 1.0 / (1.0 + exp(-double(lrow[e])));
            sel[j] = score[j] + double(bias[e]);
        } else {
            score[j] = 0.0;
            sel[j] = -INFINITY;
        }
    }
    double wsum = 0.0, mine = 0.0;  // lane k keeps the k-th chosen score
    int mine_id = 0;
    for (int k = 0; k < top_k; ++k) {
        Best b{-INFINITY, 0x7fffffff};
#pragma unroll
        for (int j = 0; j < PER; ++j)  // ascending ids: a strict > keeps the lower id on ties; absent experts hold -inf
            if (sel[j] > b.v) b = Best{sel[j], lane + 64 * j};
        b = wave_best(b);              // the same in every lane, and known to be
        const int owner = b.i & 63, slot = b.i >> 6;
        double s = 0.0;
#pragma unroll
        for (int j = 0; j < PER; ++j)
            if (j == slot) {
                s = __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(score[j]), owner),
                                     __builtin_amdgcn_readlane(__double2loint(score[j]), owner));
                if (lane == owner) sel[j] = -INFINITY;
            }
        wsum += s;
        if (lane == k) { mine = s; mine_id = b.i; }
    }
    if (lane < top_k) {
        idx_out[size_t(row) * top_k + lane] = mine_id;
        w_out[size_t(row) * top_k + lane] = float(mine / wsum);
    }
}

// ---- wire quantizer (Q0) ---------------------------------------------------------------------------
// s = 0 for an all-zero block, else the smallest e with amax <= 448 * 2^e, plus 127, clamped to
// [0, 254]: with amax = m * 2^x, m in [0.5, 1), that is x - 9 for m <= 0.875 and x - 8 above
// (448 = 0.875 * 2^9). NaNs do not take part in amax; an infinite amax gives 254.
__device__ __forceinline__ uint32_t q0_scale_byte(float amax) {
    if (!(amax > 0.0f)) return 0;
    if (amax > 3.402823466e38f) return 254;
    int x;
    const float m = frexpf(amax, &x);  // exact, subnormals included
    int s = (m <= 0.875f ? x - 9 : x - 8) + 127;
    s = s < 0 ? 0 : s;
    return uint32_t(s > 254 ? 254 : s);
}

// E4M3FN code nearest to y = x * scale (scale a positive power of two), ties to the larger magnitude,
// saturating at 448, NaN -> 0. The sign bit is "the exact product is below zero", i.e. x < 0: -0.0
// gives 0x00 while a negative value that rounds to zero keeps 0x80, also where the binary32 product
// has already underflowed to -0 (the CPU rule multiplies in binary64). Integer arithmetic on the bit
// pattern: from 2^-6 up a code is the binary32 exponent and top three mantissa bits rebased, so
// round-half-up is one add and one shift and a mantissa that rounds over carries into the exponent by
// itself (448, the clamp, is code 0x7e exactly, so nothing larger can come out); below 2^-6 the
// quantum is 2^-9 whatever the exponent, and the significand is shifted down to it.
constexpr uint32_t kE4m3NormalFrom = 121u << 23;  // binary32 bits of 2^-6
__device__ __forceinline__ uint32_t e4m3_magnitude_bits(float y) { return __float_as_uint(fminf(fabsf(y), 448.0f)); }  // a NaN leaves as 448
__device__ __forceinline__ uint32_t e4m3_code_normal(uint32_t bits) { return ((bits + 0x80000u) >> 20) - ((127u - 7u) << 3); }
__device__ __forceinline__ uint32_t e4m3_code_small(uint32_t bits) {  // code = floor(value * 512 + 1/2)
    const uint32_t sig = (bits & 0x7fffffu) | 0x800000u, sh = 141u - (bits >> 23);  // value = sig * 2^(field - 150); sh >= 21
    return sh > 31u ? 0u : (sig + (1u << (sh - 1u))) >> sh;  // under 2^-11 (zero and binary32 subnormals too): nothing
}
__device__ __forceinline__ uint32_t e4m3_signed(float x, float y, uint32_t code) {
    return y != y ? 0u : (x < 0.0f ? 0x80u : 0u) | code;
}
__device__ __forceinline__ uint32_t e4m3_half_up(float x, float scale) {
    const float y = x * scale;
    const uint32_t bits = e4m3_magnitude_bits(y);
    return e4m3_signed(x, y, bits < kE4m3NormalFrom ? e4m3_code_small(bits) : e4m3_code_normal(bits));
}
// Four at once, packed low address first: the rule above, value by value.
__device__ __forceinline__ uint32_t e4m3_half_up4_any(const float4 v, float scale) {
    return e4m3_half_up(v.x, scale) | e4m3_half_up(v.y, scale) << 8 | e4m3_half_up(v.z, scale) << 16 | e4m3_half_up(v.w, scale) << 24;
}
// The same four codes in about a third of the instructions when the scale is positive and every scaled value is
// a number of at least 2^-6 in magnitude (a block's amax lands in (224, 448], so smaller ones are rare), which
// these kernels need: a wave64 vector instruction occupies its SIMD for four cycles, and at 16 bytes in per lane
// the budget for keeping up with HBM is about 85 of them per kilobyte. What is different: the sign bit is read
// off fma(x, scale, +0), which is x * scale except that -0 * scale + 0 is +0 (the rule's "x < 0") while a
// negative product that underflows still rounds to -0; the clamp is an integer minimum on the magnitude bits
// (an infinity saturates like any large value); and the rebasing constant rides in the rounding add.
__device__ __forceinline__ uint32_t e4m3_half_up4(const float4 v, float scale) {
    const float x[4] = {v.x, v.y, v.z, v.w};
    uint32_t bits[4], mag[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        bits[j] = __float_as_uint(__builtin_fmaf(x[j], scale, 0.0f));
        mag[j] = bits[j] & 0x7fffffffu;
    }
    auto lesser = [](uint32_t a, uint32_t b) { return a < b ? a : b; };
    auto larger = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
    const uint32_t least = lesser(lesser(mag[0], mag[1]), lesser(mag[2], mag[3])), most = larger(larger(mag[0], mag[1]), larger(mag[2], mag[3]));
    if (least < kE4m3NormalFrom || most > 0x7f800000u || !(scale > 0.0f)) return e4m3_half_up4_any(v, scale);
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t code = (lesser(mag[j], 0x43e00000u /* 448 */) + (0x80000u - ((127u - 7u) << 23))) >> 20;
        word |= (((bits[j] >> 24) & 0x80u) | code) << (8 * j);
    }
    return word;
}

// Maximum over the eight lanes of a K32 block without leaving the vector unit: neighbours within a quad
// (lanes ^ 1, ^ 2), then the mirrored half-row, which pairs each quad with the other one of its eight.
constexpr int kQuadXor1 = 0xB1, kQuadXor2 = 0x4E, kHalfRowMirror = 0x141;  // DPP controls: quad_perm [1,0,3,2], [2,3,0,1], row_half_mirror
__device__ __forceinline__ float max_over_eight(float v) {
    int b = __float_as_int(v);
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(b, b, kQuadXor1, 0xf, 0xf, false)));
    b = __float_as_int(v);
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(b, b, kQuadXor2, 0xf, 0xf, false)));
    b = __float_as_int(v);
    return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(b, b, kHalfRowMirror, 0xf, 0xf, false)));
}
__device__ __forceinline__ uint32_t max_bits_over_eight(uint32_t v) {
    auto larger = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
    v = larger(v, uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), kQuadXor1, 0xf, 0xf, false)));
    v = larger(v, uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), kQuadXor2, 0xf, 0xf, false)));
    return larger(v, uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), kHalfRowMirror, 0xf, 0xf, false)));
}

// One K32 block per 8 lanes, four values per lane; a workgroup takes 32 consecutive blocks of a row
// (1024 values), blockIdx.x choosing the piece of the row and blockIdx.y striding over rows, so no
// thread divides anything. x is contiguous (row r starts at r * 32 * per_row); payload and scales
// have their own pitches; `total` blocks exist (the last row may be short when the host has cut one long
// array into rows). Four rows are in flight per thread and step.
//
// A block of numbers (no NaN, no infinity: its largest magnitude pattern is below 0x7f800000) takes the
// scale from the bit pattern: with amax = 1.f * 2^(field - 127) the rule's frexp exponent is field - 126 and
// its mantissa exceeds 0.875 exactly when f exceeds 0.75, so s = field - 8 plus the carry of f + 0.25,
// floored at 0 (subnormal and zero amax land there); 254 cannot be reached. Any other block goes the long way.
constexpr int kQuantRowsInFlight = 4;
__global__ void __launch_bounds__(256) quantize_hidden_kernel(const float* __restrict__ x, long rows, long per_row, long total,
                                                              uint8_t* __restrict__ payload, size_t payload_pitch,
                                                              uint8_t* __restrict__ scales, size_t scales_pitch,
                                                              float* __restrict__ scale_inv) {
    const uint32_t sub = threadIdx.x & 7;
    const long c = long(blockIdx.x) * 32 + (threadIdx.x >> 3);
    const bool in_row = c < per_row;  // the same for all eight lanes of a block, so the exchanges below see whole blocks
    // NaNs take no part in amax. They are zeroed first: a signalling NaN would come out of the
    // hardware maximum as a quiet one and wipe what was gathered before it.
    auto mag = [](float f) { return f != f ? 0.0f : fabsf(f); };
    auto finish = [&](long r, float4 v, bool live) {
        if (!live) v = make_float4(0.f, 0.f, 0.f, 0.f);
        const uint32_t m0 = __float_as_uint(v.x) & 0x7fffffffu, m1 = __float_as_uint(v.y) & 0x7fffffffu,
                       m2 = __float_as_uint(v.z) & 0x7fffffffu, m3 = __float_as_uint(v.w) & 0x7fffffffu;
        auto larger = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
        const uint32_t most = max_bits_over_eight(larger(larger(m0, m1), larger(m2, m3))), field = (most + 0x1fffffu) >> 23;
        uint32_t s = field > 8u ? field - 8u : 0u;
        if (most >= 0x7f800000u) {  // the same answer in all eight lanes of the block
            const float amax = max_over_eight(fmaxf(fmaxf(mag(v.x), mag(v.y)), fmaxf(mag(v.z), mag(v.w))));
            s = q0_scale_byte(amax);
        }
        // 2^(127 - s): exponent field 254 - s; s = 254 is 2^-127, the subnormal with the top mantissa bit
        const float scale = __uint_as_float(s == 254u ? 0x00400000u : (254u - s) << 23);
        if (!live) return;
        if (payload) *reinterpret_cast<uint32_t*>(payload + r * payload_pitch + c * 32 + sub * 4) = e4m3_half_up4(v, scale);
        if (sub == 0) {
            if (scales) scales[r * scales_pitch + c] = uint8_t(s);
            if (scale_inv) scale_inv[r * per_row + c] = scale;
        }
    };
    // A set is kQuantRowsInFlight rows, gridDim.y apart. The next set is asked for before this one is worked on:
    // the arithmetic of a set (some 300 vector instructions, four cycles each) is as long as a memory round
    // trip, and waves that all load, then all compute, leave HBM idle half of the time.
    const long step = gridDim.y;
    auto fetch = [&](long r, float4 (&v)[kQuantRowsInFlight], bool (&live)[kQuantRowsInFlight]) {
#pragma unroll
        for (int j = 0; j < kQuantRowsInFlight; ++j) {
            const long rj = r + j * step;
            live[j] = in_row && rj < rows && rj * per_row + c < total;
            // Every lane loads, a lane without a block the array's first one: a load under a condition would make
            // the wait ahead of the arithmetic a wait for everything in flight, this set's successor included.
            v[j] = *reinterpret_cast<const float4*>(x + ((live[j] ? rj * per_row + c : 0) * 32 + sub * 4));
        }
    };
    float4 v[kQuantRowsInFlight], ahead[kQuantRowsInFlight];
    bool live[kQuantRowsInFlight], live_ahead[kQuantRowsInFlight];
    fetch(blockIdx.y, v, live);
    for (long r = blockIdx.y; r < rows; r += kQuantRowsInFlight * step) {  // uniform over the workgroup
        fetch(r + kQuantRowsInFlight * step, ahead, live_ahead);       // nothing is live past the last row
#pragma unroll
        for (int j = 0; j < kQuantRowsInFlight; ++j)
            if (r + j * step < rows) finish(r + j * step, v[j], live[j]);
#pragma unroll
        for (int j = 0; j < kQuantRowsInFlight; ++j) {
            v[j] = ahead[j];
            live[j] = live_ahead[j];
        }
    }
}

// payload[i] = code of x[i] * scale_inv[i / 32]; four values per thread.
__global__ void __launch_bounds__(256) encode_hidden_kernel(const float* __restrict__ x, const float* __restrict__ scale_inv,
                                                            uint8_t* __restrict__ payload, int64_t n_elem) {
    const int64_t stride = int64_t(gridDim.x) * blockDim.x * 4;
    for (int64_t i = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) * 4; i < n_elem; i += stride) {
        if (i + 4 <= n_elem) {
            const float4 v = *reinterpret_cast<const float4*>(x + i);
            const float s = scale_inv[i >> 5];
            *reinterpret_cast<uint32_t*>(payload + i) = e4m3_half_up4(v, s);
        } else {
            for (int64_t j = i; j < n_elem; ++j) payload[j] = uint8_t(e4m3_half_up(x[j], scale_inv[j >> 5]));
        }
    }
}

// ---- request frame ----------------------------------------------------------------------------------
// The body of a request frame behind its header and row descriptors: t * topk route entries of twelve
// bytes (row, expert, weight bits) and t hidden rows (hid payload bytes, then hid / 32 scale bytes) at
// `pitch`. The first `row_groups` workgroups move hidden rows, one wave per token: payload and scale rows
// are read in 16-byte pieces, 1 KB per wave and step, and written as two 8-byte halves, because a frame's
// hidden rows start on 8-byte boundaries only. The remaining workgroups write the route entries, one
// route per lane; an entry is three dwords at a 4-byte boundary.
__global__ void __launch_bounds__(256) frame_fill_kernel(const int* __restrict__ idx, const float* __restrict__ wts,
                                                         const uint8_t* __restrict__ payload, const uint8_t* __restrict__ scales,
                                                         int t, int topk, int hid, uint8_t* __restrict__ routes,
                                                         uint8_t* __restrict__ hidden, int pitch, int row_groups) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (int(blockIdx.x) < row_groups) {
        const int token = blockIdx.x * 4 + wave;
        if (token >= t) return;
        uint8_t* dst = hidden + size_t(token) * pitch;
        const uint4* src = reinterpret_cast<const uint4*>(payload + size_t(token) * hid);
        for (int piece = lane; piece < hid / 16; piece += 64) {
            const uint4 v = src[piece];
            uint2* out = reinterpret_cast<uint2*>(dst + piece * 16);
            out[0] = make_uint2(v.x, v.y);
            out[1] = make_uint2(v.z, v.w);
        }
        const uint2* ssrc = reinterpret_cast<const uint2*>(scales + size_t(token) * (hid / 32));
        for (int piece = lane; piece < hid / 256; piece += 64)
            reinterpret_cast<uint2*>(dst + hid)[piece] = ssrc[piece];
        return;
    }
    const long route = long(blockIdx.x - row_groups) * 256 + threadIdx.x;
    if (route >= long(t) * topk) return;
    uint32_t* entry = reinterpret_cast<uint32_t*>(routes + route * 12);
    entry[0] = uint32_t(route / topk);
    entry[1] = uint32_t(idx[route]);
    entry[2] = __float_as_uint(wts[route]);
}

// ---- rank sum, residual, BF16 cast -----------------------------------------------------------------
__device__ __forceinline__ float bf16_value(uint32_t bits) { return __uint_as_float(bits << 16); }

// The three kernels below move eight values per lane and step in 16-byte accesses when every pointer is
// 16-byte aligned (VEC; the host checks), one value per lane otherwise; the last n % 8 values are taken one
// by one by the first lanes of the grid.
template <typename F>
__device__ __forceinline__ void each_eight(long n, F&& body8, bool vec) {
    const long tid = long(blockIdx.x) * blockDim.x + threadIdx.x, threads = long(gridDim.x) * blockDim.x;
    const long groups = vec ? n / 8 : 0;
    for (long g = tid; g < groups; g += threads) body8(g * 8, true);
    for (long i = groups * 8 + tid; i < n; i += threads) body8(i, false);
}

// s = 0; s += rank 0, 1, 2, 3: four separate FP32 additions, in that order.
__device__ __forceinline__ float rank_sum4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    float s = 0.0f;
    s = __fadd_rn(s, bf16_value(a));
    s = __fadd_rn(s, bf16_value(b));
    s = __fadd_rn(s, bf16_value(c));
    return __fadd_rn(s, bf16_value(d));
}
template <bool VEC>
__global__ void __launch_bounds__(256) rank_sum_bf16_kernel(const uint16_t* __restrict__ p0, const uint16_t* __restrict__ p1,
                                                            const uint16_t* __restrict__ p2, const uint16_t* __restrict__ p3,
                                                            float* __restrict__ out, long n) {
    each_eight(n, [&](long i, bool eight) {
        if (!eight) {
            out[i] = rank_sum4(p0[i], p1[i], p2[i], p3[i]);
            return;
        }
        const uint4 a = *reinterpret_cast<const uint4*>(p0 + i), b = *reinterpret_cast<const uint4*>(p1 + i),
                    c = *reinterpret_cast<const uint4*>(p2 + i), d = *reinterpret_cast<const uint4*>(p3 + i);
        const uint32_t wa[4] = {a.x, a.y, a.z, a.w}, wb[4] = {b.x, b.y, b.z, b.w}, wc[4] = {c.x, c.y, c.z, c.w}, wd[4] = {d.x, d.y, d.z, d.w};
        float o[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {  // a dword holds two values, the lower address in the low half
            o[2 * j] = rank_sum4(wa[j] & 0xffffu, wb[j] & 0xffffu, wc[j] & 0xffffu, wd[j] & 0xffffu);
            o[2 * j + 1] = rank_sum4(wa[j] >> 16, wb[j] >> 16, wc[j] >> 16, wd[j] >> 16);
        }
        *reinterpret_cast<float4*>(out + i) = make_float4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<float4*>(out + i + 4) = make_float4(o[4], o[5], o[6], o[7]);
    }, VEC);
}

template <bool VEC>
__global__ void __launch_bounds__(256) add_inplace_kernel(float* __restrict__ h, const float* __restrict__ a, long n) {
    each_eight(n, [&](long i, bool eight) {
        if (!eight) {
            h[i] = __fadd_rn(h[i], a[i]);
            return;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float4 u = *reinterpret_cast<const float4*>(h + i + 4 * j), v = *reinterpret_cast<const float4*>(a + i + 4 * j);
            *reinterpret_cast<float4*>(h + i + 4 * j) =
                make_float4(__fadd_rn(u.x, v.x), __fadd_rn(u.y, v.y), __fadd_rn(u.z, v.z), __fadd_rn(u.w, v.w));
        }
    }, VEC);
}

// Round to nearest even; a NaN becomes 0x7fff, as the reference's conversion intrinsic gives.
__device__ __forceinline__ uint32_t bf16_rne_nan(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x7fffffffu) > 0x7f800000u ? 0x7fffu : (b + 0x7fffu + ((b >> 16) & 1u)) >> 16;
}
template <bool VEC>
__global__ void __launch_bounds__(256) f32_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, long n) {
    each_eight(n, [&](long i, bool eight) {
        if (!eight) {
            y[i] = uint16_t(bf16_rne_nan(x[i]));
            return;
        }
        const float4 u = *reinterpret_cast<const float4*>(x + i), v = *reinterpret_cast<const float4*>(x + i + 4);
        *reinterpret_cast<uint4*>(y + i) = make_uint4(bf16_rne_nan(u.x) | bf16_rne_nan(u.y) << 16, bf16_rne_nan(u.z) | bf16_rne_nan(u.w) << 16,
                                                      bf16_rne_nan(v.x) | bf16_rne_nan(v.y) << 16, bf16_rne_nan(v.z) | bf16_rne_nan(v.w) << 16);
    }, VEC);
}

}  // namespace m26g
