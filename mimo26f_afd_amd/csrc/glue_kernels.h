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
// One wave per row; lane l holds experts l, l+64, ... (at most 16 of them, n_experts <= 1024).
// Scores and the selection run in binary64 like the reference; the k selections are k wave-wide
// arg-max rounds on (score + bias, lower id wins ties). Weights: unbiased score / sum, the sum taken
// in selection order, rounded to binary32.
constexpr int kRouterPerLane = 16;

__device__ __forceinline__ void wave_argmax(double& v, int& i) {
#pragma unroll
    for (int d = 32; d; d >>= 1) {
        const double ov = __shfl_xor(v, d);
        const int oi = __shfl_xor(i, d);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

__global__ void __launch_bounds__(256) router_topk_kernel(const float* __restrict__ logits, const float* __restrict__ bias,
                                                          int rows, int n_experts, int top_k, int* __restrict__ idx_out,
                                                          float* __restrict__ w_out) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float* lrow = logits + size_t(row) * n_experts;
    double score[kRouterPerLane], sel[kRouterPerLane];
#pragma unroll
    for (int j = 0; j < kRouterPerLane; ++j) {
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
        double v = -INFINITY;
        int i = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < kRouterPerLane; ++j) {  // ascending ids: a strict > keeps the lower id on ties
            const int e = lane + 64 * j;
            if (e < n_experts && sel[j] > v) { v = sel[j]; i = e; }
        }
        wave_argmax(v, i);
        const int owner = i & 63, slot = i >> 6;
        double s = 0.0;
#pragma unroll
        for (int j = 0; j < kRouterPerLane; ++j)
            if (j == slot && lane == owner) { s = score[j]; sel[j] = -INFINITY; }
        s = __shfl(s, owner);
        wsum += s;
        if (lane == k) { mine = s; mine_id = i; }
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
// has already underflowed to -0 (the CPU rule multiplies in binary64). Integer arithmetic on the
// significand: round-half-up is an add and a shift.
__device__ __forceinline__ uint32_t e4m3_half_up(float x, float scale) {
    const float y = x * scale;
    if (y != y) return 0;
    const uint32_t sign = x < 0.0f ? 0x80u : 0u;
    float mag = fabsf(y);
    mag = mag > 448.0f ? 448.0f : mag;
    const uint32_t bits = __float_as_uint(mag), field = bits >> 23;
    if (field < 127 - 11) return sign;  // below 2^-11: under half the smallest step (zero and subnormals too)
    const int e = int(field) - 127;
    const uint32_t sig = (bits & 0x7fffffu) | 0x800000u;  // value = sig * 2^(e - 23)
    if (e < -6) {                                          // quantum 2^-9: code = floor(value * 512 + 1/2)
        const int sh = 14 - e;                             // >= 21
        return sign | ((sig + (1u << (sh - 1))) >> sh);    // 8 is the smallest normal code
    }
    uint32_t q = (sig + 0x80000u) >> 20;                   // 8 .. 16
    uint32_t ee = uint32_t(e + 7);
    if (q == 16) { q = 8; ++ee; }
    const uint32_t code = (ee << 3) | (q - 8);
    return sign | (code > 0x7eu ? 0x7eu : code);
}

// One K32 block per 8 lanes, four values per lane. grid-stride over blocks.
__global__ void __launch_bounds__(256) quantize_hidden_kernel(const float* __restrict__ x, long rows, int cols,
                                                              uint8_t* __restrict__ payload, size_t payload_pitch,
                                                              uint8_t* __restrict__ scales, size_t scales_pitch,
                                                              float* __restrict__ scale_inv) {
    const int sub = threadIdx.x & 7, per_row = cols / 32;
    const long blocks = rows * per_row;
    const long stride = (long(gridDim.x) * blockDim.x) >> 3;
    // Whole waves walk together: the shuffles below need all eight lanes of a block present.
    const long first = (long(blockIdx.x) * blockDim.x + threadIdx.x) >> 3;
    const long rounds = (blocks + stride - 1) / stride;
    for (long it = 0; it < rounds; ++it) {
        const long b = first + it * stride;
        const bool live = b < blocks;
        const long r = live ? b / per_row : 0, c = live ? b % per_row : 0;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) v = *reinterpret_cast<const float4*>(x + (r * cols + c * 32 + sub * 4));
        // NaNs take no part in amax. They are zeroed first: a signalling NaN would come out of the
        // hardware maximum as a quiet one and wipe what was gathered before it.
        auto mag = [](float f) { return f != f ? 0.0f : fabsf(f); };
        float amax = fmaxf(fmaxf(mag(v.x), mag(v.y)), fmaxf(mag(v.z), mag(v.w)));
#pragma unroll
        for (int d = 4; d; d >>= 1) amax = fmaxf(amax, __shfl_xor(amax, d));
        const uint32_t s = q0_scale_byte(amax);
        // 2^(127 - s): exponent field 254 - s; s = 254 is 2^-127, the subnormal with the top mantissa bit
        const float scale = __uint_as_float(s == 254u ? 0x00400000u : (254u - s) << 23);
        if (!live) continue;
        const uint32_t word = e4m3_half_up(v.x, scale) | e4m3_half_up(v.y, scale) << 8 | e4m3_half_up(v.z, scale) << 16 |
                              e4m3_half_up(v.w, scale) << 24;
        if (payload) *reinterpret_cast<uint32_t*>(payload + r * payload_pitch + c * 32 + sub * 4) = word;
        if (sub == 0) {
            if (scales) scales[r * scales_pitch + c] = uint8_t(s);
            if (scale_inv) scale_inv[b] = scale;
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
            *reinterpret_cast<uint32_t*>(payload + i) = e4m3_half_up(v.x, s) | e4m3_half_up(v.y, s) << 8 |
                                                        e4m3_half_up(v.z, s) << 16 | e4m3_half_up(v.w, s) << 24;
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

// s = 0; s += rank 0, 1, 2, 3: four separate FP32 additions, in that order.
__global__ void __launch_bounds__(256) rank_sum_bf16_kernel(const uint16_t* __restrict__ p0, const uint16_t* __restrict__ p1,
                                                            const uint16_t* __restrict__ p2, const uint16_t* __restrict__ p3,
                                                            float* __restrict__ out, long n) {
    for (long i = long(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += long(gridDim.x) * blockDim.x) {
        float s = 0.0f;
        s = __fadd_rn(s, bf16_value(p0[i]));
        s = __fadd_rn(s, bf16_value(p1[i]));
        s = __fadd_rn(s, bf16_value(p2[i]));
        s = __fadd_rn(s, bf16_value(p3[i]));
        out[i] = s;
    }
}

__global__ void __launch_bounds__(256) add_inplace_kernel(float* __restrict__ h, const float* __restrict__ a, long n) {
    for (long i = long(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += long(gridDim.x) * blockDim.x)
        h[i] = __fadd_rn(h[i], a[i]);
}

// Round to nearest even; a NaN becomes 0x7fff, as the reference's conversion intrinsic gives.
__global__ void __launch_bounds__(256) f32_to_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, long n) {
    for (long i = long(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += long(gridDim.x) * blockDim.x) {
        const uint32_t b = __float_as_uint(x[i]);
        y[i] = (b & 0x7fffffffu) > 0x7f800000u ? uint16_t(0x7fff) : uint16_t((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
    }
}

}  // namespace m26g
