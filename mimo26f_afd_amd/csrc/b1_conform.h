// Conforming arm of FC1 / FC2 for layers that hold exceptional weight scales.
//
// A weight scale byte outside [2, 252] does not mean to the block-scaled MFMA what the checkpoint
// format means by it: byte 255 is a NaN scale to the hardware where the format clamps it to 254, and
// the decoded weights of bytes 253..255 saturate at +-FLT_MAX before they are multiplied where the
// hardware multiplies by the unsaturated power of two. The one-time preparation flags such a layer,
// and its calls run here instead of on the matrix pipe: every weight is decoded to its binary32 value
// by the format's own rule (codebook[nibble] * 2^(min(s, 254) - 127), saturated, zero keeping its
// sign, subnormal results kept), every activation to its binary32 value, and the products are
// summed in binary64 in ascending k, then rounded to binary32 once. Each product of two binary32
// values is exact in binary64, so the sum is the CPU rule's own dot product.
//
// Reference counterparts: the decode-then-fmaf arm of dot32
// (crates/mimo26-expert/kernels/b1/grouped.cu:42-67), dot32_exceptional
// (crates/mimo26-spark/kernels/b1_fc1_m64.cuh:30-70), the decoder
// (crates/mimo26-expert/kernels/include/mimo26_expert_bits.h:29-40) and activation_value
// (kernels/b1/grouped.cu:33-41). The reference votes per MMA and switches arms inside a dot; here the
// whole layer takes this arm, so the matrix-pipe schedules carry no vote at all. Real checkpoints
// never come here (their scale bytes lie in 118..125).
//
// Both kernels walk the plan's groups, not its chunks: one workgroup per (group, 256 columns), one
// thread per column holding the sixteen rows' sums, the group's activations of one K32 block decoded
// once into LDS and read back by every thread. The same prepared image, plan, intermediate buffers,
// fault words and combine as the matrix-pipe path.
#pragma once
#include "b1_kernels.h"

namespace m26g {

// Twice the E2M1 magnitudes, one nibble each: 0, 1, 2, 3, 4, 6, 8, 12.
constexpr uint32_t kTwiceE2M1 = 0xC8643210u;

// 2^(min(s, 254) - 128): the factor that turns a doubled magnitude into the weight's value.
__device__ __forceinline__ double mxfp4_block_factor(uint32_t s) {
    return __builtin_ldexp(1.0, int(s > 254u ? 254u : s) - 128);
}
__device__ __forceinline__ double mxfp4_value(uint32_t nibble, double factor) {
    double v = double((kTwiceE2M1 >> (4 * (nibble & 7u))) & 15u) * factor;  // exact
    v = v > double(FLT_MAX) ? double(FLT_MAX) : v;
    return (nibble & 8u) ? -v : v;
}

// E4M3FN code at UE8M0 scale byte s as binary32: NaN for codes 0x7f / 0xff and for a scale outside
// the legal window [105, 247]; a value past FLT_MAX becomes an infinity, as the CPU rule's ldexpf gives.
__device__ __forceinline__ float activation_value(uint32_t code, uint32_t s) {
    if ((code & 0x7fu) == 0x7fu || (s - 105u) > 142u) return __uint_as_float(0x7fc00000u);
    const int e = int(code >> 3) & 15, m = int(code & 7u);
    const float v = __builtin_ldexpf(float(e ? 8 + m : m), int(s) - 127 + (e ? e - 10 : -9));
    return (code & 0x80u) ? -v : v;
}

// Byte offsets inside a prepared image of the 16 payload bytes and of the scale byte of K32 block kb of
// weight row `n`: tile t of column block `block` (32 rows of gate/up with t = 0,1 gate and 2,3 up; 64 rows
// of down), `ksteps` k-steps per block.
struct WeightCell { uint64_t payload, scale; };
__device__ __forceinline__ WeightCell weight_cell(uint32_t block, uint32_t t, uint32_t row16, uint32_t kb, uint32_t ksteps) {
    const uint32_t ks = kb >> 2, lane = 16 * (kb & 3u) + row16;
    return WeightCell{block_payload(block, ksteps) + uint64_t(ks) * kStepBytes + t * 1024 + lane * 16,
                      ((uint64_t(block) * (ksteps / 4) + (ks >> 2)) * 4 + t) * 256 + lane * 4 + (ks & 3u)};
}

constexpr uint32_t kConformColumns = 256;  // columns (threads) per workgroup

// acc[r] += x[r][k] * w[k] for the 32 k of one block; `nibbles` are the 16 payload bytes, low nibble first.
__device__ __forceinline__ void conform_block(double (&acc)[16], const uint4 nibbles, double factor,
                                              const float (*xt)[16]) {
    const uint32_t word[4] = {nibbles.x, nibbles.y, nibbles.z, nibbles.w};
#pragma unroll
    for (int k = 0; k < 32; ++k) {
        const double w = mxfp4_value((word[k >> 3] >> (4 * (k & 7))) & 15u, factor);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = __builtin_fma(double(xt[k][r]), w, acc[r]);
    }
}

// FC1 + SwiGLU + quantizer v1. grid (I / 256, group capacity), 256 threads.
__global__ void __launch_bounds__(kConformColumns) fc1_conform_kernel(Fc1Args a) {
    __shared__ float xt[32][16];                     // one K32 block of the group's rows, k-major
    __shared__ float hrow[16][kConformColumns + 1];  // the activation's output, for the quantizer
    __shared__ int32_t token[16];
    uint32_t* meta = a.plan.meta;
    const uint32_t gi = blockIdx.y, tid = threadIdx.x;
    if (meta[kPlanFault] || gi >= meta[kGroupCount]) return;
    const Group* G = a.plan.groups + gi;
    const int32_t expert = G->expert, rows = G->rows;
    if (expert < 0 || expert >= int32_t(kExperts) || rows < 1 || rows > 16) {
        if (tid == 0) atomicOr(&meta[kFc1Fault], 2u);
        return;
    }
    if (tid < 16) token[tid] = int32_t(tid) < rows ? G->input_rows[tid] : -1;
    const uint32_t I = a.lay.inter, n = blockIdx.x * kConformColumns + tid;
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* w13 = img + a.lay.w13();
    const uint8_t* s13 = img + a.lay.s13();
    double gate[16], up[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) gate[r] = up[r] = 0.0;
    for (uint32_t kb = 0; kb < kHidden / 32; ++kb) {
        __syncthreads();  // the block before has been read (and `token` written, first time round)
        for (uint32_t i = tid; i < 512; i += kConformColumns) {
            const uint32_t r = i >> 5, k = i & 31u;
            const int32_t row = token[r];
            xt[k][r] = row < 0 ? 0.0f
                               : activation_value(a.x[size_t(row) * a.x_pitch + kb * 32 + k], a.xs[size_t(row) * a.xs_pitch + kb]);
        }
        __syncthreads();
        const WeightCell cg = weight_cell(n >> 5, (n >> 4) & 1u, n & 15u, kb, kHidden / 128);
        const WeightCell cu = weight_cell(n >> 5, 2 + ((n >> 4) & 1u), n & 15u, kb, kHidden / 128);
        conform_block(gate, *reinterpret_cast<const uint4*>(w13 + cg.payload), mxfp4_block_factor(s13[cg.scale]), xt);
        conform_block(up, *reinterpret_cast<const uint4*>(w13 + cu.payload), mxfp4_block_factor(s13[cu.scale]), xt);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float g = float(gate[r]), u = float(up[r]), h = silu_up(g, u);
        hrow[r][tid] = h;
        if (a.tap_h && r < rows) {
            const size_t at = (size_t(gi) * 16 + r) * I + n;
            a.tap_gate[at] = g;
            a.tap_up[at] = u;
            a.tap_h[at] = h;
        }
    }
    __syncthreads();
    // Quantizer v1, one thread per (row, K32 block of the 256 columns): 16 x 8 of them.
    if (tid < 16 * (kConformColumns / 32)) {
        const uint32_t r = tid / (kConformColumns / 32), b = tid % (kConformColumns / 32);
        if (int32_t(r) >= rows) return;
        uint32_t amax = 0;
        for (int j = 0; j < 32; ++j) {
            const uint32_t m = __float_as_uint(hrow[r][b * 32 + j]) & 0x7fffffffu;
            amax = m > amax ? m : amax;
        }
        const size_t grow = size_t(gi) * 16 + r;
        const uint32_t cb = blockIdx.x * (kConformColumns / 32) + b, block = uint32_t(grow * (I / 32) + cb);
        uint32_t fault = amax >= 0x7f800000u ? 1u : 0u;
        const int k = quant_scale_exponent(amax);
        uint32_t code[32];
        if (!fault)
            for (int j = 0; j < 32; ++j) {
                code[j] = quant_code(hrow[r][b * 32 + j], k);
                if (!quant_reconstructs(code[j], k)) fault = 2;
            }
        if (fault) {
            atomicOr(&meta[kQuantFault], fault);
            atomicMin(&meta[kQuantWhere], block);
            return;  // a faulting block publishes no bytes
        }
        uint32_t* out = reinterpret_cast<uint32_t*>(a.dq + grow * I + size_t(cb) * 32);
        for (int j = 0; j < 8; ++j)
            out[j] = code[4 * j] | code[4 * j + 1] << 8 | code[4 * j + 2] << 16 | code[4 * j + 3] << 24;
        a.dqs[grow * (I / 32) + cb] = uint8_t(k + 127);
    }
}

// FC2 + inverse scatter. grid (4096 / 256, group capacity), 256 threads.
__global__ void __launch_bounds__(kConformColumns) fc2_conform_kernel(Fc2Args a) {
    __shared__ float xt[32][16];
    uint32_t* meta = a.plan.meta;
    const uint32_t gi = blockIdx.y, tid = threadIdx.x;
    if (meta[kPlanFault] || meta[kFc1Fault] || meta[kQuantFault] || gi >= meta[kGroupCount]) return;
    const Group* G = a.plan.groups + gi;
    const int32_t expert = G->expert, rows = G->rows, base = G->route_base;
    if (expert < 0 || expert >= int32_t(kExperts) || rows < 1 || rows > 16 || base < 0) {
        if (tid == 0) atomicOr(&meta[kFc2Fault], 2u);
        return;
    }
    const uint32_t I = a.lay.inter, n = blockIdx.x * kConformColumns + tid;
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* w2 = img + a.lay.w2();
    const uint8_t* s2 = img + a.lay.s2();
    double acc[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0;
    for (uint32_t kb = 0; kb < I / 32; ++kb) {
        __syncthreads();
        for (uint32_t i = tid; i < 512; i += kConformColumns) {
            const uint32_t r = i >> 5, k = i & 31u;
            const size_t grow = size_t(gi) * 16 + r;
            xt[k][r] = int32_t(r) < rows ? activation_value(a.dq[grow * I + kb * 32 + k], a.dqs[grow * (I / 32) + kb]) : 0.0f;
        }
        __syncthreads();
        const WeightCell c = weight_cell(n >> 6, (n >> 4) & 3u, n & 15u, kb, I / 128);
        conform_block(acc, *reinterpret_cast<const uint4*>(w2 + c.payload), mxfp4_block_factor(s2[c.scale]), xt);
    }
    bool lost = false;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        if (r >= rows) continue;
        const int32_t route = a.plan.original[base + r];
        if (route < 0 || uint32_t(route) >= a.routes) { lost = true; continue; }
        if (a.y_bf16) reinterpret_cast<uint16_t*>(a.y)[size_t(route) * kHidden + n] = uint16_t(bf16_bits_rne(float(acc[r])));
        else a.y[size_t(route) * kHidden + n] = float(acc[r]);
    }
    if (lost) atomicOr(&meta[kFc2Fault], 5u);
}

}  // namespace m26g
