// gfx950 kernels of the routed-expert FFN (B1, numerical mode E-W4A8-v1).
//
// Stage map against the reference (paths relative to the reference repository):
//   prepare_kernel  <- crates/mimo26-expert/kernels/b1/prepare.cu:39-57 (one-time byte permutation)
//                      + crates/mimo26-spark/kernels/b1_fc1_m64.cuh:496-512 (scale scan)
//   plan_kernel     <- crates/mimo26-expert/kernels/b1/group_plan.cu:32-79 (stable plan, the spec)
//                      + crates/mimo26-spark/kernels/b1_serve.cu:36-96 (one-CTA serving planner, chunks)
//   fc1_kernel      <- kernels/b1/grouped.cu:74-113 + connected.cu:9-37 (gate/up MMA + SwiGLU)
//                      fused with kernels/b1/quant_v1.cu:34-68 (intermediate quantizer v1)
//   fc2_kernel      <- kernels/b1/grouped.cu:135-154 + connected.cu:48-79 (down MMA + inverse scatter)
//   reduce_kernel   <- kernels/b1/route_reduce.cu:61-124 (weight-once slot-ordered sum, BF16 RNE); the same
//                      arithmetic (combine4) runs inside the FC2 kernels when the combine is fused
//                      (combine_completed), and on BF16 per-route rows in the opt-in mode of
//                      crates/mimo26-spark/kernels/b1_serve.cu:98-143
//   quantize_kernel <- kernels/b1/quant_v1.cu:34-68 (stand-alone form, same device functions)
#pragma once
#include <hip/hip_runtime.h>
#include <float.h>
#include "b1_layout.h"

namespace m26g {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t v2u __attribute__((ext_vector_type(2)));

struct Canonical {
    const uint8_t* pool[4];  // ranks x (256 quarter-slice images)
    uint32_t ranks;          // 1 or 4
};

struct PlanView {
    int32_t* inverse;
    int32_t* original;
    float* gw;
    Group* groups;
    Chunk* chunks;
    uint32_t* meta;
    uint32_t* done;  // [rows][64] completion counts of the fused combine (see combine_completed), or null
};

// ---------------------------------------------------------------------------------------------
// One-time weight preparation: canonical v2 rank images -> the G950 operand order.
// grid (any, 256 experts), 256 threads. Pure byte moves; *abnormal is OR-ed with 1 when a weight
// scale byte lies outside [2, 252].
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) prepare_kernel(Canonical c, uint8_t* __restrict__ prepared, Prepared lay,
                                                      uint32_t* __restrict__ abnormal) {
    const uint32_t e = blockIdx.y, I = lay.inter;
    uint8_t* dst = prepared + uint64_t(e) * lay.bytes();
    const uint64_t img = uint64_t(e) * kImageBytes;
    const uint32_t stride = gridDim.x * blockDim.x, first = blockIdx.x * blockDim.x + threadIdx.x;
    bool odd = false;
    for (uint32_t cell = first; cell < I * 256; cell += stride) {  // w13 payload
        const uint32_t lane = cell & 63, t = (cell >> 6) & 3, ks = (cell >> 11) & 31, cb = (cell >> 16) * kSetBlocks + ((cell >> 8) & 7);
        const uint32_t n = cb * 32 + (t & 1) * 16 + (lane & 15), g = lane >> 4;
        const uint8_t* src = c.pool[n / kRankI] + img + (t < 2 ? kGatePayload : kUpPayload) +
                             uint64_t(n % kRankI) * 2048 + ks * 64 + g * 16;
        *reinterpret_cast<uint4*>(dst + lay.w13() + uint64_t(cell) * 16) = *reinterpret_cast<const uint4*>(src);
    }
    for (uint32_t cell = first; cell < I * 64; cell += stride) {  // w13 scales
        const uint32_t lane = cell & 63, t = (cell >> 6) & 3, q = (cell >> 8) & 7, cb = cell >> 11;
        const uint32_t n = cb * 32 + (t & 1) * 16 + (lane & 15), g = lane >> 4;
        const uint8_t* src = c.pool[n / kRankI] + img + (t < 2 ? kGateScales : kUpScales) + uint64_t(n % kRankI) * 128;
        uint32_t word = 0;
        for (uint32_t b = 0; b < 4; ++b) {
            const uint32_t s = src[4 * (4 * q + b) + g];
            odd = odd || s < 2 || s > 252;
            word |= s << (8 * b);
        }
        *reinterpret_cast<uint32_t*>(dst + lay.s13() + uint64_t(cell) * 4) = word;
    }
    const uint32_t ksteps = I / 128, quads = I / 512;
    for (uint32_t cell = first; cell < I * 128; cell += stride) {  // w2 payload
        const uint32_t lane = cell & 63, t = (cell >> 6) & 3, ks = (cell >> 11) % ksteps;
        const uint32_t ob = (cell >> 11) / ksteps * kSetBlocks + ((cell >> 8) & 7);
        const uint32_t n = ob * 64 + t * 16 + (lane & 15), kb = 4 * ks + (lane >> 4);
        const uint8_t* src = c.pool[kb / 16] + img + kDownPayload + uint64_t(n) * 256 + (kb % 16) * 16;
        *reinterpret_cast<uint4*>(dst + lay.w2() + uint64_t(cell) * 16) = *reinterpret_cast<const uint4*>(src);
    }
    for (uint32_t cell = first; cell < I * 32; cell += stride) {  // w2 scales
        const uint32_t lane = cell & 63, t = (cell >> 6) & 3, q = (cell >> 8) % quads, ob = (cell >> 8) / quads;
        const uint32_t n = ob * 64 + t * 16 + (lane & 15), g = lane >> 4;
        uint32_t word = 0;
        for (uint32_t b = 0; b < 4; ++b) {
            const uint32_t kb = 4 * (4 * q + b) + g;
            const uint32_t s = c.pool[kb / 16][img + kDownScales + uint64_t(n) * 16 + kb % 16];
            odd = odd || s < 2 || s > 252;
            word |= s << (8 * b);
        }
        *reinterpret_cast<uint32_t*>(dst + lay.s2() + uint64_t(cell) * 4) = word;
    }
    if (odd) atomicOr(abnormal, 1u);
}

// ---------------------------------------------------------------------------------------------
// Stage 1: token -> expert bucketing. One workgroup of 1024 threads, LDS counting sort.
//
// Bit-exact with the reference's serial planner: routes of one expert keep ascending route order.
// Each of the 16 waves owns one contiguous run of routes; a wave ranks its 64 routes per step with
// ballots (no atomics touch a position), per-wave histograms give every wave its start inside each
// expert, and the second walk places routes. Dynamic LDS holds one id byte per route.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kPlanThreads = 1024, kPlanWaves = kPlanThreads / 64;
constexpr uint32_t kDoneBlocks = kHidden / 64;  // completion counts per token: one per 64 output columns

__device__ __forceinline__ uint64_t same_expert_lanes(uint32_t e, bool valid) {
    uint64_t m = __ballot(valid);
#pragma unroll
    for (uint32_t b = 0; b < 8; ++b) {
        const bool bit = (e >> b) & 1u;
        const uint64_t have = __ballot(bit);
        m &= bit ? have : ~have;
    }
    return m;
}

// Exclusive scan of 256 values held 4 per lane by one wave; writes base[0..256].
__device__ __forceinline__ void wave_scan256(const uint32_t (&v)[4], uint32_t* base, uint32_t lane) {
    const uint32_t total = v[0] + v[1] + v[2] + v[3];
    uint32_t incl = total;
#pragma unroll
    for (uint32_t d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
    }
    uint32_t run = incl - total;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        base[4 * lane + j] = run;
        run += v[j];
    }
    if (lane == 63) base[256] = run;
}

__device__ __forceinline__ uint32_t last_not_above(const uint32_t* base, uint32_t value) {
    uint32_t lo = 0, hi = 256;  // largest e in [0,256) with base[e] <= value
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (base[mid] <= value) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ void __launch_bounds__(kPlanThreads)
plan_kernel(const int32_t* __restrict__ ids, const float* __restrict__ w, uint32_t rows,
            const uint8_t* __restrict__ resident, PlanView p, uint32_t gpc, uint32_t reset_capacity, bool want_gw) {
    extern __shared__ __align__(16) uint8_t id_byte[];
    __shared__ uint32_t hist[kPlanWaves][256];
    __shared__ uint32_t cnt[256], rbase[257], gbase[257], cbase[257];
    __shared__ uint32_t first_bad;
    __shared__ uint8_t present[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, routes = rows * kTopk;

    // Validation keys order faults as the serial planner meets them: (route + 1) << 4 | check,
    // check 1 = id or residency, 2 = weight, 3 = expert repeated inside the token.
    // One token (its eight routes) per thread and trip, two trips in flight: the walk is bound by the
    // latency of these loads, not by their volume. The first trip's loads are asked for ahead of everything else
    // (the checks need the residency bytes in LDS first): one memory latency for both instead of one after the other.
    typedef v4i __attribute__((aligned(4))) v4i_u;
    typedef v4f __attribute__((aligned(4))) v4f_u;
    const v4i_u* ids4 = reinterpret_cast<const v4i_u*>(ids);
    const v4f_u* w4 = reinterpret_cast<const v4f_u*>(w);
    struct Trip { v4i ia, ib, ic, id; v4f wa, wb, wc, wd; };
    auto fetch = [&](uint32_t t) {
        const uint32_t u = t + kPlanThreads;
        const bool two = u < rows;
        return Trip{ids4[2 * t], ids4[2 * t + 1], ids4[two ? 2 * u : 2 * t], ids4[two ? 2 * u + 1 : 2 * t + 1],
                    w4[2 * t], w4[2 * t + 1], w4[two ? 2 * u : 2 * t], w4[two ? 2 * u + 1 : 2 * t + 1]};
    };
    Trip first{};
    if (tid < rows) first = fetch(tid);
    const uint8_t here = tid < 256 ? resident[tid] : uint8_t(0);
    for (uint32_t i = tid; i < kPlanWaves * 256; i += kPlanThreads) (&hist[0][0])[i] = 0;
    if (tid == 0) first_bad = 0xffffffffu;
    if (tid < 256) present[tid] = here;
    if (p.done)  // every call starts its completion counts from zero, whatever the call before left
        for (uint32_t i = tid; i < rows * kDoneBlocks; i += kPlanThreads) p.done[i] = 0;
    __syncthreads();
    if (here > 1) atomicMin(&first_bad, 1u);
    auto check_token = [&](uint32_t t, const v4i& ia, const v4i& ib, const v4f& wa, const v4f& wb) {
        const int32_t e8[8] = {ia.x, ia.y, ia.z, ia.w, ib.x, ib.y, ib.z, ib.w};
        const float w8[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
        uint32_t packed[2] = {0, 0};
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const int32_t e = e8[j];
            uint32_t check = 0;
            if (e < 0 || e >= int32_t(kExperts) || !present[e & 255]) check = 1;
            else if (!(w8[j] >= 0.0f && w8[j] <= FLT_MAX)) check = 2;
            if (check) atomicMin(&first_bad, ((t * 8 + j + 1) << 4) | check);
            packed[j >> 2] |= (uint32_t(e) & 0xffu) << (8 * (j & 3));
        }
        *reinterpret_cast<uint2*>(id_byte + t * 8) = uint2{packed[0], packed[1]};
    };
    for (uint32_t t = tid; t < rows; t += 2 * kPlanThreads) {
        const Trip trip = t == tid ? first : fetch(t);
        check_token(t, trip.ia, trip.ib, trip.wa, trip.wb);
        if (t + kPlanThreads < rows) check_token(t + kPlanThreads, trip.ic, trip.id, trip.wc, trip.wd);
    }
    __syncthreads();
    const uint32_t run = (((routes + kPlanWaves - 1) / kPlanWaves) + 63u) & ~63u;
    const uint32_t begin = wv * run, end = begin + run < routes ? begin + run : routes;
    for (uint32_t s = begin; s < end; s += 64) {
        const uint32_t i = s + lane;
        const bool valid = i < routes;
        const uint32_t e = valid ? id_byte[i] : 0;
        const uint64_t m = same_expert_lanes(e, valid);
        const uint64_t below = m & ((1ull << lane) - 1);
        if (valid) {
            if (below & (0xffull << (lane & ~7u))) atomicMin(&first_bad, ((i + 1) << 4) | 3u);
            if (!below) hist[wv][e] += __popcll(m);
        }
    }
    __syncthreads();
    if (first_bad != 0xffffffffu) {
        if (tid == 0) {
            const uint32_t check = first_bad & 15u;
            p.meta[kPlanFault] = check == 2 ? 8u : 7u;  // Status::nonfinite : Status::metadata
            p.meta[kGroupCount] = 0;
            p.meta[kChunkCount] = 0;
        }
        return;
    }
    // The serial planner rewrites every capacity slot once the routes are accepted (inverse /
    // original = -1, weights = 0, groups = {-1, 0, -1, {-1 x 16}}). Only the stand-alone plan entry
    // asks for it; the FFN kernels never read past the live counts.
    for (uint32_t i = tid; i < reset_capacity * 19; i += kPlanThreads) {
        reinterpret_cast<int32_t*>(p.groups)[i] = (i % 19 == 1) ? 0 : -1;
        if (i < reset_capacity) {
            p.inverse[i] = -1;
            p.original[i] = -1;
            p.gw[i] = 0.0f;
        }
    }
    if (tid < 256) {
        uint32_t acc = 0;
        for (uint32_t k = 0; k < kPlanWaves; ++k) {
            const uint32_t t = hist[k][tid];
            hist[k][tid] = acc;
            acc += t;
        }
        cnt[tid] = acc;
    }
    __syncthreads();
    if (wv == 0) {
        uint32_t a[4], b[4], c[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            a[j] = cnt[4 * lane + j];
            b[j] = (a[j] + 15) / 16;
            c[j] = (b[j] + gpc - 1) / gpc;
        }
        wave_scan256(a, rbase, lane);
        wave_scan256(b, gbase, lane);
        wave_scan256(c, cbase, lane);
    }
    __syncthreads();
    for (uint32_t s = begin; s < end; s += 64) {
        const uint32_t i = s + lane;
        const bool valid = i < routes;
        const uint32_t e = valid ? id_byte[i] : 0;
        const uint64_t m = same_expert_lanes(e, valid);
        const uint64_t below = m & ((1ull << lane) - 1);
        if (valid) {
            const uint32_t rel = hist[wv][e] + __popcll(below);
            const uint32_t pos = rbase[e] + rel;
            p.original[pos] = int32_t(i);
            p.inverse[i] = int32_t(pos);
            p.groups[gbase[e] + rel / 16].input_rows[rel % 16] = int32_t(i / kTopk);
            if (!below) hist[wv][e] += __popcll(m);
        }
    }
    __syncthreads();
    // Weights in grouped order: part of the planner's output, but nothing downstream reads it (the
    // combine takes the caller's weights by route), so the FFN path only fills it for the taps.
    if (want_gw)
        for (uint32_t s0 = tid; s0 < routes; s0 += 8 * kPlanThreads) {
            float wt[8];
            int32_t at[8];
#pragma unroll
            for (uint32_t j = 0; j < 8; ++j) {
                const uint32_t i = s0 + j * kPlanThreads;
                wt[j] = i < routes ? w[i] : 0.0f;
                at[j] = i < routes ? p.inverse[i] : -1;
            }
#pragma unroll
            for (uint32_t j = 0; j < 8; ++j)
                if (at[j] >= 0) p.gw[at[j]] = wt[j];
        }
    const uint32_t ngroups = gbase[256], nchunks = cbase[256];
    for (uint32_t gi = tid; gi < ngroups; gi += kPlanThreads) {
        const uint32_t e = last_not_above(gbase, gi), k = gi - gbase[e];
        const uint32_t left = cnt[e] - 16 * k, n = left < 16 ? left : 16;
        Group& G = p.groups[gi];
        G.expert = int32_t(e);
        G.rows = int32_t(n);
        G.route_base = int32_t(rbase[e] + 16 * k);
        for (uint32_t slot = n; slot < 16; ++slot) G.input_rows[slot] = -1;
    }
    for (uint32_t ci = tid; ci < nchunks; ci += kPlanThreads) {
        const uint32_t e = last_not_above(cbase, ci), j = ci - cbase[e];
        const uint32_t ng = (cnt[e] + 15) / 16, left = ng - gpc * j;
        p.chunks[ci] = Chunk{int32_t(gbase[e] + gpc * j), int32_t(left < gpc ? left : gpc), int32_t(e), 0};
    }
    // The fault word is left alone: a rejected plan of an earlier call on this scratch stays on record,
    // and keeps the stage kernels of every later call out, until the host has read and cleared it.
    if (tid == 0) {
        p.meta[kGroupCount] = ngroups;
        p.meta[kChunkCount] = nchunks;
    }
}

// ---------------------------------------------------------------------------------------------
// Stage 1 for large calls: the same stable counting sort spread over several compute units.
//
// One workgroup scatters its results through one memory pipeline; at 65536 routes the placement's
// three uncoalesced stores per route kept that pipeline busy for 0.1 ms. Here a wave still owns one
// contiguous run of routes (256 of them: wave w of all workgroups taken together owns routes
// [256 w, 256 w + 256)), so the order inside an expert is the serial planner's, and the work is cut
// into three launches on the stream:
//   plan_count_kernel  validates, and leaves every wave's per-expert counts in `work`;
//   plan_scan_kernel   (one workgroup) turns them into every wave's first position inside each
//                      expert, scans experts into route / group / chunk bases, fills group headers
//                      and chunks, publishes the counts or the fault;
//   plan_place_kernel  walks the routes again and places them.
// The sum over earlier waves is taken in two levels: the count kernel, which holds its sixteen waves' counts in
// LDS anyway, leaves every wave's start inside its own workgroup and the workgroup's totals; the scan turns the
// totals (one row per workgroup, sixteen at 8192 rows) into every workgroup's start; the placement adds the two.
// (Summed in one level by the scan alone, 256 rows of counts walked twice by one workgroup, the scan took 18 us.)
// work: [0] first fault key (0xffffffff = none; the scan re-arms it), [1..3] unused,
//       [4 ..) starts[wave][256] inside the wave's workgroup, then totals[workgroup][256] (which the scan turns
//       into the workgroups' starts), then route and group bases [2][257].
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kWideRoutesPerWave = 256, kWideRoutesPerGroup = kPlanWaves * kWideRoutesPerWave;
__host__ __device__ constexpr uint32_t wide_plan_groups(uint32_t routes) { return (routes + kWideRoutesPerGroup - 1) / kWideRoutesPerGroup; }
__host__ __device__ constexpr uint64_t wide_plan_words(uint32_t routes) {
    return 4 + uint64_t(wide_plan_groups(routes)) * (kPlanWaves + 1) * 256 + 2 * 257;
}

__global__ void __launch_bounds__(kPlanThreads)
plan_count_kernel(const int32_t* __restrict__ ids, const float* __restrict__ w, uint32_t rows,
                  const uint8_t* __restrict__ resident, uint32_t* __restrict__ work, uint32_t* __restrict__ done) {
    __shared__ __align__(16) uint8_t id_byte[kWideRoutesPerGroup];
    __shared__ uint32_t hist[kPlanWaves][256];
    __shared__ uint8_t present[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, routes = rows * kTopk;
    const uint32_t first_route = blockIdx.x * kWideRoutesPerGroup;
    for (uint32_t i = tid; i < kPlanWaves * 256; i += kPlanThreads) (&hist[0][0])[i] = 0;
    if (done)  // the completion counts of this workgroup's tokens start from zero
        for (uint32_t i = first_route / kTopk * kDoneBlocks + tid; i < (first_route + kWideRoutesPerGroup) / kTopk * kDoneBlocks && i < rows * kDoneBlocks; i += kPlanThreads)
            done[i] = 0;
    if (tid < 256) {
        const uint8_t here = resident[tid];
        if (here > 1 && blockIdx.x == 0) atomicMin(&work[0], 1u);
        present[tid] = here;
    }
    __syncthreads();
    const uint32_t t = first_route / kTopk + tid;  // one token per thread, the first half of the workgroup
    if (tid < kWideRoutesPerGroup / kTopk && t < rows) {
        typedef v4i __attribute__((aligned(4))) v4i_u;
        typedef v4f __attribute__((aligned(4))) v4f_u;
        const v4i ia = reinterpret_cast<const v4i_u*>(ids)[2 * t], ib = reinterpret_cast<const v4i_u*>(ids)[2 * t + 1];
        const v4f wa = reinterpret_cast<const v4f_u*>(w)[2 * t], wb = reinterpret_cast<const v4f_u*>(w)[2 * t + 1];
        const int32_t e8[8] = {ia.x, ia.y, ia.z, ia.w, ib.x, ib.y, ib.z, ib.w};
        const float w8[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
        uint32_t packed[2] = {0, 0};
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const int32_t e = e8[j];
            uint32_t check = 0;
            if (e < 0 || e >= int32_t(kExperts) || !present[e & 255]) check = 1;
            else if (!(w8[j] >= 0.0f && w8[j] <= FLT_MAX)) check = 2;
            if (check) atomicMin(&work[0], ((t * 8 + j + 1) << 4) | check);
            packed[j >> 2] |= (uint32_t(e) & 0xffu) << (8 * (j & 3));
        }
        *reinterpret_cast<uint2*>(id_byte + tid * 8) = uint2{packed[0], packed[1]};
    }
    __syncthreads();
#pragma unroll
    for (uint32_t step = 0; step < kWideRoutesPerWave / 64; ++step) {
        const uint32_t local = wv * kWideRoutesPerWave + step * 64 + lane, i = first_route + local;
        const bool valid = i < routes;
        const uint32_t e = valid ? id_byte[local] : 0;
        const uint64_t m = same_expert_lanes(e, valid);
        const uint64_t below = m & ((1ull << lane) - 1);
        if (valid) {
            if (below & (0xffull << (lane & ~7u))) atomicMin(&work[0], ((i + 1) << 4) | 3u);
            if (!below) hist[wv][e] += __popcll(m);
        }
    }
    __syncthreads();
    if (tid < 256) {  // per expert: every wave's start inside this workgroup, and the workgroup's total
        uint32_t* starts = work + 4 + uint64_t(blockIdx.x) * kPlanWaves * 256 + tid;
        uint32_t run = 0;
#pragma unroll
        for (uint32_t k = 0; k < kPlanWaves; ++k) {
            starts[k * 256] = run;
            run += hist[k][tid];
        }
        work[4 + uint64_t(gridDim.x) * kPlanWaves * 256 + blockIdx.x * 256 + tid] = run;
    }
}

__global__ void __launch_bounds__(kPlanThreads)
plan_scan_kernel(uint32_t routes, uint32_t* __restrict__ work, PlanView p, uint32_t gpc) {
    __shared__ uint32_t cnt[256], rbase[257], gbase[257], cbase[257];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const uint32_t waves = wide_plan_groups(routes) * kPlanWaves;
    const uint32_t first_bad = work[0];
    if (first_bad != 0xffffffffu) {
        __syncthreads();
        if (tid == 0) {
            p.meta[kPlanFault] = (first_bad & 15u) == 2 ? 8u : 7u;  // Status::nonfinite : Status::metadata
            p.meta[kGroupCount] = 0;
            p.meta[kChunkCount] = 0;
            work[0] = 0xffffffffu;
        }
        return;
    }
    // One thread per expert turns the workgroups' totals into the workgroups' starts (all loads first: the walk
    // is latency) and leaves the expert's row count.
    const uint32_t groups = wide_plan_groups(routes);
    uint32_t* totals = work + 4 + uint64_t(waves) * 256;
    if (tid < 256) {
        uint32_t t[kMaxRows * kTopk / kWideRoutesPerGroup];
#pragma unroll
        for (uint32_t g = 0; g < kMaxRows * kTopk / kWideRoutesPerGroup; ++g) t[g] = g < groups ? totals[g * 256 + tid] : 0;
        uint32_t run = 0;
#pragma unroll
        for (uint32_t g = 0; g < kMaxRows * kTopk / kWideRoutesPerGroup; ++g) {
            if (g < groups) totals[g * 256 + tid] = run;
            run += t[g];
        }
        cnt[tid] = run;
    }
    __syncthreads();
    if (wv == 0) {
        uint32_t a[4], b[4], c[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            a[j] = cnt[4 * lane + j];
            b[j] = (a[j] + 15) / 16;
            c[j] = (b[j] + gpc - 1) / gpc;
        }
        wave_scan256(a, rbase, lane);
        wave_scan256(b, gbase, lane);
        wave_scan256(c, cbase, lane);
    }
    __syncthreads();
    uint32_t* bases = work + 4 + uint64_t(waves + groups) * 256;
    for (uint32_t i = tid; i < 257; i += kPlanThreads) {
        bases[i] = rbase[i];
        bases[257 + i] = gbase[i];
    }
    const uint32_t ngroups = gbase[256], nchunks = cbase[256];
    for (uint32_t gi = tid; gi < ngroups; gi += kPlanThreads) {
        const uint32_t ex = last_not_above(gbase, gi), k = gi - gbase[ex];
        const uint32_t left = cnt[ex] - 16 * k, n = left < 16 ? left : 16;
        Group& G = p.groups[gi];
        G.expert = int32_t(ex);
        G.rows = int32_t(n);
        G.route_base = int32_t(rbase[ex] + 16 * k);
        for (uint32_t slot = n; slot < 16; ++slot) G.input_rows[slot] = -1;
    }
    for (uint32_t ci = tid; ci < nchunks; ci += kPlanThreads) {
        const uint32_t ex = last_not_above(cbase, ci), j = ci - cbase[ex];
        const uint32_t ng = (cnt[ex] + 15) / 16, left = ng - gpc * j;
        p.chunks[ci] = Chunk{int32_t(gbase[ex] + gpc * j), int32_t(left < gpc ? left : gpc), int32_t(ex), 0};
    }
    // The fault word is left alone: a rejected plan of an earlier call on this scratch stays on record,
    // and keeps the stage kernels of every later call out, until the host has read and cleared it.
    if (tid == 0) {
        p.meta[kGroupCount] = ngroups;
        p.meta[kChunkCount] = nchunks;
    }
}

__global__ void __launch_bounds__(kPlanThreads)
plan_place_kernel(const int32_t* __restrict__ ids, const float* __restrict__ w, uint32_t rows,
                  const uint32_t* __restrict__ work, PlanView p, bool want_gw) {
    __shared__ uint32_t start[kPlanWaves][256], rbase[257], gbase[257];
    if (p.meta[kPlanFault]) return;  // a rejected plan writes nothing
    const uint32_t tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, routes = rows * kTopk;
    const uint32_t waves = wide_plan_groups(routes) * kPlanWaves;
    const uint32_t* mine = work + 4 + (uint64_t(blockIdx.x) * kPlanWaves + wv) * 256;   // the wave's starts inside this workgroup
    const uint32_t* ours = work + 4 + uint64_t(waves) * 256 + blockIdx.x * 256;          // this workgroup's starts
    const uint32_t* bases = work + 4 + uint64_t(waves + gridDim.x) * 256;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) start[wv][lane + 64 * j] = mine[lane + 64 * j] + ours[lane + 64 * j];
    for (uint32_t i = tid; i < 257; i += kPlanThreads) {
        rbase[i] = bases[i];
        gbase[i] = bases[257 + i];
    }
    __syncthreads();
    const uint32_t first_route = blockIdx.x * kWideRoutesPerGroup + wv * kWideRoutesPerWave;
    int32_t e4[kWideRoutesPerWave / 64];
    float w4[kWideRoutesPerWave / 64];
#pragma unroll
    for (uint32_t step = 0; step < kWideRoutesPerWave / 64; ++step) {  // all loads first: the walk is short
        const uint32_t i = first_route + step * 64 + lane;
        e4[step] = i < routes ? ids[i] : 0;
        w4[step] = i < routes && want_gw ? w[i] : 0.0f;
    }
#pragma unroll
    for (uint32_t step = 0; step < kWideRoutesPerWave / 64; ++step) {
        const uint32_t i = first_route + step * 64 + lane;
        const bool valid = i < routes;
        const uint32_t e = uint32_t(e4[step]) & 255u;
        const uint64_t m = same_expert_lanes(e, valid);
        const uint64_t below = m & ((1ull << lane) - 1);
        if (valid) {
            const uint32_t rel = start[wv][e] + __popcll(below);
            const uint32_t pos = rbase[e] + rel;
            p.original[pos] = int32_t(i);
            p.inverse[i] = int32_t(pos);
            p.groups[gbase[e] + rel / 16].input_rows[rel % 16] = int32_t(i / kTopk);
            if (want_gw) p.gw[pos] = w4[step];
            if (!below) start[wv][e] += __popcll(m);
        }
    }
}

// Clears the count and fault words once the host has read them.
__global__ void meta_reset_kernel(uint32_t* meta) {
    if (threadIdx.x < kMetaWords) meta[threadIdx.x] = threadIdx.x == kQuantWhere ? 0xffffffffu : 0u;
}

// ---------------------------------------------------------------------------------------------
// Intermediate quantizer v1 on FP32 bit patterns (byte-exact contract):
// crates/mimo26-expert/kernels/b1/quant_v1.cuh:32-100, oracle/lattice/quant_v1.py:74-87.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kQuantFloorBits = 0x38d1b717u;  // FP32(1e-4)

// k = smallest integer with amax <= 448 * 2^k, amax already floored (so it is a normal number).
__device__ __forceinline__ int quant_scale_exponent(uint32_t amax_bits) {
    const uint32_t a = amax_bits < kQuantFloorBits ? kQuantFloorBits : amax_bits;
    return int(a >> 23) - 127 - ((a & 0x7fffffu) <= 0x600000u ? 8 : 7);
}

// E4M3FN codes of h0 * 2^-k and h1 * 2^-k in the two low bytes (h0 lowest), on top of `old`'s other
// half when HIGH. The scaling is exact (a power of two; where it would underflow the product is far
// below half the E4M3 quantum anyway) and gfx950's conversion is the OCP one: round to nearest even,
// subnormals kept, sign of zero kept. |h| <= amax <= 448 * 2^k, so nothing saturates.
template <bool HIGH>
__device__ __forceinline__ uint32_t quant_pair(float h0, float h1, int k, uint32_t old = 0) {
    return uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(__builtin_ldexpf(h0, -k), __builtin_ldexpf(h1, -k), int(old), HIGH));
}
__device__ __forceinline__ uint32_t quant_code(float h, int k) { return quant_pair<false>(h, 0.0f, k) & 0xffu; }

// The reconstruction code * 2^k leaves FP32 only for a normal code with field - 7 + k > 127, which
// needs k >= 120: blocks below that skip the check.
__device__ __forceinline__ bool quant_reconstructs(uint32_t code, int k) {
    const uint32_t field = (code & 0x7fu) >> 3;
    return field == 0 || int(field) - 7 + k <= 127;
}

// Stand-alone quantizer: one K32 block per half-wave (two blocks per wave per step).
__global__ void __launch_bounds__(256) quantize_kernel(const float* __restrict__ h, uint64_t blocks,
                                                       uint8_t* __restrict__ payload, uint8_t* __restrict__ scales,
                                                       uint32_t* __restrict__ faults) {
    const uint32_t sub = threadIdx.x & 31;
    const uint64_t first = (uint64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> 5;
    const uint64_t stride = (uint64_t(gridDim.x) * blockDim.x) >> 5;
    for (uint64_t b = first; b < blocks; b += stride) {
        const uint32_t bits = __float_as_uint(h[b * 32 + sub]);
        uint32_t amax = bits & 0x7fffffffu;
#pragma unroll
        for (int d = 16; d; d >>= 1) {
            const uint32_t o = __shfl_xor(amax, d);
            amax = o > amax ? o : amax;
        }
        if (amax >= 0x7f800000u) {
            if (sub == 0) faults[b] = 1;
            continue;
        }
        const int k = quant_scale_exponent(amax);
        const uint32_t code = quant_code(__uint_as_float(bits), k);
        uint32_t over = quant_reconstructs(code, k) ? 0u : 1u;
#pragma unroll
        for (int d = 16; d; d >>= 1) over |= __shfl_xor(over, d);
        if (sub == 0) faults[b] = over ? 2u : 0u;
        if (over) continue;
        payload[b * 32 + sub] = uint8_t(code);
        if (sub == 0) scales[b] = uint8_t(k + 127);
    }
}

// ---------------------------------------------------------------------------------------------
// Block-scaled grouped GEMM core, shared by FC1 and FC2.
//
// One wave owns four 16-row weight tiles (SrcA, FP4, streamed once, fully coalesced 1 KB per
// tile per k-step) and TT 16-row activation tiles (SrcB, FP8, row-major rows gathered by
// pointer). A k-step is K = 128; a block's next k-step lies kStepBytes further on.
// ---------------------------------------------------------------------------------------------
// Weight fragments of one k-step (four tiles) and the activation fragments of one k-step.
struct WeightStep { v4i a[4]; };
template <int TT>
struct ActStep {
    v4i lo[TT], hi[TT];
    uint32_t sb[TT];
};

__device__ __forceinline__ void load_weights(WeightStep& o, const uint8_t* __restrict__ wp, int ks) {
#pragma unroll
    for (int t = 0; t < 4; ++t) o.a[t] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(wp + size_t(ks) * kStepBytes + t * 1024));
}
template <int TT>
__device__ __forceinline__ void load_acts(ActStep<TT>& o, int ks, const uint8_t* const (&xrow)[TT],
                                          const uint8_t* const (&xsrow)[TT]) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        o.lo[tt] = *reinterpret_cast<const v4i*>(xrow[tt] + ks * 128);
        o.hi[tt] = *reinterpret_cast<const v4i*>(xrow[tt] + ks * 128 + 64);
        o.sb[tt] = *reinterpret_cast<const uint32_t*>(xsrow[tt] + ks * 4);
    }
}

template <int TT, int SEL>
__device__ __forceinline__ void mfma_step(v4f (&acc)[4][TT], const WeightStep& w, const ActStep<TT>& x,
                                          const uint32_t (&sw)[4], uint32_t shift, uint32_t& bad) {
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const uint32_t s = (x.sb[tt] >> shift) & 0xffu;
        bad |= (s - 105u) > 142u ? 1u : 0u;  // activation scales are legal only in [105, 247]
        const v8i b = {x.lo[tt].x, x.lo[tt].y, x.lo[tt].z, x.lo[tt].w, x.hi[tt].x, x.hi[tt].y, x.hi[tt].z, x.hi[tt].w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const v8i a = {w.a[t].x, w.a[t].y, w.a[t].z, w.a[t].w, 0, 0, 0, 0};
            acc[t][tt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[t][tt], 4 /*A: E2M1*/,
                                                                          0 /*B: E4M3*/, SEL, int(sw[t]), 0, int(s));
        }
    }
}

// wp / sp already include the lane offset (lane*16, lane*4). ksteps is a multiple of 4.
//
// This is the schedule of the HBM-bound sizes: the weight stream (4 KB per wave and k-step, each byte used
// once) is asked for three k-steps ahead of the MFMAs in a ring of four register sets; activation rows come
// from L2 and run one k-step ahead; the weight scale dwords of the next quad of k-steps are fetched a quad
// ahead. Past the end the last k-step is fetched again rather than branching.
template <int TT>
__device__ __forceinline__ void gemm_chunk(v4f (&acc)[4][TT], const uint8_t* __restrict__ wp,
                                           const uint8_t* __restrict__ sp, int ksteps,
                                           const uint8_t* const (&xrow)[TT], const uint8_t* const (&xsrow)[TT],
                                           uint32_t lane, uint32_t& bad) {
    const uint32_t shift = 8 * (lane >> 4);
    const int quads = ksteps / 4, last = ksteps - 1;
    auto upto = [&](int g) { return g < last ? g : last; };
    WeightStep w[4];
    ActStep<TT> x[2];
    uint32_t sw[4], swn[4];
    load_weights(w[0], wp, 0);
    load_weights(w[1], wp, 1);
    load_weights(w[2], wp, 2);
    load_acts<TT>(x[0], 0, xrow, xsrow);
#pragma unroll
    for (int t = 0; t < 4; ++t) sw[t] = *reinterpret_cast<const uint32_t*>(sp + t * 256);
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int q = 0; q < quads; ++q) {
        const int g = 4 * q, qn = q + 1 < quads ? q + 1 : q;
#pragma unroll
        for (int t = 0; t < 4; ++t) swn[t] = *reinterpret_cast<const uint32_t*>(sp + size_t(qn) * 1024 + t * 256);
        load_weights(w[3], wp, g + 3);
        load_acts<TT>(x[1], g + 1, xrow, xsrow);
        mfma_step<TT, 0>(acc, w[0], x[0], sw, shift, bad);
        load_weights(w[0], wp, upto(g + 4));
        load_acts<TT>(x[0], g + 2, xrow, xsrow);
        mfma_step<TT, 1>(acc, w[1], x[1], sw, shift, bad);
        load_weights(w[1], wp, upto(g + 5));
        load_acts<TT>(x[1], g + 3, xrow, xsrow);
        mfma_step<TT, 2>(acc, w[2], x[0], sw, shift, bad);
        load_weights(w[2], wp, upto(g + 6));
        load_acts<TT>(x[0], upto(g + 4), xrow, xsrow);
        mfma_step<TT, 3>(acc, w[3], x[1], sw, shift, bad);
#pragma unroll
        for (int t = 0; t < 4; ++t) sw[t] = swn[t];
    }
}

// e^t for t <= 0 in binary32 on the hardware 2^x: the product t * log2(e) is formed as a rounded head and
// its exact remainder (one FMA gives the head's rounding error, a second adds the part of log2(e) that
// binary32 cannot hold), the head goes through v_exp_f32 and the remainder is applied as a first-order
// factor. Within 2 ulp of the true value over the whole range, the accuracy class of the expf the
// reference's own kernels call (crates/mimo26-expert/kernels/b1/grouped.cu:89), in six instructions.
// Below -104 the true value is under half the smallest binary32 subnormal, i.e. zero once rounded: the
// clamp keeps the hardware function inside its range for gates as large as 2^127 (an earlier form, a
// Cody-Waite reduction by ln 2, lost its footing beyond about 2^24 and returned NaN there).
__device__ __forceinline__ float exp_nonpositive(float t) {
    constexpr float kLog2eHi = 1.44269502162933349609375f, kLog2eLo = 1.925963033500011e-08f, kLn2 = 0.693147182464599609375f;
    asm("v_max_f32 %0, 0xc2d00000, %0" : "+v"(t));  // max(t, -104) without the NaN canonicalisation fmaxf brings along
    const float head = t * kLog2eHi;
    float tail = __builtin_fmaf(t, kLog2eHi, -head);
    tail = __builtin_fmaf(t, kLog2eLo, tail);
    const float e = __builtin_amdgcn_exp2f(head);
    return __builtin_fmaf(e, tail * kLn2, e);
}

// SwiGLU in the reference's stable form (kernels/b1/grouped.cu:89-93): e = exp(-|g|);
// s = g >= 0 ? g/(1+e) : (g*e)/(1+e); h = s*u. The quotient is the numerator times the hardware reciprocal
// (1 ulp). The whole activation stays within a few binary32 ulp of the CPU rule, which rounds every step
// once; the epilogues are bound by vector-instruction issue, and the exactly rounded form costs three
// times the instructions.
__device__ __forceinline__ float silu_up(float g, float u) {
    const float e = exp_nonpositive(g >= 0.0f ? -g : g);
    const float d = 1.0f + e, num = g >= 0.0f ? g : g * e;
    return (num * __builtin_amdgcn_rcpf(d)) * u;
}

struct Fc1Args {
    const uint8_t* prepared;
    Prepared lay;
    PlanView plan;
    const uint8_t* x;         // E4M3 rows
    size_t x_pitch;
    const uint8_t* xs;        // UE8M0 K32 scale rows
    size_t xs_pitch;
    const uint8_t* zero_row;  // >= 4096 + 64 zero bytes, stands in for padded rows
    const uint8_t* unit_scales;  // >= 128 bytes of 127
    uint8_t* dq;              // [groups*16][I] E4M3 intermediate
    uint8_t* dqs;             // [groups*16][I/32] its scales
    float* tap_gate;          // optional FP32 taps [groups*16][I]
    float* tap_up;
    float* tap_h;
    // Tile schedule only: per-chunk activation scales in MFMA lane order, [chunk][K/512][8 tiles][64 lanes]
    // dwords whose byte b is the scale of k-block 4*(4q+b) + lane/16 of row lane%16.
    const uint8_t* xg;     // FC1 input scales, gathered by gather_scales_kernel
    const uint32_t* rowbad;  // [chunk][16]: bit 0 set where a row index of the chunk met an illegal input scale,
                             // bit 8+t set where tile t holds a token in that row
    const int32_t* xrows;    // [chunk][8 tiles][16]: the token each row of each tile reads, -1 for none
    uint8_t* dg;           // the intermediate's scales in the same order, written here for FC2
    unsigned long long* clock;  // tile schedule only, may be null: see TileClock in b1_tile.h
};

// FC1 epilogue of one wave for one activation tile: SwiGLU on the gate/up accumulators (tiles 0,1
// gate, 2,3 up), then quantizer v1 of each row's 32-column block straight from registers (amax across
// the four lanes that share a row, frexp-rule exponent, exact-grid RNE, reconstruction check), packed
// stores of payload and scale. `bad` must already be uniform over the four lanes of a row. dg_chunk,
// when given, also receives the scale byte in the order FC2's tile schedule reads (see Fc1Args::dg).
// SERIAL computes one activation at a time, for callers whose k-loop registers are still live.
template <bool SERIAL>
__device__ __forceinline__ void fc1_finish_tile(const Fc1Args& a, const Chunk ch, uint32_t cb, uint32_t lane, int tt,
                                                const v4f (&acc)[4], uint32_t bad, bool live, uint8_t* dg_chunk) {
    uint32_t* meta = a.plan.meta;
    const uint32_t r = lane & 15, g = lane >> 4, I = a.lay.inter;
    float h[2][4];
    uint32_t amax = 0;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            h[t2][i] = silu_up(acc[t2][i], acc[t2 + 2][i]);
            const uint32_t m = __float_as_uint(h[t2][i]) & 0x7fffffffu;
            amax = m > amax ? m : amax;
            if (SERIAL) __builtin_amdgcn_sched_barrier(0);  // bounds live registers
        }
    uint32_t o = __shfl_xor(amax, 16);
    amax = o > amax ? o : amax;
    o = __shfl_xor(amax, 32);
    amax = o > amax ? o : amax;
    const size_t grow = size_t(ch.first_group + tt) * 16 + r;
    const size_t col = size_t(cb) * 32 + 4 * g;
    if (live && a.tap_h) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
            *reinterpret_cast<v4f*>(a.tap_gate + grow * I + col + 16 * t2) = acc[t2];
            *reinterpret_cast<v4f*>(a.tap_up + grow * I + col + 16 * t2) = acc[t2 + 2];
            *reinterpret_cast<v4f*>(a.tap_h + grow * I + col + 16 * t2) = v4f{h[t2][0], h[t2][1], h[t2][2], h[t2][3]};
        }
    }
    const uint32_t block = uint32_t(grow * (I / 32) + cb);
    uint32_t fault = (amax >= 0x7f800000u || bad) ? 1u : 0u;
    const int k = quant_scale_exponent(amax);
    uint32_t word[2];
    uint32_t over = 0;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
        word[t2] = quant_pair<false>(h[t2][0], h[t2][1], k);
        word[t2] = quant_pair<true>(h[t2][2], h[t2][3], k, word[t2]);
    }
    if (__ballot(k >= 120)) {  // wave-uniform, and practically never taken
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
            for (int i = 0; i < 4; ++i) over |= quant_reconstructs((word[t2] >> (8 * i)) & 0xffu, k) ? 0u : 1u;
        over |= __shfl_xor(over, 16);
        over |= __shfl_xor(over, 32);
    }
    if (!fault && over) fault = 2;
    if (!live) return;
    if (fault) {
        if (g == 0) {
            atomicOr(&meta[kQuantFault], fault);
            atomicMin(&meta[kQuantWhere], block);
        }
        return;  // a faulting block publishes no bytes
    }
    *reinterpret_cast<uint32_t*>(a.dq + grow * I + col) = word[0];
    *reinterpret_cast<uint32_t*>(a.dq + grow * I + col + 16) = word[1];
    if (g == 0) {
        a.dqs[grow * (I / 32) + cb] = uint8_t(k + 127);
        // Block cb is k-block cb of FC2: k-step cb/4, lane group cb%4.
        if (dg_chunk) dg_chunk[((((cb >> 4) * 8 + tt) * 64 + (cb & 3) * 16 + r) << 2) + ((cb >> 2) & 3)] = uint8_t(k + 127);
    }
}

template <int TT>
__device__ __forceinline__ void fc1_finish(const Fc1Args& a, const Chunk ch, uint32_t cb, uint32_t lane,
                                           v4f (&acc)[4][TT], uint32_t bad, const bool (&live)[TT]) {
    bad |= __shfl_xor(bad, 16);
    bad |= __shfl_xor(bad, 32);
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const v4f tile[4] = {acc[0][tt], acc[1][tt], acc[2][tt], acc[3][tt]};
        fc1_finish_tile<true>(a, ch, cb, lane, tt, tile, bad, live[tt], nullptr);
    }
}

// One wave's share of FC1 for a chunk of TT groups: 32 intermediate columns x 16*TT rows.
template <int TT>
__device__ __forceinline__ void fc1_body(const Fc1Args& a, const Chunk ch, uint32_t cb, uint32_t lane) {
    const uint32_t r = lane & 15, g = lane >> 4;
    const Group* grp = a.plan.groups + ch.first_group;
    const int32_t expert = ch.expert;
    const uint8_t* xrow[TT];
    const uint8_t* xsrow[TT];
    bool live[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const int32_t row = tt < ch.groups ? grp[tt].input_rows[r] : -1;
        live[tt] = row >= 0;
        xrow[tt] = (live[tt] ? a.x + size_t(row) * a.x_pitch : a.zero_row) + g * 16;
        xsrow[tt] = live[tt] ? a.xs + size_t(row) * a.xs_pitch : a.unit_scales;
    }
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* wp = img + a.lay.w13() + block_payload(cb, 32) + lane * 16;
    const uint8_t* sp = img + a.lay.s13() + uint64_t(cb) * (8 * 1024) + lane * 4;
    v4f acc[4][TT];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
    uint32_t bad = 0;
    gemm_chunk<TT>(acc, wp, sp, 32, xrow, xsrow, lane, bad);
    fc1_finish<TT>(a, ch, cb, lane, acc, bad, live);
}

// A workgroup's chunk record and the eight meta words, by scalar loads: both are the same for every lane
// and were written by earlier launches, and the scalar path does not queue behind the operand stream of
// the workgroup next door, where a vector load of sixteen bytes waits some thousand cycles.
struct ItemHead { Chunk ch; uint32_t meta[kMetaWords]; };
__device__ __forceinline__ ItemHead load_item_head(const Chunk* record, const uint32_t* meta) {
    v4i r;
    v8i m;
    asm volatile("s_load_dwordx4 %0, %2, 0x0\n\ts_load_dwordx8 %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(r), "=&s"(m) : "s"(record), "s"(meta) : "memory");
    return ItemHead{Chunk{r.x, r.y, r.z, r.w},
                    {uint32_t(m[0]), uint32_t(m[1]), uint32_t(m[2]), uint32_t(m[3]), uint32_t(m[4]), uint32_t(m[5]), uint32_t(m[6]), uint32_t(m[7])}};
}

// Stages 2+3: gate/up grouped GEMM, SwiGLU and the v1 requantisation of the intermediate.
// grid (I/128, chunk capacity) x 256 threads, or (I/32, chunk capacity) x 64 for the smallest calls (the waves
// share nothing; the host picks the workgroup); each wave owns one 32-column K32 block of the
// intermediate for every row of its chunk, so a quantizer block never leaves the wave. A chunk
// holds at most NT groups; the body is compiled for 1, 2, 4 and 8 activation tiles.
template <int NT>
__global__ void __launch_bounds__(256) fc1_kernel(Fc1Args a) {
    uint32_t* meta = a.plan.meta;
    const uint32_t c = blockIdx.y;
    const ItemHead head = load_item_head(a.plan.chunks + c, meta);  // the chunk table covers the whole grid
    const Chunk ch = head.ch;
    if (head.meta[kPlanFault] || c >= head.meta[kChunkCount]) return;
    const uint32_t lane = threadIdx.x & 63, cb = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int32_t expert = ch.expert;
    if (expert < 0 || expert >= int32_t(kExperts) || ch.groups < 1 || ch.groups > NT) {
        if (lane == 0) atomicOr(&meta[kFc1Fault], 2u);
        return;
    }
    if (NT == 1 || ch.groups == 1) fc1_body<1>(a, ch, cb, lane);
    else if (NT == 2 || ch.groups == 2) fc1_body<2>(a, ch, cb, lane);
    else if (NT >= 4 && ch.groups <= 4) fc1_body<(NT >= 4 ? 4 : 1)>(a, ch, cb, lane);
    else fc1_body<(NT >= 8 ? 8 : 1)>(a, ch, cb, lane);
}

struct Fc2Args {
    const uint8_t* prepared;
    Prepared lay;
    PlanView plan;
    const uint8_t* dq;
    const uint8_t* dqs;
    const uint8_t* zero_row;
    const uint8_t* unit_scales;
    float* y;         // [routes][4096], original (token, slot) order, unweighted; BF16 bits when y_bf16
    uint32_t routes;
    const uint8_t* dg;  // tile schedule only: the intermediate's scales in MFMA lane order (see Fc1Args)
    const int32_t* yrows;  // tile schedule only, [chunk][8 tiles][16]: the route (row of y) of each row, -1 for none
    const uint32_t* rowbad;  // tile schedule only: as in Fc1Args (bit 8+t: tile t holds a token in that row)
    unsigned long long* clock;  // tile schedule only, may be null: see TileClock in b1_tile.h
    // The combine, done here by whichever wave completes a token's eighth row (plan.done != null):
    const float* w;     // [rows][8] router weights, the caller's array
    uint16_t* bf16;     // [rows][4096] BF16 bits out
    float* partial;     // [rows][4096] FP32 sums out, or null
    bool y_bf16;        // per-route rows are kept as BF16 bits (the opt-in mode of b1_serve.cu:98-143,400-405), not FP32
};

// ---------------------------------------------------------------------------------------------
// Stage 4b, the combine's arithmetic (kernels/b1/route_reduce.cu:61-74): per column v = 0; for slot 0..7:
// v = RN(v + RN(w * z)), multiply and add rounded separately; BF16 RNE; a weight outside [0, FLT_MAX], a
// nonfinite z or running sum, or a BF16 exponent of all ones fails the element group (NaN / zero out).
// Four columns of one token. Returns false when the group failed.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ bool combine4(const v4f (&z)[8], const float (&wt)[8], float (&v)[4], uint32_t (&code)[4]) {
    bool ok = true;
    v[0] = v[1] = v[2] = v[3] = 0.0f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        ok = ok && wt[s] >= 0.0f && wt[s] <= FLT_MAX;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            ok = ok && fabsf(z[s][k]) <= FLT_MAX;
            v[k] = __fadd_rn(v[k], __fmul_rn(wt[s], z[s][k]));
            ok = ok && fabsf(v[k]) <= FLT_MAX;
        }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const uint32_t b = __float_as_uint(v[k]);
        code[k] = (b + 0x7fffu + ((b >> 16) & 1u)) >> 16;
        ok = ok && (code[k] & 0x7f80u) != 0x7f80u;
    }
    if (!ok) {
        v[0] = v[1] = v[2] = v[3] = __uint_as_float(0x7fc00000u);
        code[0] = code[1] = code[2] = code[3] = 0;
    }
    return ok;
}
// BF16 bits -> binary32, and the reference's store rule for BF16 per-route rows (connected.cu:41-44).
__device__ __forceinline__ float bf16_value(uint32_t bits16) { return __uint_as_float(bits16 << 16); }
__device__ __forceinline__ uint32_t bf16_bits_rne(float v) {
    const uint32_t b = __float_as_uint(v);
    return (b + 0x7fffu + ((b >> 16) & 1u)) >> 16;
}

// Hand-over of per-route rows between waves of one launch that run on different XCDs, each with an L2 of
// its own: the rows are stored with device-scope write-through stores (sc1) and read back with device-scope
// loads (sc1), which no L2 answers from a stale line; between them stand the writer's wait for its stores'
// acknowledgements and a device-scope atomic on the token's count. The language-level fence that would
// order plain stores instead writes the whole L2 back (27 times the time of this form in a probe of 65,536
// rows of 2 KB, which also showed 1.8 million stale values per launch with plain stores and none with sc1).
// The stores are asm statements, and with them comes a duty the compiler otherwise carries: a store of more
// than eight bytes reads the upper half of its data a little after it issues, so the next two wait states
// must not write those registers. The compiler cannot see that an asm statement is such a store (it reused
// the registers at once, and the last two of four columns came out wrong now and then): the wait states are
// part of the statement.
__device__ __forceinline__ void store_route4(const Fc2Args& a, uint32_t route, uint32_t col, const v4f v) {
    if (a.y_bf16) {
        uint16_t* dst = reinterpret_cast<uint16_t*>(a.y) + size_t(route) * kHidden + col;
        const v2u packed = {bf16_bits_rne(v.x) | bf16_bits_rne(v.y) << 16, bf16_bits_rne(v.z) | bf16_bits_rne(v.w) << 16};
        asm volatile("global_store_dwordx2 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(packed) : "memory");
    } else {
        float* dst = a.y + size_t(route) * kHidden + col;
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
    }
}
__device__ __forceinline__ void wait_stores_acknowledged() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// One more row of `token` lies complete in y for output block ob (64 columns): returns true for the lane
// whose row was the token's eighth. Integer atomics decide only who sums, never the order of the sum.
__device__ __forceinline__ bool completes_token(const Fc2Args& a, uint32_t token, uint32_t ob) {
    return __hip_atomic_fetch_add(a.plan.done + size_t(token) * kDoneBlocks + ob, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == kTopk - 1;
}

// The wave sums, for output block ob, every token a lane names in `token` (-1: none): sixteen lanes and four
// columns each per token, four tokens at a time, the eight rows of a token fetched before the first is used,
// summed in slot order exactly as reduce_kernel does.
__device__ __forceinline__ void combine_completed(const Fc2Args& a, uint32_t ob, uint32_t lane, int32_t token) {
    uint64_t todo = __ballot(token >= 0);
    bool failed = false;
    while (todo) {
        uint32_t from = 64;  // the lane that names this lane group's token
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t first = todo ? uint32_t(__builtin_ctzll(todo)) : 64u;
            if (i == (lane >> 4)) from = first;
            todo &= todo - 1;
        }
        const int32_t mine = __shfl(token, int(from & 63u));
        if (from < 64) {
            const uint32_t col = ob * 64 + 4 * (lane & 15);
            const size_t first_row = size_t(mine) * kTopk;
            v4f z[8];
            float wt[8];
            if (a.y_bf16) {
                const uint16_t* src = reinterpret_cast<const uint16_t*>(a.y) + first_row * kHidden + col;
                v2u raw[8];
                asm volatile(
                    "global_load_dwordx2 %0, %8, off sc1\n\tglobal_load_dwordx2 %1, %9, off sc1\n\t"
                    "global_load_dwordx2 %2, %10, off sc1\n\tglobal_load_dwordx2 %3, %11, off sc1\n\t"
                    "global_load_dwordx2 %4, %12, off sc1\n\tglobal_load_dwordx2 %5, %13, off sc1\n\t"
                    "global_load_dwordx2 %6, %14, off sc1\n\tglobal_load_dwordx2 %7, %15, off sc1\n\t"
                    "s_waitcnt vmcnt(0)"
                    : "=&v"(raw[0]), "=&v"(raw[1]), "=&v"(raw[2]), "=&v"(raw[3]), "=&v"(raw[4]), "=&v"(raw[5]), "=&v"(raw[6]), "=&v"(raw[7])
                    : "v"(src), "v"(src + kHidden), "v"(src + 2 * kHidden), "v"(src + 3 * kHidden), "v"(src + 4 * kHidden),
                      "v"(src + 5 * kHidden), "v"(src + 6 * kHidden), "v"(src + 7 * kHidden)
                    : "memory");
#pragma unroll
                for (int s = 0; s < 8; ++s)
                    z[s] = v4f{bf16_value(raw[s].x & 0xffffu), bf16_value(raw[s].x >> 16), bf16_value(raw[s].y & 0xffffu), bf16_value(raw[s].y >> 16)};
            } else {
                const float* src = a.y + first_row * kHidden + col;
                asm volatile(
                    "global_load_dwordx4 %0, %8, off sc1\n\tglobal_load_dwordx4 %1, %9, off sc1\n\t"
                    "global_load_dwordx4 %2, %10, off sc1\n\tglobal_load_dwordx4 %3, %11, off sc1\n\t"
                    "global_load_dwordx4 %4, %12, off sc1\n\tglobal_load_dwordx4 %5, %13, off sc1\n\t"
                    "global_load_dwordx4 %6, %14, off sc1\n\tglobal_load_dwordx4 %7, %15, off sc1\n\t"
                    "s_waitcnt vmcnt(0)"
                    : "=&v"(z[0]), "=&v"(z[1]), "=&v"(z[2]), "=&v"(z[3]), "=&v"(z[4]), "=&v"(z[5]), "=&v"(z[6]), "=&v"(z[7])
                    : "v"(src), "v"(src + kHidden), "v"(src + 2 * kHidden), "v"(src + 3 * kHidden), "v"(src + 4 * kHidden),
                      "v"(src + 5 * kHidden), "v"(src + 6 * kHidden), "v"(src + 7 * kHidden)
                    : "memory");
            }
#pragma unroll
            for (int s = 0; s < 8; ++s) wt[s] = a.w[first_row + s];
            float v[4];
            uint32_t code[4];
            failed = !combine4(z, wt, v, code) || failed;
            if (a.partial) *reinterpret_cast<v4f*>(a.partial + size_t(mine) * kHidden + col) = v4f{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<uint2*>(a.bf16 + size_t(mine) * kHidden + col) = make_uint2(code[0] | (code[1] << 16), code[2] | (code[3] << 16));
        }
    }
    if (failed) atomicOr(&a.plan.meta[kReduceFault], 8u);  // Status::nonfinite
}

// FC2 epilogue of one wave: unweighted rows back to y[original route]; then, with the combine fused, one count
// per row and the sum of every token this wave's rows completed.
template <int TT>
__device__ __forceinline__ void fc2_finish(const Fc2Args& a, uint32_t ob, uint32_t lane, v4f (&acc)[4][TT],
                                           const int32_t (&route)[TT]) {
    const uint32_t g = lane >> 4;
    bool lost = false;
    // The stores below are asm statements (they carry a cache policy the language has no word for), and the
    // compiler's hazard tables do not look inside one: a matrix instruction's result lands up to eight passes
    // after issue, and a store issued sooner sends what the register held before (seen as the last two of four
    // columns of a tile's rows 12..15 wrong, now and then). These statements take every accumulator as an operand,
    // so they sit behind the last MFMA, and spend the wait states the compiler would have inserted.
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc[0][tt]), "+v"(acc[1][tt]), "+v"(acc[2][tt]), "+v"(acc[3][tt]));
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        if (route[tt] < 0) continue;
        if (uint32_t(route[tt]) >= a.routes) { lost = true; continue; }
#pragma unroll
        for (int t = 0; t < 4; ++t) store_route4(a, uint32_t(route[tt]), ob * 64 + 16 * t + 4 * g, acc[t][tt]);
    }
    if (lost) atomicOr(&a.plan.meta[kFc2Fault], 5u);
    if (!a.plan.done) return;
    wait_stores_acknowledged();
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {  // lanes 0..15 hold one row each of the tile (the other lane groups hold the same rows)
        const bool counts = g == 0 && route[tt] >= 0 && uint32_t(route[tt]) < a.routes;
        const int32_t token = counts && completes_token(a, uint32_t(route[tt]) >> 3, ob) ? route[tt] >> 3 : -1;
        combine_completed(a, ob, lane, token);
    }
}

// One wave's share of FC2 for a chunk of TT groups: 64 output columns x 16*TT rows.
template <int TT>
__device__ __forceinline__ void fc2_body(const Fc2Args& a, const Chunk ch, uint32_t ob, uint32_t lane) {
    const uint32_t r = lane & 15, g = lane >> 4, I = a.lay.inter;
    const Group* grp = a.plan.groups + ch.first_group;
    const int32_t expert = ch.expert;
    const uint8_t* xrow[TT];
    const uint8_t* xsrow[TT];
    int32_t route[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const bool live = tt < ch.groups && int32_t(r) < grp[tt].rows;
        const size_t grow = size_t(ch.first_group + tt) * 16 + r;
        route[tt] = live ? a.plan.original[grp[tt].route_base + r] : -1;
        xrow[tt] = (live ? a.dq + grow * I : a.zero_row) + g * 16;
        xsrow[tt] = live ? a.dqs + grow * (I / 32) : a.unit_scales;
    }
    const uint32_t ksteps = I / 128;
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* wp = img + a.lay.w2() + block_payload(ob, ksteps) + lane * 16;
    const uint8_t* sp = img + a.lay.s2() + uint64_t(ob) * (ksteps / 4) * 1024 + lane * 4;
    v4f acc[4][TT];
    uint32_t bad = 0;
    gemm_chunk<TT>(acc, wp, sp, int(ksteps), xrow, xsrow, lane, bad);
    fc2_finish<TT>(a, ob, lane, acc, route);
}

// Stage 4a: down grouped GEMM on the requantised intermediate; rows go back to y[original route].
// grid (16, chunk capacity) x 256 threads or (64, chunk capacity) x 64; each wave owns 64 output columns. (Two neighbouring blocks per wave
// in one stream halve the workgroups, and at 128 tokens the longer tail of the launch cost more than the longer
// streams saved, 172 against 154 us.)
template <int NT>
__global__ void __launch_bounds__(256) fc2_kernel(Fc2Args a) {
    uint32_t* meta = a.plan.meta;
    const uint32_t c = blockIdx.y;
    const ItemHead head = load_item_head(a.plan.chunks + c, meta);
    const Chunk ch = head.ch;
    if (head.meta[kPlanFault] || head.meta[kFc1Fault] || head.meta[kQuantFault] || c >= head.meta[kChunkCount]) return;
    const uint32_t lane = threadIdx.x & 63, ob = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int32_t expert = ch.expert;
    if (expert < 0 || expert >= int32_t(kExperts) || ch.groups < 1 || ch.groups > NT) {
        if (lane == 0) atomicOr(&meta[kFc2Fault], 2u);
        return;
    }
    if (NT == 1 || ch.groups == 1) fc2_body<1>(a, ch, ob, lane);
    else if (NT == 2 || ch.groups == 2) fc2_body<2>(a, ch, ob, lane);
    else if (NT >= 4 && ch.groups <= 4) fc2_body<(NT >= 4 ? 4 : 1)>(a, ch, ob, lane);
    else fc2_body<(NT >= 8 ? 8 : 1)>(a, ch, ob, lane);
}

// Stage 4b as a launch of its own (the conforming arm, and the stand-alone entry): the same arithmetic
// (combine4). Four columns per thread. Y16: the per-route rows are BF16 bits (crates/mimo26-spark/kernels/
// b1_serve.cu:98-143: same order, same roundings and fault rules on the widened values, no FP32 sum kept
// by the reference; here `partial` is still written when asked for).
template <bool Y16>
__global__ void __launch_bounds__(256) reduce_kernel(const void* __restrict__ y_rows, const float* __restrict__ w,
                                                     uint32_t rows, float* __restrict__ partial,
                                                     uint16_t* __restrict__ bf16, uint32_t* __restrict__ fault,
                                                     const uint32_t* __restrict__ gate) {
    if (gate && (gate[kPlanFault] || gate[kFc1Fault] || gate[kQuantFault] || gate[kFc2Fault])) return;
    const uint64_t n4 = uint64_t(rows) * (kHidden / 4);
    bool failed = false;
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += uint64_t(gridDim.x) * blockDim.x) {
        const uint64_t row = i / (kHidden / 4), col = (i % (kHidden / 4)) * 4;
        v4f z[8];
        if (Y16) {
            const uint16_t* y = static_cast<const uint16_t*>(y_rows);
#pragma unroll
            for (int s = 0; s < 8; ++s) {
                const v2u raw = __builtin_nontemporal_load(reinterpret_cast<const v2u*>(y + (row * 8 + s) * kHidden + col));
                z[s] = v4f{bf16_value(raw.x & 0xffffu), bf16_value(raw.x >> 16), bf16_value(raw.y & 0xffffu), bf16_value(raw.y >> 16)};
            }
        } else {
            const float* y = static_cast<const float*>(y_rows);
#pragma unroll
            for (int s = 0; s < 8; ++s)  // read once: streamed past the caches (6.3 against 4.9 TB/s at 8192 rows)
                z[s] = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(y + (row * 8 + s) * kHidden + col));
        }
        float wt[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) wt[s] = w[row * 8 + s];
        float v[4];
        uint32_t code[4];
        failed = !combine4(z, wt, v, code) || failed;
        if (partial) *reinterpret_cast<v4f*>(partial + row * kHidden + col) = v4f{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<uint2*>(bf16 + row * kHidden + col) = make_uint2(code[0] | (code[1] << 16), code[2] | (code[3] << 16));
    }
    if (failed) atomicOr(fault, 8u);  // Status::nonfinite
}

}  // namespace m26g
