// Prefill-size schedule of FC1 / FC2: four waves per workgroup, one per SIMD, each holding a
// 128-row x (16*TT)-row accumulator block (eight weight tiles x TT activation tiles, up to 256
// accumulator registers). Operands travel global -> LDS with the direct-to-LDS loads of gfx950
// (no staging registers, so the prefetch depth is paid in LDS, not in VGPRs), always two k-steps
// ahead of the MFMAs that consume them: every wave streams its own weight fragments into a private
// two-stage ring (a stage is free once its fragments sit in registers), and the chunk's activation
// tiles are staged once per workgroup in a three-stage ring shared by the four waves, so each
// activation byte leaves L2 once per 256 (FC1) or 512 (FC2) output columns.
//
// Reference counterparts: fc1_m64 / fc2_m64, the weight-reuse chunk kernels of
// crates/mimo26-spark/kernels/b1_fc1_m64.cuh:111-205,378-491 (cp.async multi-stage staging there).
//
// LDS, dynamic:  [4 waves][2 stages][8 tiles][64 lanes][16 B]   weight fragments (private per wave)
//                [3 stages][TT tiles][2 halves][64 lanes][16 B] activation fragments (shared)
//                [TT tiles][ksteps][16 rows][4 B]               activation scale bytes of the chunk
// All fragment cells sit in MFMA lane order, so one direct load fills a 1 KB cell row and one
// ds_read_b128 per lane reads it back without bank conflicts. The compiler does not order LDS reads
// against direct-to-LDS loads; the vmcnt waits below do, and rely on the issue order stated there.
// The k-loop has no branch: branches inside it let the compiler sink the MFMAs away from their
// operands.
#pragma once
#include <type_traits>
#include "b1_kernels.h"

namespace m26g {

constexpr int kTileThreads = 256, kTileWaves = 4, kWeightStages = 2, kActStages = 3;

__host__ __device__ constexpr uint32_t tile_lds_bytes(int tt, uint32_t k) {
    return uint32_t(kTileWaves) * kWeightStages * 8192 + uint32_t(kActStages) * tt * 2048 + (k / 128) * tt * 64;
}

typedef __attribute__((address_space(3))) void* lds_ptr;
typedef const __attribute__((address_space(1))) void* global_ptr;

// 64 lanes x 16 bytes from each lane's own global address into lds_row + lane*16.
__device__ __forceinline__ void load_row_to_lds(const uint8_t* lane_src, uint8_t* lds_row) {
    __builtin_amdgcn_global_load_lds((global_ptr)lane_src, (lds_ptr)lds_row, 16, 0, 0);
}
template <int N> __device__ __forceinline__ void wait_loads_but() {
    static_assert(N >= 0 && N < 64, "vmcnt immediate");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// LDS-only workgroup barrier: outstanding global prefetches stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// acc += A(FP4, scale byte SEL of sa) x B(FP8, scale byte 0 of sb), in place. Written as an
// instruction so destination and addend are the same registers: left to the compiler, a third of
// these MFMAs get a different destination and the loop drowns in accumulator copies. Half of a
// wave's accumulators are pinned to accumulation registers and half to vector registers, which
// leaves the other half of the accumulation file to the register allocator as spill space.
#define M26G_MFMA(sel_text, cons)                                                                              \
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 " sel_text " cbsz:4"                  \
                 : cons(acc) : "v"(a), "v"(b), "v"(sa), "v"(sb))
template <int SEL, bool AGPR>
__device__ __forceinline__ void mfma_acc(v4f& acc, const v4i& a, const v8i& b, uint32_t sa, uint32_t sb) {
    if constexpr (AGPR) {
        if constexpr (SEL == 0) M26G_MFMA("op_sel_hi:[0,0,0]", "+a");
        else if constexpr (SEL == 1) M26G_MFMA("op_sel:[1,0,0] op_sel_hi:[0,0,0]", "+a");
        else if constexpr (SEL == 2) M26G_MFMA("op_sel_hi:[1,0,0]", "+a");
        else M26G_MFMA("op_sel:[1,0,0] op_sel_hi:[1,0,0]", "+a");
    } else {
        if constexpr (SEL == 0) M26G_MFMA("op_sel_hi:[0,0,0]", "+v");
        else if constexpr (SEL == 1) M26G_MFMA("op_sel:[1,0,0] op_sel_hi:[0,0,0]", "+v");
        else if constexpr (SEL == 2) M26G_MFMA("op_sel_hi:[1,0,0]", "+v");
        else M26G_MFMA("op_sel:[1,0,0] op_sel_hi:[1,0,0]", "+v");
    }
}
#undef M26G_MFMA

// One workgroup's GEMM for a chunk. Wave `wv` accumulates eight weight tiles (two 4-tile blocks at
// wp0 / wp1, scales sp0 / sp1) against all TT activation tiles. The wave stages TT/4 activation
// tiles per k-step: `row[i]` / `srow[i]` are this lane's row of tile wv*(TT/4)+i (lane offset
// 16*(lane/16) included), so the lane that loads a fragment cell is the lane that will hold it.
template <int TT>
__device__ __forceinline__ void gemm_chunk_lds(v4f (&acc0)[4][TT], v4f (&acc1)[4][TT], const uint8_t* __restrict__ wp0,
                                               const uint8_t* __restrict__ wp1, const uint8_t* __restrict__ sp0,
                                               const uint8_t* __restrict__ sp1, int ksteps,
                                               const uint8_t* const (&row)[TT / 4], const uint8_t* const (&srow)[TT / 4],
                                               uint32_t wv, uint32_t lane, uint8_t* lds, uint32_t& bad) {
    static_assert(TT == 4 || TT == 8, "activation tiles per chunk");
    constexpr int kMine = TT / kTileWaves;  // activation tiles this wave stages
    const uint32_t r = lane & 15, g = lane >> 4;
    uint8_t* wring = lds + wv * (kWeightStages * 8192);                 // [stage][tile][lane][16]
    uint8_t* aring = lds + kTileWaves * kWeightStages * 8192;           // [stage][tt][half][lane][16]
    uint8_t* stab = aring + kActStages * TT * 2048;                     // [tt][ks][r][4]
    // The chunk's activation scale bytes, [tt][ks][row] dwords: one direct load moves the dwords of four
    // k-steps x 16 rows (lane = 16*j + row fetches k-step 4*i + j of its row).
#pragma unroll
    for (int m = 0; m < kMine; ++m)
        for (int i = 0; i < ksteps / 4; ++i)
            __builtin_amdgcn_global_load_lds((global_ptr)(srow[m] + (4 * i + g) * 4),
                                             (lds_ptr)(stab + ((wv * kMine + m) * ksteps + 4 * i) * 64), 4, 0, 0);
    // The direct loads of one k-step: item i < 2*kMine is an activation cell (tile i/2, half i%2),
    // the other eight are the weight rows. A k-step issues exactly kPerStep of them, spread over its
    // TT groups of MFMAs so the memory pipeline never sees a burst; the waits count on that total.
    constexpr int kPerStep = 2 * kMine + 8;
    auto stage_item = [&](int item, int ks, uint32_t astage, uint32_t wstage) {
        if (item < 2 * kMine) {
            const int m = item >> 1, half = item & 1;
            load_row_to_lds(row[m] + ks * 128 + half * 64, aring + ((astage * TT + wv * kMine + m) * 2 + half) * 1024);
        } else {
            const int t = item - 2 * kMine;
            load_row_to_lds((t < 4 ? wp0 : wp1) + size_t(ks) * 4096 + (t & 3) * 1024, wring + wstage * 8192 + t * 1024);
        }
    };
    auto stage_all = [&](int ks, uint32_t astage, uint32_t wstage) {
#pragma unroll
        for (int item = 0; item < kPerStep; ++item) stage_item(item, ks, astage, wstage);
    };
    v4i af[2][8];  // weight fragments of this k-step and the next
    auto read_weights = [&](v4i (&a)[8], uint32_t stage) {
#pragma unroll
        for (int t = 0; t < 8; ++t) a[t] = *reinterpret_cast<const v4i*>(wring + stage * 8192 + t * 1024 + lane * 16);
    };
    const int last = ksteps - 1;
    stage_all(0, 0, 0);
    stage_all(1 < last ? 1 : last, 1, 1);
    wait_loads_but<kPerStep>();  // step 0 has landed, step 1 may still fly
    read_weights(af[0], 0);
    lds_barrier();
    uint32_t wr = 0, ar = 0;  // weight stage holding step k+... see below; activation stage of step k
#pragma unroll 1
    for (int q = 0; q < ksteps / 4; ++q) {
        uint32_t sw[8];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            sw[t] = *reinterpret_cast<const uint32_t*>(sp0 + size_t(q) * 1024 + t * 256);
            sw[4 + t] = *reinterpret_cast<const uint32_t*>(sp1 + size_t(q) * 1024 + t * 256);
        }
        // One k-step with MFMA scale select b = ks % 4 (an immediate, hence the macro).
#define M26G_KSTEP(b)                                                                                          \
        {                                                                                                      \
            const int ks = 4 * q + (b);                                                                        \
            /* Weights of step k sit in registers, so their stage `wr` takes step k+2; step k+1 is in     */  \
            /* stage wr^1. Activations: step k reads stage ar, k+1 sits in ar+1, k+2 goes to ar+2.        */  \
            const uint32_t ar1 = ar == kActStages - 1 ? 0 : ar + 1, ar2 = ar1 == kActStages - 1 ? 0 : ar1 + 1; \
            /* Past the end the last step is staged again into stages nobody reads any more. */               \
            const int ahead = ks + 2 < last ? ks + 2 : last;                                                   \
            const uint8_t* fs = aring + ar * TT * 2048 + lane * 16;                                            \
            const uint8_t* ss = stab + (ks * 16 + r) * 4 + g;                                                  \
            v4i lo = *reinterpret_cast<const v4i*>(fs), hi = *reinterpret_cast<const v4i*>(fs + 1024);         \
            uint32_t s = ss[0];                                                                                \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) {                                                \
                _Pragma("unroll") for (int item = 0; item < kPerStep; ++item)                                  \
                    if (item * TT / kPerStep == tt) stage_item(item, ahead, ar2, wr);                          \
                const v8i bv = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};                               \
                const uint32_t sc = s;                                                                         \
                bad |= (sc - 105u) > 142u ? 1u : 0u; /* activation scales are legal only in [105, 247] */      \
                if (tt + 1 < TT) { /* the next fragment is on its way while this one multiplies */             \
                    lo = *reinterpret_cast<const v4i*>(fs + (tt + 1) * 2048);                                  \
                    hi = *reinterpret_cast<const v4i*>(fs + (tt + 1) * 2048 + 1024);                           \
                    s = ss[(tt + 1) * ksteps * 64];                                                            \
                } else {                                                                                       \
                    /* Everything but this step's own loads (step k+2) has landed: activations and */          \
                    /* weights of step k+1, issued one whole k-step ago.                            */          \
                    wait_loads_but<kPerStep>();                                                                \
                    read_weights(af[((b) + 1) & 1], wr ^ 1);                                                   \
                }                                                                                              \
                __builtin_amdgcn_sched_barrier(0);                                                             \
                _Pragma("unroll") for (int t = 0; t < 4; ++t)                                                  \
                    mfma_acc<(b), true>(acc0[t][tt], af[(b) & 1][t], bv, sw[t], sc);                            \
                _Pragma("unroll") for (int t = 0; t < 4; ++t)                                                  \
                    mfma_acc<(b), false>(acc1[t][tt], af[(b) & 1][4 + t], bv, sw[4 + t], sc);                    \
                __builtin_amdgcn_sched_barrier(0);                                                             \
            }                                                                                                  \
            wr ^= 1;                                                                                           \
            ar = ar1;                                                                                          \
            lds_barrier();                                                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
        }
        M26G_KSTEP(0)
        M26G_KSTEP(1)
        M26G_KSTEP(2)
        M26G_KSTEP(3)
#undef M26G_KSTEP
    }
    wait_loads_but<0>();  // the re-staged tail loads must land before the LDS is reused or the wave ends
    // The MFMAs above are opaque to the compiler's hazard tracking: let the last ones retire before
    // the epilogue reads the accumulators (8 passes of 4 cycles, plus margin).
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
}

// FC1 for one chunk of up to TT groups by one workgroup: 256 intermediate columns x 16*TT rows.
template <int TT>
__device__ __forceinline__ void fc1_tile_body(const Fc1Args& a, const Chunk ch, uint32_t wv, uint32_t lane, uint8_t* lds) {
    constexpr int kMine = TT / kTileWaves;
    const uint32_t r = lane & 15, g = lane >> 4, cb0 = blockIdx.x * 8 + wv * 2;
    const Group* grp = a.plan.groups + ch.first_group;
    const int32_t expert = grp[0].expert;
    const uint8_t* row[kMine];
    const uint8_t* srow[kMine];
#pragma unroll
    for (int m = 0; m < kMine; ++m) {
        const int lt = int(wv) * kMine + m;
        const int32_t mine = lt < ch.groups ? grp[lt].input_rows[r] : -1;
        row[m] = (mine >= 0 ? a.x + size_t(mine) * a.x_pitch : a.zero_row) + g * 16;
        srow[m] = mine >= 0 ? a.xs + size_t(mine) * a.xs_pitch : a.unit_scales;
    }
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* wp = img + a.lay.w13() + uint64_t(cb0) * (32 * 4096) + lane * 16;
    const uint8_t* sp = img + a.lay.s13() + uint64_t(cb0) * (8 * 1024) + lane * 4;
    v4f acc0[4][TT], acc1[4][TT];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc0[t][tt] = acc1[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
    uint32_t bad = 0;
    gemm_chunk_lds<TT>(acc0, acc1, wp, wp + 32 * 4096, sp, sp + 8 * 1024, int(kHidden / 128), row, srow, wv, lane, lds, bad);
    bad |= __shfl_xor(bad, 16);  // a row's four lanes see its four scale bytes of a k-step
    bad |= __shfl_xor(bad, 32);
    bool live[TT];  // looked up after the GEMM: nothing extra stays live across the k-loop
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) live[tt] = tt < ch.groups && grp[tt].input_rows[r] >= 0;
    fc1_finish<TT>(a, ch, cb0, lane, acc0, bad, live);
    fc1_finish<TT>(a, ch, cb0 + 1, lane, acc1, bad, live);
}

// FC2 for one chunk by one workgroup: 512 output columns x 16*TT rows.
template <int TT>
__device__ __forceinline__ void fc2_tile_body(const Fc2Args& a, const Chunk ch, uint32_t wv, uint32_t lane, uint8_t* lds) {
    constexpr int kMine = TT / kTileWaves;
    const uint32_t r = lane & 15, g = lane >> 4, ob0 = blockIdx.x * 8 + wv * 2, I = a.lay.inter;
    const Group* grp = a.plan.groups + ch.first_group;
    const int32_t expert = grp[0].expert;
    int32_t route[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
        const bool live = tt < ch.groups && int32_t(r) < grp[tt].rows;
        route[tt] = live ? a.plan.original[grp[tt].route_base + r] : -1;
    }
    const uint8_t* row[kMine];
    const uint8_t* srow[kMine];
#pragma unroll
    for (int m = 0; m < kMine; ++m) {
        const int lt = int(wv) * kMine + m;
        const bool mine = lt < ch.groups && int32_t(r) < grp[lt].rows;
        const size_t grow = size_t(ch.first_group + lt) * 16 + r;
        row[m] = (mine ? a.dq + grow * I : a.zero_row) + g * 16;
        srow[m] = mine ? a.dqs + grow * (I / 32) : a.unit_scales;
    }
    const uint32_t ksteps = I / 128;
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* wp = img + a.lay.w2() + uint64_t(ob0) * ksteps * 4096 + lane * 16;
    const uint8_t* sp = img + a.lay.s2() + uint64_t(ob0) * (ksteps / 4) * 1024 + lane * 4;
    v4f acc0[4][TT], acc1[4][TT];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc0[t][tt] = acc1[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
    uint32_t bad = 0;
    gemm_chunk_lds<TT>(acc0, acc1, wp, wp + size_t(ksteps) * 4096, sp, sp + size_t(ksteps / 4) * 1024, int(ksteps), row, srow,
                       wv, lane, lds, bad);
    fc2_finish<TT>(a, ob0, lane, acc0, route);
    fc2_finish<TT>(a, ob0 + 1, lane, acc1, route);
}

// grid (I/256, chunk capacity), 256 threads. Chunks of one or two groups run the register-only
// bodies (each wave is independent there, two column blocks in turn); larger chunks share
// activations through LDS.
__global__ void __launch_bounds__(kTileThreads) fc1_tile_kernel(Fc1Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t* meta = a.plan.meta;
    const uint32_t c = blockIdx.y;
    if (meta[kPlanFault] || c >= meta[kChunkCount]) return;
    const Chunk ch = a.plan.chunks[c];
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int32_t expert = a.plan.groups[ch.first_group].expert;
    if (expert < 0 || expert >= int32_t(kExperts) || ch.groups < 1 || ch.groups > 8) {
        if (lane == 0) atomicOr(&meta[kFc1Fault], 2u);
        return;
    }
    if (ch.groups <= 2) {
        for (uint32_t i = 0; i < 2; ++i) {
            const uint32_t cb = blockIdx.x * 8 + wv * 2 + i;
            if (ch.groups == 1) fc1_body<1>(a, ch, cb, lane);
            else fc1_body<2>(a, ch, cb, lane);
        }
    } else if (ch.groups <= 4) fc1_tile_body<4>(a, ch, wv, lane, lds);
    else fc1_tile_body<8>(a, ch, wv, lane, lds);
}

// grid (8, chunk capacity), 256 threads: 512 output columns per workgroup.
__global__ void __launch_bounds__(kTileThreads) fc2_tile_kernel(Fc2Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t* meta = a.plan.meta;
    const uint32_t c = blockIdx.y;
    if (meta[kPlanFault] || meta[kFc1Fault] || meta[kQuantFault] || c >= meta[kChunkCount]) return;
    const Chunk ch = a.plan.chunks[c];
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int32_t expert = a.plan.groups[ch.first_group].expert;
    if (expert < 0 || expert >= int32_t(kExperts) || ch.groups < 1 || ch.groups > 8) {
        if (lane == 0) atomicOr(&meta[kFc2Fault], 2u);
        return;
    }
    if (ch.groups <= 2) {
        for (uint32_t i = 0; i < 2; ++i) {
            const uint32_t ob = blockIdx.x * 8 + wv * 2 + i;
            if (ch.groups == 1) fc2_body<1>(a, ch, ob, lane);
            else fc2_body<2>(a, ch, ob, lane);
        }
    } else if (ch.groups <= 4) fc2_tile_body<4>(a, ch, wv, lane, lds);
    else fc2_tile_body<8>(a, ch, wv, lane, lds);
}

}  // namespace m26g
