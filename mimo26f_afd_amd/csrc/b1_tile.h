// Prefill-size schedule of FC1 / FC2: one workgroup of eight waves per compute unit.
//
// A wave accumulates one column block (four weight tiles: 32 intermediate columns of FC1, 64 output
// columns of FC2) against all TT activation tiles of its chunk: 4*TT accumulator tiles, 128
// accumulation registers at TT = 8, half of the register file of a wave at two waves per SIMD. The two
// waves of a SIMD belong to the same workgroup and run the same k-step; each fills the issue gaps of
// the other (a wave's own loads and LDS reads hold its in-order issue for longer than an MFMA's
// shadow).
//
// Operands travel global -> LDS with the direct-to-LDS loads of gfx950 (no staging registers, so the
// prefetch depth is paid in LDS, not in VGPRs), always three k-steps ahead of the MFMAs that consume
// them: every wave streams its own weight fragments into a private three-stage ring (a stage is free
// once its fragments sit in registers), and the chunk's activation tiles are staged once per
// workgroup in a four-stage ring shared by the eight waves. Scales never touch LDS: weight scales
// are stored in MFMA lane order by the one-time preparation, and activation scales are brought into
// the same order per chunk (gather_scales_kernel for the caller's rows, the FC1 epilogue for the
// intermediate), so one dword per lane carries the scale bytes of four k-steps and the MFMA picks
// its byte with op_sel.
//
// Reference counterparts: fc1_m64 / fc2_m64, the weight-reuse chunk kernels of
// crates/mimo26-spark/kernels/b1_fc1_m64.cuh:111-205,378-491 (cp.async multi-stage staging there).
//
// LDS, dynamic, 160 KB: [8 waves][3 stages][4 tiles][64 lanes][16 B]   weight fragments (private per wave)
//                       [4 stages][8 tiles][2 halves][64 lanes][16 B]  activation fragments (shared)
// All fragment cells sit in MFMA lane order, so one direct load fills a 1 KB cell row and one
// ds_read_b128 per lane reads it back without bank conflicts. The compiler does not order LDS reads
// against direct-to-LDS loads; the vmcnt waits below do, and rely on the issue order stated there.
// The k-loop has no branch: branches inside it let the compiler sink the MFMAs away from their
// operands.
#pragma once
#include <type_traits>
#include "b1_kernels.h"

namespace m26g {

// A tile workgroup's shape: W waves, operands D k-steps ahead. Weight fragments sit in a private ring of D
// stages per wave (a stage is free once its fragments are in registers), activation fragments in a ring
// of D + 1 stages shared by the waves (the extra stage decouples the slowest reader from the next load).
template <int W, int D>
struct TileShape {
    static constexpr int kWaves = W, kAhead = D, kThreads = 64 * W, kWeightStages = D, kActStages = D + 1;
    static constexpr uint32_t kLdsBytes = W * D * 4096 + (D + 1) * 8 * 2048;
};
// Eight waves, three k-steps ahead: the whole LDS of a compute unit for one workgroup. Against four waves two
// steps ahead, two workgroups per compute unit (80 KB each, what this schedule was first built as), a chunk's rows
// enter the compute unit once instead of twice (48 instead of 64 KB per k-step) and the saved LDS buys the third
// step of prefetch: measured on one box 4 % off FC1 and 6.4 % off FC2 at 8192 tokens, ahead from 256 rows up,
// level at 192, 2 % behind at 130.
using PrefillTile = TileShape<8, 3>;
static_assert(PrefillTile::kLdsBytes == 160 * 1024, "the 160 KB of a compute unit");
// Bytes of one chunk's gathered activation scales for a K-deep product: [K/512][8][64] dwords.
__host__ __device__ constexpr uint32_t gathered_scale_bytes(uint32_t k) { return (k / 512) * 2048; }

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
template <int N> __device__ __forceinline__ void wait_lds_but() {
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}
// One lane's 32 bytes of an activation fragment: the two 16-byte cells at `at` and `at` + 1024.
__device__ __forceinline__ void read_fragment(v4i& lo, v4i& hi, uint32_t at) {
    asm volatile("ds_read_b128 %0, %1" : "=v"(lo) : "v"(at) : "memory");
    asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(hi) : "v"(at) : "memory");
}
// LDS-only workgroup barrier: outstanding global prefetches stay in flight across it.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// acc += A(FP4, scale byte SEL of sa) x B(FP8, scale byte SEL of sb), in place, accumulator pinned
// to the accumulation registers. Written as an instruction so destination and addend are the same
// registers: left to the compiler, a third of these MFMAs get a different destination and the loop
// drowns in accumulator copies.
#define M26G_MFMA(sel_text)                                                                                    \
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 " sel_text " cbsz:4"                  \
                 : "+a"(acc) : "v"(a), "v"(b), "v"(sa), "v"(sb))
template <int SEL>
__device__ __forceinline__ void mfma_acc(v4f& acc, const v4i& a, const v8i& b, uint32_t sa, uint32_t sb) {
    if constexpr (SEL == 0) M26G_MFMA("op_sel_hi:[0,0,0]");
    else if constexpr (SEL == 1) M26G_MFMA("op_sel:[1,1,0] op_sel_hi:[0,0,0]");
    else if constexpr (SEL == 2) M26G_MFMA("op_sel_hi:[1,1,0]");
    else M26G_MFMA("op_sel:[1,1,0] op_sel_hi:[1,1,0]");
}
#undef M26G_MFMA

// Rewrites the activation scale rows of every chunk into MFMA lane order (layout at Fc1Args::xg) and
// checks them against the legal window [105, 247] (crates/mimo26-expert/kernels/b1/grouped.cu:28,37
// holds the reference's check). Padded rows get the unit scale 127. rowbad[chunk][r] collects, for
// row r of all tiles, the verdict in bit 0 (the granularity the FC1 epilogue reports faults at) and
// in bit 8+t whether tile t holds a token there, so the epilogue looks nothing else up. xrows / yrows
// list, per tile and row, the token FC1 reads and the route FC2 writes (-1 for none).
// grid (chunk capacity), 256 threads = 8 tiles x 16 rows x 2 halves of a scale row.
__global__ void __launch_bounds__(256) gather_scales_kernel(PlanView plan, const uint8_t* __restrict__ xs, size_t xs_pitch,
                                                            uint32_t* __restrict__ xg, uint32_t* __restrict__ rowbad,
                                                            int32_t* __restrict__ xrows, int32_t* __restrict__ yrows) {
    __shared__ uint32_t flags[16];
    const uint32_t c = blockIdx.x, tid = threadIdx.x;
    if (plan.meta[kPlanFault] || c >= plan.meta[kChunkCount]) return;
    const Chunk ch = plan.chunks[c];
    if (ch.groups < 1 || ch.groups > 8) return;  // FC1 reports the broken chunk
    const uint32_t tt = tid >> 5, r = (tid >> 1) & 15, half = tid & 1;
    if (tid < 16) flags[tid] = 0;
    __syncthreads();
    const int32_t row = int32_t(tt) < ch.groups ? plan.groups[ch.first_group + tt].input_rows[r] : -1;
    if (half == 0) {  // the chunk's rows flattened: FC1 and FC2 find them one load after their chunk index
        xrows[c * 128 + tt * 16 + r] = row;
        yrows[c * 128 + tt * 16 + r] = row >= 0 ? plan.original[plan.groups[ch.first_group + tt].route_base + r] : -1;
    }
    uint32_t bad = 0;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t q = 4 * half + j;
        uint32_t in[4] = {0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu, 0x7f7f7f7fu};
        if (row >= 0) {
            const uint8_t* src = xs + size_t(row) * xs_pitch + 16 * q;
#pragma unroll
            for (uint32_t b = 0; b < 4; ++b)
                in[b] = uint32_t(src[4 * b]) | uint32_t(src[4 * b + 1]) << 8 | uint32_t(src[4 * b + 2]) << 16 |
                        uint32_t(src[4 * b + 3]) << 24;
        }
#pragma unroll
        for (uint32_t g = 0; g < 4; ++g) {
            uint32_t out = 0;
#pragma unroll
            for (uint32_t b = 0; b < 4; ++b) {
                const uint32_t s = (in[b] >> (8 * g)) & 0xffu;
                bad |= (s - 105u) > 142u ? 1u : 0u;
                out |= s << (8 * b);
            }
            xg[((size_t(c) * (kHidden / 512) + q) * 8 + tt) * 64 + g * 16 + r] = out;
        }
    }
    const uint32_t verdict = bad | (row >= 0 ? 0x100u << tt : 0u);
    if (verdict) atomicOr(&flags[r], verdict);
    __syncthreads();
    if (tid < 16) rowbad[c * 16 + tid] = flags[tid];
}

// One wave's GEMM for a chunk: four weight tiles (fragments at wp, scale dwords at sp, both with the
// lane offset included) against TT activation tiles. The wave stages TT/4 of the activation tiles
// per k-step: `row[i]` is this lane's row of tile wv*(TT/4)+i (lane offset 16*(lane/16) included),
// so the lane that loads a fragment cell is the lane that will hold it. `sx` points at this lane's
// dword of tile 0, quad 0 of the chunk's gathered activation scales.
// ONE: the product is a single quad of k-steps deep (FC2 at one rank's share); otherwise the number of quads is
// even (8 for FC1, 4 for FC2 of a whole layer), which fixes the scale set the last quad runs on.
template <class S, int TT, bool ONE>
__device__ __forceinline__ void gemm_chunk_lds(v4f (&acc)[4][TT], const uint8_t* __restrict__ wp,
                                               const uint8_t* __restrict__ sp, const uint8_t* __restrict__ sx, int ksteps,
                                               const uint8_t* const (&row)[(2 * TT / S::kWaves + 1) / 2], uint32_t wv,
                                               uint32_t lane, uint8_t* lds) {
    static_assert(TT == 4 || TT == 8, "activation tiles per chunk");
    constexpr int kWeightStages = S::kWeightStages, kActStages = S::kActStages, kAhead = S::kAhead;
    // Activation cells (a tile's two 1 KB halves) this wave stages per k-step: cells wv*kCells .. +kCells-1 of the
    // chunk's 2*TT. With eight waves and four tiles that is half a tile.
    constexpr int kCells = 2 * TT / S::kWaves;
    static_assert(kCells >= 1, "every wave stages at least one cell");
    uint8_t* wring = lds + wv * (kWeightStages * 4096);          // [stage][tile][lane][16]
    uint8_t* aring = lds + S::kWaves * kWeightStages * 4096;      // [stage][tt][half][lane][16]
    // The direct loads of one k-step: item i < kCells is an activation cell, the other four are the weight
    // rows. A k-step issues exactly kPerStep of them, spread over its TT groups of MFMAs so the memory
    // pipeline never sees a burst; the waits count on that total.
    constexpr int kPerStep = kCells + 4;
    auto stage_item = [&](int item, int ks, uint32_t astage, uint32_t wstage) {
        if (item < kCells) {
            const uint32_t cell = wv * kCells + item, half = cell & 1u;  // row[] is indexed from the wave's first tile
            const int m = int(item + ((wv * kCells) & 1u)) >> 1;
            load_row_to_lds(row[m] + ks * 128 + half * 64, aring + (astage * TT * 2 + cell) * 1024);
        } else {
            const int t = item - kCells;
            load_row_to_lds(wp + size_t(ks) * kStepBytes + t * 1024, wring + wstage * 4096 + t * 1024);
        }
    };
    auto stage_all = [&](int ks, uint32_t astage, uint32_t wstage) {
#pragma unroll
        for (int item = 0; item < kPerStep; ++item) stage_item(item, ks, astage, wstage);
    };
    // LDS reads are issued by hand too, with their own lgkmcnt waits. Left to the compiler, every wait
    // on an LDS read is a wait for all of them (it knows of the direct loads above and drains
    // everything to be safe), the fragment fetched for the next MFMA group included. As with the
    // scales, nothing but the MFMAs, behind those waits, may read the registers so filled.
    const uint32_t wring_at = uint32_t(uintptr_t((lds_ptr)wring)) + lane * 16;
    const uint32_t aring_at = uint32_t(uintptr_t((lds_ptr)aring)) + lane * 16;
    v4i af[2][4];  // weight fragments of this k-step and the next
    auto read_weights = [&](v4i (&a)[4], uint32_t stage) {
        const uint32_t at = wring_at + stage * 4096;
#pragma unroll
        for (int t = 0; t < 4; ++t) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[t]) : "v"(at), "n"(t * 1024) : "memory");
    };
    // Scale dwords of a quad of k-steps (four weight tiles, TT activation tiles), in two register sets
    // that alternate. They are loaded by hand a whole quad ahead: a load the compiler knows of makes
    // it drain every outstanding load, the direct ones included, before the first use. The compiler
    // takes these registers for loaded the moment the instruction issues, so nothing but the MFMAs
    // may read them, and those sit behind the vmcnt waits of the quad before.
    uint32_t sw0[4], sa0[TT], sw1[4], sa1[TT];
    auto load_scales = [&](uint32_t (&w)[4], uint32_t (&x)[TT], int q) {
        const uint8_t* pw = sp + size_t(q) * 1024;
        const uint8_t* px = sx + size_t(q) * 2048;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            asm volatile("global_load_dword %0, %1, off offset:%2" : "=v"(w[t]) : "v"(pw), "n"(t * 256) : "memory");
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
            asm volatile("global_load_dword %0, %1, off offset:%2" : "=v"(x[tt]) : "v"(px), "n"(tt * 256) : "memory");
    };
    const int last = ksteps - 1, quads = ksteps / 4;
    load_scales(sw0, sa0, 0);
#pragma unroll
    for (int d = 0; d < kAhead; ++d) stage_all(d < last ? d : last, d, d);
    wait_loads_but<(kAhead - 1) * kPerStep>();  // step 0 and the first scales have landed, the later steps may still fly
    read_weights(af[0], 0);
    lds_barrier();
    v4i flo, fhi;  // the fragment a k-step starts with
    read_fragment(flo, fhi, aring_at);
    uint32_t wr = 0, ar = 0;  // weight stage of step k, which takes step k+kAhead; activation stage of step k
    int q = 0;
    // One k-step with MFMA scale select b = ks % 4 (an immediate, hence the macro).
    //
    // A wave issues in order, roughly one instruction every four or five cycles, while an MFMA holds the
    // matrix pipe for 32: whatever else the step needs (fragment reads, direct loads with their address
    // arithmetic) is slotted between the MFMAs of a group, a few instructions per gap, so the pipe never
    // waits for them. The workgroup barrier sits ahead of the last group's MFMAs, not behind them: what
    // it orders (every wave's loads of step k+1 landed, every wave's reads of step k done) is true by
    // then, and the first fragment of step k+1 and the next weights are fetched under those MFMAs.
#define M26G_KSTEP(b, SW, SA, STAGE, ALLOW, NEXT)                                                              \
    {                                                                                                          \
        const int ks = 4 * q + (b);                                                                            \
        /* Weights of step k sit in registers, so their stage `wr` takes step k+kAhead; step k+1 is   */      \
        /* in the stage after it. Activations: step k reads stage ar, k+1 sits in the next one, and   */      \
        /* step k+kAhead goes to the stage before ar, which step k-1 has finished with.               */      \
        const uint32_t ar1 = ar == kActStages - 1 ? 0 : ar + 1, ar2 = ar == 0 ? kActStages - 1 : ar - 1;       \
        const uint32_t wr1 = wr == kWeightStages - 1 ? 0 : wr + 1;                                             \
        const int ahead = ks + kAhead; /* the step staged under this one (STAGE: it exists) */               \
        const uint32_t fs = aring_at + ar * TT * 2048;                                                         \
        v4i lo = flo, hi = fhi; /* fragment 0, fetched at the end of the step before */                       \
        _Pragma("unroll") for (int tt = 0; tt < TT; ++tt) {                                                    \
            v4i nlo = lo, nhi = hi;                                                                            \
            if (tt == TT - 1) {                                                                                \
                if (STAGE) {                                                                                   \
                    _Pragma("unroll") for (int item = 0; item < kPerStep; ++item)                              \
                        if (item * TT / kPerStep == tt) stage_item(item, ahead, ar2, wr);                      \
                }                                                                                              \
                __builtin_amdgcn_sched_barrier(0);                                                             \
                if (NEXT) {                                                                                    \
                    /* Everything but the ALLOW youngest loads has landed: activations and weights of   */      \
                    /* step k+1 are older than those.                                                   */      \
                    wait_loads_but<(ALLOW)>();                                                                 \
                    lds_barrier(); /* with the wait for this group's fragment */                               \
                    read_fragment(flo, fhi, aring_at + ar1 * TT * 2048);                                       \
                    read_weights(af[((b) + 1) & 1], wr1);                                                      \
                } else {                                                                                       \
                    wait_lds_but<0>(); /* the chunk's last step: nothing to fetch, nobody to wait for */      \
                }                                                                                              \
            } else {                                                                                           \
                wait_lds_but<0>();                                                                             \
            }                                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            const v8i bv = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};                                   \
            mfma_acc<(b)>(acc[0][tt], af[(b) & 1][0], bv, SW[0], SA[tt]);                                       \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            if (tt + 1 < TT) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(nlo) : "v"(fs), "n"((tt + 1 < TT ? tt + 1 : 0) * 2048) : "memory"); \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            mfma_acc<(b)>(acc[1][tt], af[(b) & 1][1], bv, SW[1], SA[tt]);                                       \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            if (tt + 1 < TT) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(nhi) : "v"(fs), "n"((tt + 1 < TT ? tt + 1 : 0) * 2048 + 1024) : "memory"); \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            mfma_acc<(b)>(acc[2][tt], af[(b) & 1][2], bv, SW[2], SA[tt]);                                       \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            if (STAGE && tt + 1 < TT) {                                                                        \
                _Pragma("unroll") for (int item = 0; item < kPerStep; ++item)                                  \
                    if (item * TT / kPerStep == tt) stage_item(item, ahead, ar2, wr);                          \
            }                                                                                                  \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            mfma_acc<(b)>(acc[3][tt], af[(b) & 1][3], bv, SW[3], SA[tt]);                                       \
            __builtin_amdgcn_sched_barrier(0);                                                                 \
            lo = nlo;                                                                                          \
            hi = nhi;                                                                                          \
        }                                                                                                      \
        wr = wr1;                                                                                              \
        ar = ar1;                                                                                              \
    }
    // A quad: fetch the next quad's scales into the other set, then four k-steps on this set. A step leaves
    // the loads of the kAhead-1 steps behind the next one in flight; the next quad's scales were asked for at
    // the head of step 0, behind the loads of the step before, so with more than one step in flight they lie
    // inside that window and step 0 leaves them in flight too.
#define M26G_ALLOW(b) ((kAhead - 1) * kPerStep + ((b) == 0 && kAhead > 2 ? 4 + TT : 0))
#define M26G_QUAD(SW, SA, NW, NA)                                                                              \
    {                                                                                                          \
        load_scales(NW, NA, q + 1);                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                     \
        M26G_KSTEP(0, SW, SA, 1, M26G_ALLOW(0), 1)                                                             \
        M26G_KSTEP(1, SW, SA, 1, M26G_ALLOW(1), 1)                                                             \
        M26G_KSTEP(2, SW, SA, 1, M26G_ALLOW(2), 1)                                                             \
        M26G_KSTEP(3, SW, SA, 1, M26G_ALLOW(3), 1)                                                             \
        /* The compiler may put anything behind a quad, a copy of an accumulator included (it hands them to */ \
        /* the code after the loop in other registers when it likes), and it does not know that the last  */ \
        /* MFMA's result is eight passes away: sixteen wait states cover that with room to spare.         */ \
        asm volatile("s_nop 15" ::: "memory");                                                                \
        ++q;                                                                                                   \
    }
    // The chunk's last quad stages only the steps that exist (step j stages step j + kAhead of the quad),
    // leaves in flight only what is younger than the step after it, and its last step fetches nothing
    // and meets nobody: no load is issued for a step past the end.
#define M26G_TAIL_STAGE(j) ((j) + kAhead <= 3)
#define M26G_TAIL_ALLOW(j) (((kAhead - 1) < (2 - (j)) ? (kAhead - 1) : (2 - (j))) * kPerStep)
#define M26G_TAIL(SW, SA)                                                                                      \
    {                                                                                                          \
        M26G_KSTEP(0, SW, SA, M26G_TAIL_STAGE(0), M26G_TAIL_ALLOW(0), 1)                                       \
        M26G_KSTEP(1, SW, SA, M26G_TAIL_STAGE(1), M26G_TAIL_ALLOW(1), 1)                                       \
        M26G_KSTEP(2, SW, SA, M26G_TAIL_STAGE(2), M26G_TAIL_ALLOW(2), 1)                                       \
        M26G_KSTEP(3, SW, SA, 0, 0, 0)                                                                         \
        asm volatile("s_nop 15" ::: "memory");                                                                \
        ++q;                                                                                                   \
    }
    if constexpr (ONE) {
        M26G_TAIL(sw0, sa0)
    } else {
        const int whole = quads - 1;  // quads that have a quad behind them: an odd number
#pragma unroll 1
        while (q + 1 < whole) {
            M26G_QUAD(sw0, sa0, sw1, sa1)
            M26G_QUAD(sw1, sa1, sw0, sa0)
        }
        M26G_QUAD(sw0, sa0, sw1, sa1)
        M26G_TAIL(sw1, sa1)
    }
#undef M26G_TAIL
#undef M26G_TAIL_ALLOW
#undef M26G_TAIL_STAGE
#undef M26G_ALLOW
#undef M26G_QUAD
#undef M26G_KSTEP
    wait_loads_but<0>();  // nothing is left in flight by now; the LDS is about to be reused
    wait_lds_but<0>();
    // The last fetches of scales, fragment and weights feed no MFMA. To the compiler such a register is
    // free the moment the load has issued, and whatever it puts there next is overwritten when the
    // data lands. Naming them here keeps them reserved until the waits above have passed.
#pragma unroll
    for (int t = 0; t < 4; ++t) asm volatile("" ::"v"(sw0[t]), "v"(sw1[t]), "v"(af[0][t]), "v"(af[1][t]));
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) asm volatile("" ::"v"(sa0[tt]), "v"(sa1[tt]));
    asm volatile("" ::"v"(flo), "v"(fhi));
    // The MFMAs above are opaque to the compiler's hazard tracking: let the last ones retire before
    // the epilogue reads the accumulators (8 passes of 4 cycles, plus margin).
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
}

// The epilogues index everything by the lane number. Handing them a copy the compiler cannot see
// through keeps their address arithmetic behind the k-loop, where it would otherwise be hoisted to
// and held in registers the loop needs.
__device__ __forceinline__ uint32_t after_loop(uint32_t lane) {
    asm volatile("" : "+v"(lane));
    return lane;
}

// FC1 for chunk c by one workgroup: 128 intermediate columns x 16*TT rows; the wave owns block cb.
// `token[m]` is the row table's entry for this lane's row of tile wv*(TT/4)+m, fetched by the caller beside
// the chunk record so that the rows' addresses are one memory latency behind the workgroup's start, not two.
// Activation tiles a wave of shape S stages rows of, per k-step, in a chunk of TT tiles, and the first of them.
template <class S, int TT> constexpr int staged_tiles() { return (2 * TT / S::kWaves + 1) / 2; }
template <class S, int TT> __device__ __forceinline__ uint32_t first_staged_tile(uint32_t wv) { return (wv * (2 * TT / S::kWaves)) >> 1; }

template <class S, int TT>
__device__ __forceinline__ void fc1_tile_body(const Fc1Args& a, const Chunk ch, uint32_t c, uint32_t cb, uint32_t wv,
                                              uint32_t lane, uint8_t* lds, const int32_t (&token)[staged_tiles<S, TT>()]) {
    constexpr int kMine = staged_tiles<S, TT>();
    const uint32_t g = lane >> 4;
    const int32_t expert = ch.expert;
    const uint8_t* row[kMine];
#pragma unroll
    for (int m = 0; m < kMine; ++m) row[m] = (token[m] >= 0 ? a.x + size_t(token[m]) * a.x_pitch : a.zero_row) + g * 16;
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* wp = img + a.lay.w13() + block_payload(cb, 32) + lane * 16;
    const uint8_t* sp = img + a.lay.s13() + uint64_t(cb) * (8 * 1024) + lane * 4;
    const uint8_t* sx = a.xg + size_t(c) * gathered_scale_bytes(kHidden) + lane * 4;
    v4f acc[4][TT];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
    gemm_chunk_lds<S, TT, false>(acc, wp, sp, sx, int(kHidden / 128), row, wv, lane, lds);
    const uint32_t lane2 = after_loop(lane), r2 = lane2 & 15;
    const uint32_t verdict = a.rowbad[c * 16 + r2], bad = verdict & 1u;
    // The accumulators leave the accumulation registers through LDS, sixteen tiles at a time: whole-tile
    // writes keep them out of the register allocator's hands until the very end (element reads straight
    // from the accumulation file make it split their live ranges across the k-loop), and the epilogue
    // becomes one rolled loop over the activation tiles. Unrolled it is 70 KB of code, and workgroups
    // in different phases then evict each other's instructions from the cache the compute units share.
    // Every wave has drained its own direct loads; after the barrier nobody's are left, and each wave
    // takes 16 KB of its own from the front of the rings.
    asm volatile("s_barrier" ::: "memory");
    uint8_t* bounce = lds + wv * 16384 + lane2 * 16;
    const uint32_t bounce_at = uint32_t(uintptr_t((lds_ptr)bounce));
    auto park = [&](int half) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(bounce_at), "a"(acc[t][(TT == 8 ? half * 4 : 0) + j]),
                             "n"((j * 4 + t) * 1024)
                             : "memory");
    };
    uint8_t* dg_chunk = a.dg + size_t(c) * gathered_scale_bytes(a.lay.inter);
    park(0);
#pragma unroll 1
    for (int tt = 0; tt < TT; ++tt) {
        if (TT == 8 && tt == 4) park(1);  // in-order LDS: the first half has been read by now
        v4f tile[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) tile[t] = *reinterpret_cast<const v4f*>(bounce + ((tt & 3) * 4 + t) * 1024);
        const bool live = (verdict >> (8 + tt)) & 1u;
        fc1_finish_tile<false>(a, ch, cb, lane2, tt, tile, bad, live, dg_chunk);
    }
}

// FC2 for chunk c by one workgroup: 256 output columns x 16*TT rows; the wave owns block ob.
// `verdict` is rowbad[c][lane % 16] (bit 8+t: tile t holds a token in this row), fetched by the caller beside
// the chunk record.
template <class S, int TT, bool ONE>
__device__ __forceinline__ void fc2_tile_body(const Fc2Args& a, const Chunk ch, uint32_t c, uint32_t ob, uint32_t wv,
                                              uint32_t lane, uint8_t* lds, const uint32_t verdict) {
    constexpr int kMine = staged_tiles<S, TT>();
    const uint32_t r = lane & 15, g = lane >> 4, I = a.lay.inter;
    const int32_t expert = ch.expert;
    const uint8_t* row[kMine];
#pragma unroll
    for (int m = 0; m < kMine; ++m) {
        const int lt = int(first_staged_tile<S, TT>(wv)) + m;
        const bool mine = (verdict >> (8 + lt)) & 1u;
        const size_t grow = size_t(ch.first_group + lt) * 16 + r;
        row[m] = (mine ? a.dq + grow * I : a.zero_row) + g * 16;
    }
    const uint32_t ksteps = I / 128;
    const uint8_t* img = a.prepared + uint64_t(expert) * a.lay.bytes();
    const uint8_t* wp = img + a.lay.w2() + block_payload(ob, ksteps) + lane * 16;
    const uint8_t* sp = img + a.lay.s2() + uint64_t(ob) * (ksteps / 4) * 1024 + lane * 4;
    const uint8_t* sx = a.dg + size_t(c) * gathered_scale_bytes(I) + lane * 4;
    v4f acc[4][TT];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) acc[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
    gemm_chunk_lds<S, TT, ONE>(acc, wp, sp, sx, int(ksteps), row, wv, lane, lds);
    const uint32_t lane2 = after_loop(lane);
    // A lane holds four consecutive output columns of one token per tile, so a store straight from the
    // accumulators touches sixteen token rows with 64 bytes each. One trip through the wave's own, now
    // idle, weight ring regroups a tile row into 256 contiguous bytes per token (sixteen lanes) and
    // four tokens per store: a tenth off the kernel at 8192 tokens. Cells are 272 bytes apart so the
    // regrouped reads (same token, sixteen cells) fall on different banks.
    uint8_t* ring = lds + wv * (S::kWeightStages * 4096);
    const uint32_t cell = lane2 & 15, token4 = lane2 >> 4;  // regrouped: sixteen 16-byte cells of one token, four tokens
    const uint32_t put_at = uint32_t(uintptr_t((lds_ptr)ring)) + (lane2 >> 4) * 272 + (lane2 & 15) * 16;
    bool lost = false;
    int32_t route[TT][4];  // all looked up at once: one latency, not thirty-two
#pragma unroll
    for (int tt = 0; tt < TT; ++tt)
#pragma unroll
        for (int j = 0; j < 4; ++j) route[tt][j] = a.yrows[c * 128 + tt * 16 + 4 * j + token4];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(put_at), "a"(acc[t][tt]), "n"(t * 4 * 272) : "memory");
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t token = 4 * j + token4;
            const v4f v = *reinterpret_cast<const v4f*>(ring + cell * 272 + token * 16);
            const int32_t rt = route[tt][j];
            if (rt < 0) continue;
            if (uint32_t(rt) >= a.routes) { lost = true; continue; }
            store_route4(a, uint32_t(rt), ob * 64 + cell * 4, v);
        }
    }
    if (lost) atomicOr(&a.plan.meta[kFc2Fault], 5u);
    if (!a.plan.done) return;
    // The combine, fused: one count per row this wave has just written, then the sum of every token whose eighth
    // row that was (b1_kernels.h, combine_completed). A lane takes rows lane and lane + 64 of the chunk.
    wait_stores_acknowledged();
#pragma unroll 1
    for (int half = 0; half < TT / 4; ++half) {
        const int32_t rt = a.yrows[c * 128 + half * 64 + lane2];
        const bool counts = rt >= 0 && uint32_t(rt) < a.routes;
        const int32_t token = counts && completes_token(a, uint32_t(rt) >> 3, ob) ? rt >> 3 : -1;
        combine_completed(a, ob, lane2, token);
    }
}

// The clock a tile launch ran at. The shader clock of these parts is not a constant of the launch: under the
// load of the tile kernels the power management takes it well below what the same part holds on a loop of
// nothing but MFMAs, so a cycle count says little without it. The workgroup of the middle chunk's first column
// set (every compute unit busy around it, once the call is large enough to fill them) reads the shader-clock
// counter and the fixed 100 MHz counter at both ends of its item and leaves the two differences in clock[0..1];
// their ratio x 0.1 is the clock in GHz.
struct TileClock {
    unsigned long long shader, fixed;
    __device__ __forceinline__ void start() { shader = __builtin_amdgcn_s_memtime(), fixed = __builtin_amdgcn_s_memrealtime(); }
    __device__ __forceinline__ void stop(unsigned long long* out, bool mine) const {
        if (out && mine && threadIdx.x == 0) {
            out[0] = __builtin_amdgcn_s_memtime() - shader;
            out[1] = __builtin_amdgcn_s_memrealtime() - fixed;
        }
    }
};

// Work item of a tile workgroup. Workgroups are handed to the eight XCDs in turn, each with an L2 of
// its own: the `columns` workgroups of one chunk all take ids of one residue mod 8, so a chunk's
// activation rows enter one L2 only. FC2 hands an XCD runs of two neighbouring chunks: chunks are in
// expert order, two neighbours mostly share their expert, and their workgroups of one column, dispatched
// back to back, stream the same weights through that L2. Measured with eight-wave workgroups at 8192
// tokens: runs of two against single chunks take 1.4 % off FC2 and add 1.8 % to FC1 (whose workgroup
// streams four times the weight bytes per chunk and shares less of its time with its neighbour); runs of
// four lose 2 % and 5 %. The grid is columns * (chunk capacity rounded up to 8 runs).
struct TileItem { uint32_t chunk, column; };
constexpr uint32_t kFc1Run = 1, kFc2Run = 2, kTileRunMax = 2;  // neighbouring chunks per XCD
template <uint32_t RUN>
__device__ __forceinline__ TileItem tile_item(uint32_t columns) {
    const uint32_t id = blockIdx.x, xcd = id & 7, slot = id >> 3;
    const uint32_t per = columns * RUN, run = slot / per, within = slot % per;
    return TileItem{(run * 8 + xcd) * RUN + within % RUN, within / RUN};
}
__host__ inline uint32_t tile_grid(uint32_t columns, uint32_t chunk_cap, uint32_t run) {
    return columns * ((chunk_cap + 8 * run - 1) / (8 * run) * (8 * run));
}

// One workgroup of S::kWaves waves per (chunk, 32 * kWaves intermediate columns). Chunks of one or two groups
// run the register-only bodies (each wave is independent there); larger chunks share activations
// through LDS.
template <class S>
__global__ void __launch_bounds__(S::kThreads, 8 / S::kWaves) fc1_tile_kernel(Fc1Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t* meta = a.plan.meta;
    TileClock clock;
    clock.start();
    const TileItem it = tile_item<kFc1Run>(a.lay.inter / (32 * S::kWaves));
    const uint32_t c = it.chunk;
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6, cb = it.column * S::kWaves + wv;
    // The row table's entries this lane may need, as four tiles and as eight, asked for beside the record:
    // the table covers the whole grid.
    const int32_t* xr = a.xrows + size_t(c) * 128 + (lane & 15);
    int32_t token4[staged_tiles<S, 4>()], token8[staged_tiles<S, 8>()];
#pragma unroll
    for (int m = 0; m < staged_tiles<S, 4>(); ++m) token4[m] = xr[(first_staged_tile<S, 4>(wv) + m) * 16];
#pragma unroll
    for (int m = 0; m < staged_tiles<S, 8>(); ++m) token8[m] = xr[(first_staged_tile<S, 8>(wv) + m) * 16];
    const ItemHead head = load_item_head(a.plan.chunks + c, meta);  // the chunk table covers the whole grid too
    const Chunk ch = head.ch;
    if (head.meta[kPlanFault] || c >= head.meta[kChunkCount]) return;
    const int32_t expert = ch.expert;
    if (expert < 0 || expert >= int32_t(kExperts) || ch.groups < 1 || ch.groups > 8) {
        if (lane == 0) atomicOr(&meta[kFc1Fault], 2u);
        return;
    }
    if (ch.groups == 1) fc1_body<1>(a, ch, cb, lane);
    else if (ch.groups == 2) fc1_body<2>(a, ch, cb, lane);
    else if (ch.groups <= 4) fc1_tile_body<S, 4>(a, ch, c, cb, wv, lane, lds, token4);
    else fc1_tile_body<S, 8>(a, ch, c, cb, wv, lane, lds, token8);
    clock.stop(a.clock, c == head.meta[kChunkCount] / 2 && it.column == 0);
}

// One workgroup per (chunk, 64 * kWaves output columns). ONE: the layer holds one rank's share (I = 512, a single
// quad of k-steps); otherwise I = 2048.
template <class S, bool ONE>
__global__ void __launch_bounds__(S::kThreads, 8 / S::kWaves) fc2_tile_kernel(Fc2Args a) {
    extern __shared__ __align__(16) uint8_t lds[];
    uint32_t* meta = a.plan.meta;
    TileClock clock;
    clock.start();
    const TileItem it = tile_item<kFc2Run>(kHidden / (64 * S::kWaves));
    const uint32_t c = it.chunk;
    const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6, ob = it.column * S::kWaves + wv;
    const uint32_t verdict = a.rowbad[c * 16 + (lane & 15)];  // beside the record: the table covers the whole grid
    const ItemHead head = load_item_head(a.plan.chunks + c, meta);
    const Chunk ch = head.ch;
    if (head.meta[kPlanFault] || head.meta[kFc1Fault] || head.meta[kQuantFault] || c >= head.meta[kChunkCount]) return;
    const int32_t expert = ch.expert;
    if (expert < 0 || expert >= int32_t(kExperts) || ch.groups < 1 || ch.groups > 8) {
        if (lane == 0) atomicOr(&meta[kFc2Fault], 2u);
        return;
    }
    if (ch.groups == 1) fc2_body<1>(a, ch, ob, lane);
    else if (ch.groups == 2) fc2_body<2>(a, ch, ob, lane);
    else if (ch.groups <= 4) fc2_tile_body<S, 4, ONE>(a, ch, c, ob, wv, lane, lds, verdict);
    else fc2_tile_body<S, 8, ONE>(a, ch, c, ob, wv, lane, lds, verdict);
    clock.stop(a.clock ? a.clock + 2 : nullptr, c == head.meta[kChunkCount] / 2 && it.column == 0);
}

}  // namespace m26g
