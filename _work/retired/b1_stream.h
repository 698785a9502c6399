// FC2 for the large chunks of a prefill-size call: one persistent workgroup of eight waves per
// compute unit, operands in one continuous pipeline across work items.
//
// The tile kernels (b1_tile.h) pay, per work item, for looking the item up, for the wait on its
// first operands and for an epilogue during which no MFMA issues: a third of FC2's time at 8192
// tokens. Here a workgroup walks a list of items and never drains its pipeline between them:
//   * the direct-to-LDS loads run two k-steps ahead of the MFMAs and simply move on to the next
//     item's operands when the current item's last two k-steps are multiplied;
//   * a wave holds two sets of accumulators (4 weight tiles x 4 activation tiles, 64 registers
//     each). While one set accumulates item n, the finished set of item n-1 leaves for y[route]
//     between those MFMAs: one activation tile every four k-steps, regrouped through a private
//     strip of LDS into 256-byte runs per route exactly as the tile kernel does;
//   * an item's first k-step multiplies onto a zero addend, so no accumulator is cleared.
// Waves w and w+4 share a weight ring (same 64 output columns, rows 0..63 and 64..127 of the
// chunk), so a 128-row chunk still streams its weights once; all eight share the activation ring.
//
// Only chunks of five to eight groups come here (their records are collected by
// gather_scales_kernel); the tile kernel keeps the smaller ones. Rows that hold no token multiply
// whatever lies in the intermediate buffer: MFMA rows are independent and such rows are never
// stored, which spares the pipeline a per-lane lookup of which rows are live.
//
// Reference counterpart: fc2_m64 (crates/mimo26-spark/kernels/b1_fc1_m64.cuh:378-491), whose CTA
// also walks several tiles; the pipeline across items and the deferred stores are new.
//
// LDS, dynamic: [4 column blocks][3 stages][4 tiles][64 lanes][16 B]   weights, 48 KB
//               [3 stages][8 tiles][2 halves][64 lanes][16 B]          activations, 48 KB
//               [8 waves][16 cells of 272 B]                           regrouping strips, 34 KB
#pragma once
#include "b1_tile.h"

namespace m26g {

constexpr int kStreamThreads = 512, kStreamWaves = 8, kStreamStages = 3, kStreamSteps = 16;  // k-steps per item: I = 2048
constexpr uint32_t kStreamWeightRing = 4 * kStreamStages * 4096, kStreamActRing = kStreamStages * 16384;
constexpr uint32_t kStreamStrip = 16 * 272;
constexpr uint32_t kStreamLdsBytes = kStreamWeightRing + kStreamActRing + kStreamWaves * kStreamStrip;

// A large chunk as the stream kernel wants it: everything one scalar load away from the item index.
struct BigChunk { int32_t chunk, expert, first_group, groups; };
static_assert(sizeof(BigChunk) == 16, "one 16-byte record");
// big[0].chunk counts the records that follow from big[1] on (written by gather_scales_kernel).

#define M26G_MFMA_NEW(sel_text)                                                                                \
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 " sel_text " cbsz:4"                   \
                 : "=a"(acc) : "v"(a), "v"(b), "v"(sa), "v"(sb))
// acc = A x B (zero addend): the first k-step of an item.
template <int SEL>
__device__ __forceinline__ void mfma_new(v4f& acc, const v4i& a, const v8i& b, uint32_t sa, uint32_t sb) {
    if constexpr (SEL == 0) M26G_MFMA_NEW("op_sel_hi:[0,0,0]");
    else if constexpr (SEL == 1) M26G_MFMA_NEW("op_sel:[1,1,0] op_sel_hi:[0,0,0]");
    else if constexpr (SEL == 2) M26G_MFMA_NEW("op_sel_hi:[1,1,0]");
    else M26G_MFMA_NEW("op_sel:[1,1,0] op_sel_hi:[1,1,0]");
}
#undef M26G_MFMA_NEW

struct StreamArgs {
    Fc2Args f;
    const BigChunk* big;  // [0] = count, records from [1]
};

// grid = compute units (a multiple of 8), 512 threads. Workgroup g serves XCD g % 8.
__global__ void __launch_bounds__(kStreamThreads, 1) fc2_stream_kernel(StreamArgs s) {
    extern __shared__ __align__(16) uint8_t lds[];
    const Fc2Args& a = s.f;
    uint32_t* meta = a.plan.meta;
    if (meta[kPlanFault] || meta[kFc1Fault] || meta[kQuantFault]) return;
    const uint32_t lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), p = wv & 3, h = wv >> 2;
    const uint32_t xcd = blockIdx.x & 7, local = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
    // The list is cut into pairs of neighbouring records (two chunks of one expert, mostly); pair number
    // n belongs to XCD n % 8, and its 32 items (16 column blocks x 2 chunks, the two chunks of a column
    // side by side) are dealt round-robin to that XCD's workgroups: with 32 of them the two chunks run
    // at the same time, column for column, and stream the same weights through one L2.
    const uint32_t nbig = uint32_t(s.big[0].chunk), pairs = (nbig + 1) / 2;
    const uint32_t mine_pairs = pairs > xcd ? (pairs - xcd + 7) / 8 : 0, seq = mine_pairs * 32;
    const uint32_t items = seq > local ? (seq - local + per_xcd - 1) / per_xcd : 0;
    if (items == 0) return;
    constexpr int KS = kStreamSteps;
    const uint32_t I = a.lay.inter;

    uint8_t* wring = lds + p * (kStreamStages * 4096);
    uint8_t* aring = lds + kStreamWeightRing;
    uint8_t* strip = lds + kStreamWeightRing + kStreamActRing + wv * kStreamStrip;
    const uint32_t wring_at = uint32_t(uintptr_t((lds_ptr)wring)) + lane * 16;
    const uint32_t aring_at = uint32_t(uintptr_t((lds_ptr)aring)) + lane * 16 + h * (4 * 2048);  // this wave's four tiles
    const uint32_t put_at = uint32_t(uintptr_t((lds_ptr)strip)) + (lane >> 4) * 272 + (lane & 15) * 16;
    const uint32_t get_at = uint32_t(uintptr_t((lds_ptr)strip)) + (lane & 15) * 272 + (lane >> 4) * 16;

    // Item k of this workgroup: position in the XCD's sequence -> (large chunk, column block).
    struct Item { BigChunk rec; uint32_t ob; };
    // Position q in the XCD's sequence -> record and column block. An odd list ends in half a pair: its
    // missing chunk is the last record once more (the same rows written twice with the same values).
    auto record_of = [&](uint32_t q) {
        const uint32_t b = ((q / 32) * 8 + xcd) * 2 + (q & 1);
        return b < nbig ? b : nbig - 1;
    };
    auto item_of = [&](uint32_t k) {
        const uint32_t q = local + k * per_xcd;
        return Item{s.big[1 + record_of(q)], ((q % 32) >> 1) * 4 + p};
    };
    // Addresses are a uniform base (scalar registers) plus a 32-bit lane offset: the prepared pool, the
    // intermediate and y all stay below 4 GB, and 64-bit lane pointers for every stream would not fit
    // beside two sets of accumulators.
    auto weights_of = [&](const Item& it) {  // offset into the prepared pool of this wave's weight stream
        return uint32_t(uint64_t(it.rec.expert) * a.lay.bytes() + a.lay.w2() + uint64_t(it.ob) * (KS * 4096)) + lane * 16;
    };
    auto rows_of = [&](const Item& it) {  // offset into the intermediate of this lane's row of activation tile wv
        return uint32_t((size_t(it.rec.first_group + int32_t(wv)) * 16 + (lane & 15)) * I) + (lane >> 4) * 16;
    };
    auto weight_scales_of = [&](const Item& it) {  // uniform
        return a.prepared + uint64_t(it.rec.expert) * a.lay.bytes() + a.lay.s2() + uint64_t(it.ob) * ((KS / 4) * 1024);
    };
    auto act_scales_of = [&](const Item& it) {  // uniform
        return a.dg + size_t(it.rec.chunk) * gathered_scale_bytes(I) + h * (4 * 256);
    };
    const uint32_t lane4 = lane * 4;

    // Later records are fetched with a scalar load issued by hand at an item's end and first read
    // twelve k-steps on: left to the compiler the lookup is a vector load, and the wait for it
    // drains the whole operand pipeline at every item boundary.
    auto request_record = [&](uint32_t k, v4i& raw) {
        const uint32_t q = local + k * per_xcd;
        const BigChunk* at = s.big + 1 + record_of(q);
        asm volatile("s_load_dwordx4 %0, %1, 0x0" : "=s"(raw) : "s"(at) : "memory");
    };
    Item cur = item_of(0), nxt = item_of(items > 1 ? 1 : 0);
    v4i nxt_raw = {nxt.rec.chunk, nxt.rec.expert, nxt.rec.first_group, nxt.rec.groups};
    uint32_t nxt_index = items > 1 ? 1 : 0;
    uint32_t wl = weights_of(cur);  // the loader's place, two k-steps ahead of the MFMAs
    uint32_t xl = rows_of(cur);
    const uint8_t* sw_at = weight_scales_of(cur);
    const uint8_t* sa_at = act_scales_of(cur);
    // The loads of one k-step for this wave: activation tile wv (two 64-byte halves of its rows) and
    // weight tiles 2h, 2h+1 of column block p. Four per k-step; the waits below count on that.
    auto stage_item = [&](int item, uint32_t stage) {
        if (item < 2) load_row_to_lds(a.dq + (xl + item * 64), aring + ((stage * 8 + wv) * 2 + item) * 1024);
        else load_row_to_lds(a.prepared + (wl + (2 * h + item - 2) * 1024), wring + stage * 4096 + (2 * h + item - 2) * 1024);
    };
    v4i af[4];  // one set: a tile's fragment of the next k-step is fetched right behind the last MFMA that reads the old one
    auto read_weights = [&](v4i (&f)[4], uint32_t stage) {
        const uint32_t at = wring_at + stage * 4096;
#pragma unroll
        for (int t = 0; t < 4; ++t) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f[t]) : "v"(at), "n"(t * 1024) : "memory");
    };
    uint32_t sw0[4], sa0[4], sw1[4], sa1[4];
    auto load_scales = [&](uint32_t (&w)[4], uint32_t (&x)[4], const uint8_t* pw, const uint8_t* px) {
#pragma unroll
        for (int t = 0; t < 4; ++t) asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(w[t]) : "v"(lane4), "s"(pw), "n"(t * 256) : "memory");
#pragma unroll
        for (int t = 0; t < 4; ++t) asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(x[t]) : "v"(lane4), "s"(px), "n"(t * 256) : "memory");
    };
    v4f accA[4][4], accB[4][4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) accB[t][g] = v4f{0.f, 0.f, 0.f, 0.f};  // "finished" before the first item: stored to the spare row

    // Start of the stream: k-steps 0 and 1 of the first item.
    load_scales(sw0, sa0, sw_at, sa_at);
#pragma unroll
    for (int item = 0; item < 4; ++item) stage_item(item, 0);
    wl += 4096; xl += 128;
#pragma unroll
    for (int item = 0; item < 4; ++item) stage_item(item, 1);
    wl += 4096; xl += 128;
    wait_loads_but<4>();
    lds_barrier();
    read_weights(af, 0);
    v4i lo, hi;  // the activation fragment the next MFMA group multiplies
    read_fragment(lo, hi, aring_at);
    uint32_t st = 0;  // stage the MFMAs read; st+1 holds the next k-step, st+2 takes this step's loads
    uint32_t done = 0;
    // The finished set's way out, for activation tile G (one every four k-steps):
    //   step 4G    four route lookups (row 4j + lane/16 of the tile), hand-issued like the scales;
    //   step 4G+1  the tile's four 16x16 blocks into the strip (a lane holds four columns of one token);
    //   steps 4G+2, 4G+3  two stores each: a lane now holds 16 bytes of a 256-byte run, four tokens a store.
    // Dead rows (route -1) and routes beyond the call go to the spare row behind y.
    uint32_t prev_chunk = 0, prev_ob = 0;
    bool have_prev = false;
    int32_t route[4];

    // One k-step. S = its index inside the item (scale byte S % 4), ACC the set it accumulates, PREV the
    // finished set. VM = vector-memory operations this step issues ahead of its closing wait, which
    // lets exactly those stay in flight: everything older, the next k-step's operands included, has landed.
#define M26G_STREAM_STEP(S, ACC, PREV, SW, SA)                                                                    \
    {                                                                                                             \
        constexpr int B = (S) & 3, G = (S) >> 2;                                                                   \
        constexpr int VM = 4 + (B == 0 ? 8 + 4 : 0) + (B >= 2 ? 2 : 0);                                            \
        const uint32_t st1 = st == kStreamStages - 1 ? 0 : st + 1, st2 = st1 == kStreamStages - 1 ? 0 : st1 + 1;  \
        const uint32_t fs = aring_at + st * 16384;                                                                \
        if (B == 0) {                                                                                             \
            const int32_t* yr = a.yrows + size_t(prev_chunk) * 128 + (4 * prev_h_tile + G) * 16; /* uniform */      \
            _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                         \
                asm volatile("global_load_dword %0, %1, %2 offset:%3" : "=v"(route[j]) : "v"(token4x4), "s"(yr), "n"(j * 16) : "memory"); \
        }                                                                                                         \
        _Pragma("unroll") for (int tt = 0; tt < 4; ++tt) {                                                        \
            v4i nlo = lo, nhi = hi;                                                                               \
            if (tt == 3) {                                                                                        \
                stage_item(3, st2);                                                                               \
                __builtin_amdgcn_sched_barrier(0);                                                                \
                wait_loads_but<VM>();                                                                             \
                lds_barrier();                                                                                    \
                read_fragment(nlo, nhi, aring_at + st1 * 16384);                                                  \
            } else {                                                                                              \
                wait_lds_but<0>();                                                                                \
            }                                                                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            const v8i bv = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};                                      \
            if ((S) == 0) mfma_new<B>(ACC[0][tt], af[0], bv, SW[0], SA[tt]);                               \
            else mfma_acc<B>(ACC[0][tt], af[0], bv, SW[0], SA[tt]);                                                 \
            if (tt == 3) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[0]) : "v"(wring_at + st1 * 4096), "n"(0 * 1024) : "memory");                                        \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            if (tt < 3) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(nlo) : "v"(fs), "n"((tt < 3 ? tt + 1 : 0) * 2048) : "memory"); \
            /* through four vector registers: handed over as an accumulator operand the tile is first copied */ \
            /* to spare accumulation registers, and with both sets alive there are none                     */ \
            if (B == 1) asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(put_at), "v"(PREV[tt][G]), "n"(tt * 4 * 272) : "memory"); \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            if ((S) == 0) mfma_new<B>(ACC[1][tt], af[1], bv, SW[1], SA[tt]);                               \
            else mfma_acc<B>(ACC[1][tt], af[1], bv, SW[1], SA[tt]);                                                 \
            if (tt == 3) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[1]) : "v"(wring_at + st1 * 4096), "n"(1 * 1024) : "memory");                                        \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            if (tt < 3) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(nhi) : "v"(fs), "n"((tt < 3 ? tt + 1 : 0) * 2048 + 1024) : "memory"); \
            v4i out;                                                                                              \
            if (B >= 2 && tt < 2) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(out) : "v"(get_at), "n"(((B >= 2 ? 2 * (B - 2) : 0) + (tt < 2 ? tt : 0)) * 64) : "memory"); \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            if ((S) == 0) mfma_new<B>(ACC[2][tt], af[2], bv, SW[2], SA[tt]);                               \
            else mfma_acc<B>(ACC[2][tt], af[2], bv, SW[2], SA[tt]);                                                 \
            if (tt == 3) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[2]) : "v"(wring_at + st1 * 4096), "n"(2 * 1024) : "memory");                                        \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            if (tt < 3) stage_item(tt, st2);                                                                      \
            if (B >= 2 && tt < 2) {                                                                               \
                wait_lds_but<0>();                                                                                \
                int32_t rt = route[(B >= 2 ? 2 * (B - 2) : 0) + (tt < 2 ? tt : 0)];                                                             \
                asm volatile("" : "+v"(rt), "+v"(out)); /* read only behind the waits above */                    \
                /* -1 (no token) and anything else past the call's routes: the spare row */                     \
                const uint32_t row = !have_prev || uint32_t(rt) >= a.routes ? a.routes : uint32_t(rt);            \
                asm volatile("global_store_dwordx4 %0, %1, %2" ::"v"(row * (kHidden * 4) + cell16), "v"(out), "s"(a.y + prev_ob * 64) : "memory"); \
            }                                                                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            if ((S) == 0) mfma_new<B>(ACC[3][tt], af[3], bv, SW[3], SA[tt]);                               \
            else mfma_acc<B>(ACC[3][tt], af[3], bv, SW[3], SA[tt]);                                                 \
            if (tt == 3) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(af[3]) : "v"(wring_at + st1 * 4096), "n"(3 * 1024) : "memory");                                        \
            __builtin_amdgcn_sched_barrier(0);                                                                    \
            lo = nlo;                                                                                             \
            hi = nhi;                                                                                             \
        }                                                                                                         \
        st = st1;                                                                                                 \
        if ((S) == KS - 3) { wl = weights_of(nxt); xl = rows_of(nxt); } /* the loader enters the next item */     \
        else { wl += 4096; xl += 128; }                                                                           \
        asm volatile("" : "+v"(wl), "+v"(xl)); /* one running offset each: nothing derived from them is kept */   \
    }
    // A quad of k-steps on one set of scales; the other set is fetched for the quad after it, which
    // for the last quad of an item is the first quad of the next item.
#define M26G_STREAM_QUAD(Q, ACC, PREV, SW, SA, NW, NA)                                                            \
    {                                                                                                             \
        if ((Q) == 3) {                                                                                           \
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* the next item's record, requested an item ago */  \
            asm volatile("" : "+s"(nxt_raw));                                                                     \
            const uint32_t q_ = local + nxt_index * per_xcd;                                                      \
            nxt = Item{BigChunk{nxt_raw.x, nxt_raw.y, nxt_raw.z, nxt_raw.w}, ((q_ % 32) >> 1) * 4 + p};            \
            load_scales(NW, NA, weight_scales_of(nxt), act_scales_of(nxt));                                       \
        }                                                                                                         \
        else load_scales(NW, NA, sw_at + ((Q) + 1) * 1024, sa_at + ((Q) + 1) * 2048);                             \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        M26G_STREAM_STEP(4 * (Q) + 0, ACC, PREV, SW, SA)                                                          \
        M26G_STREAM_STEP(4 * (Q) + 1, ACC, PREV, SW, SA)                                                          \
        M26G_STREAM_STEP(4 * (Q) + 2, ACC, PREV, SW, SA)                                                          \
        M26G_STREAM_STEP(4 * (Q) + 3, ACC, PREV, SW, SA)                                                          \
    }
#define M26G_STREAM_ITEM(ACC, PREV)                                                                               \
    {                                                                                                             \
        M26G_STREAM_QUAD(0, ACC, PREV, sw0, sa0, sw1, sa1)                                                        \
        M26G_STREAM_QUAD(1, ACC, PREV, sw1, sa1, sw0, sa0)                                                        \
        M26G_STREAM_QUAD(2, ACC, PREV, sw0, sa0, sw1, sa1)                                                        \
        M26G_STREAM_QUAD(3, ACC, PREV, sw1, sa1, sw0, sa0)                                                        \
        /* The fragments fetched for the next k-step land before control leaves this block: where two    */   \
        /* blocks meet the compiler may move them to other registers, and it takes them for loaded.       */   \
        wait_lds_but<0>();                                                                                        \
        asm volatile("" : "+v"(lo), "+v"(hi), "+v"(af[0]), "+v"(af[1]), "+v"(af[2]), "+v"(af[3]));                 \
        /* the set just filled becomes the finished one; the item after next is looked up */                     \
        prev_chunk = uint32_t(cur.rec.chunk);                                                                     \
        prev_ob = cur.ob;                                                                                         \
        have_prev = true;                                                                                         \
        ++done;                                                                                                   \
        cur = nxt;                                                                                                \
        sw_at = weight_scales_of(cur);                                                                            \
        sa_at = act_scales_of(cur);                                                                               \
        nxt_index = done + 1 < items ? done + 1 : items - 1;                                                      \
        request_record(nxt_index, nxt_raw);                                                                       \
    }
    const uint32_t prev_h_tile = h;  // the finished set covers activation tiles 4h .. 4h+3
    const uint32_t token4x4 = (lane >> 4) * 4, cell16 = (lane & 15) * 16;  // byte offsets of this lane's route word and of its 16 bytes of a run
    // One pass more than there are items: the last pass multiplies the last item again and stores
    // nothing of it; under it the last finished set leaves like every other. (Storing it after the
    // loop instead would keep both sets alive across the whole loop for the register allocator, which
    // then has no room left for the operands.)
#pragma unroll 1
    for (;;) {
        M26G_STREAM_ITEM(accA, accB)
        if (done > items) break;
        M26G_STREAM_ITEM(accB, accA)
        if (done > items) break;
    }
#undef M26G_STREAM_ITEM
#undef M26G_STREAM_QUAD
#undef M26G_STREAM_STEP
    wait_loads_but<0>();  // the loads staged past the end, and the last stores
    wait_lds_but<0>();
#pragma unroll
    for (int t = 0; t < 4; ++t) asm volatile("" ::"v"(sw0[t]), "v"(sw1[t]), "v"(sa0[t]), "v"(sa1[t]), "v"(af[t]), "v"(route[t]));
    asm volatile("" ::"v"(lo), "v"(hi));
}

}  // namespace m26g
