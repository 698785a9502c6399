// C ABI of the gfx950 routed-expert FFN: handles, buffer ownership, launch schedule, fault decode.
// Mirrors the contract of crates/mimo26-spark/kernels/b1_serve.cu:145-574 of the reference (names,
// argument meaning, return codes, the ms[8] phase report); the schedule itself is new: no host
// round trip between the planner and the GEMMs (grids are sized by capacity and idle workgroups
// leave on the device-side counts), and the intermediate quantizer is fused into FC1.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/m26s_b1.h"
#include "b1_stream.h"

using namespace m26g;

namespace {

struct Dev {
    void* p = nullptr;
    size_t n = 0;
    hipError_t ensure(size_t bytes) {
        if (bytes <= n) return hipSuccess;
        if (p) (void)hipFree(p);
        p = nullptr;
        n = 0;
        const size_t want = bytes < 256 ? 256 : bytes;
        const hipError_t e = hipMalloc(&p, want);
        if (e == hipSuccess) n = want;
        return e;
    }
    template <class T> T* as() const { return static_cast<T*>(p); }
    ~Dev() { if (p) (void)hipFree(p); }
};

void set_err(char* err, size_t len, const char* what, hipError_t e) {
    if (err && len) std::snprintf(err, len, "%s: %s", what, hipGetErrorString(e));
}
void set_msg(char* err, size_t len, const char* msg) {
    if (err && len) std::snprintf(err, len, "%s", msg);
}

uint32_t capacity_class(uint32_t rows) { return rows <= 256 ? 256u : rows <= 2048 ? 2048u : rows <= 4096 ? 4096u : 8192u; }
// Groups of at most 16 rows: every expert adds at most one ragged group.
uint64_t group_bound(uint64_t routes) { const uint64_t b = routes / 16 + kExperts; return b < routes ? b : routes; }
uint64_t chunk_bound(uint64_t routes, uint32_t gpc) {
    const uint64_t b = routes / (16ull * gpc) + 2 * kExperts;
    return b < routes ? b : routes;
}
// Activation tiles one wave carries: decode-size calls keep one pass over each touched expert's
// weights for up to 32 rows; larger calls reuse each weight fragment over 128 rows. The tile schedule
// runs small chunks through the same register-only bodies, and measured from 192 rows up it is never
// slower than the direct one (Zipf routing: 0.51 against 0.53 ms at 192 rows, 0.62 against 0.67 at 384).
constexpr uint32_t kWidePlanFrom = 512;  // rows above which the planner runs on several compute units
uint32_t tiles_for(uint32_t rows) { return rows <= 32 ? 1u : rows <= 128 ? 2u : 8u; }

// Kernels whose dynamic LDS passes 64 KB need the limit raised once per process.
bool lds_ready = false;
uint32_t compute_units = 0;  // of the device the first scratch was made on
hipError_t plan_lds_attr() {
    if (lds_ready) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(plan_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(kMaxRows * kTopk));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fc1_tile_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(kTileLdsBytes));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fc2_tile_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(kTileLdsBytes));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fc2_stream_kernel),
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(kStreamLdsBytes));
    int device = 0, cus = 0;
    if (e == hipSuccess) e = hipGetDevice(&device);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
    compute_units = uint32_t(cus);
    lds_ready = e == hipSuccess;
    return e;
}

}  // namespace

struct m26s_b1_layer {
    uint8_t* prepared = nullptr;
    uint8_t* resident = nullptr;
    Prepared lay{};
    bool all_normal = false;
};

struct m26s_b1_scratch {
    hipStream_t st = nullptr;
    bool own_stream = false;
    hipEvent_t e0 = nullptr, ep = nullptr, ea = nullptr, ec = nullptr, e1 = nullptr;
    Dev x, xs, iw, inv, orig, gw, groups, chunks, meta, dq, dqs, y, bf16, pad, tap_gate, tap_up, tap_h, xg, rowbad, dg, planw, xrows, yrows, big;
    std::vector<uint8_t> hiw;
    bool taps = false;
    bool stream_fc2 = false;  // FC2's large chunks through the persistent kernel of b1_stream.h
    uint32_t last_rows = 0, last_inter = 0;
};

namespace {

int layer_build(const Canonical& c, uint32_t inter, m26s_b1_layer** out, char* err, size_t errlen) {
    auto* L = new (std::nothrow) m26s_b1_layer();
    if (!L) { set_msg(err, errlen, "b1 layer: host allocation failed"); return 2; }
    L->lay.inter = inter;
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&L->prepared), L->lay.bytes() * kExperts);
    if (e != hipSuccess) { set_err(err, errlen, "b1 layer prepared alloc", e); delete L; return 2; }
    uint32_t* flag = nullptr;
    uint32_t h = 1;
    std::vector<uint8_t> present(kExperts, 1);
    if ((e = hipMalloc(reinterpret_cast<void**>(&L->resident), kExperts)) != hipSuccess ||
        (e = hipMemcpy(L->resident, present.data(), kExperts, hipMemcpyHostToDevice)) != hipSuccess ||
        (e = hipMalloc(reinterpret_cast<void**>(&flag), 4)) != hipSuccess ||
        (e = hipMemset(flag, 0, 4)) != hipSuccess) {
        set_err(err, errlen, "b1 layer metadata", e);
        m26s_b1_layer_free(L);
        return 2;
    }
    prepare_kernel<<<dim3(inter / 8, kExperts), 256>>>(c, L->prepared, L->lay, flag);
    if ((e = hipGetLastError()) != hipSuccess || (e = hipMemcpy(&h, flag, 4, hipMemcpyDeviceToHost)) != hipSuccess ||
        (e = hipDeviceSynchronize()) != hipSuccess) {
        (void)hipFree(flag);
        set_err(err, errlen, "b1 prepare", e);
        m26s_b1_layer_free(L);
        return 2;
    }
    (void)hipFree(flag);
    L->all_normal = h == 0;
    *out = L;
    return 0;
}

int scratch_build(hipStream_t stream, bool own, m26s_b1_scratch** out, char* err, size_t errlen) {
    if (!out) { set_msg(err, errlen, "b1 scratch: null out"); return 1; }
    auto* S = new (std::nothrow) m26s_b1_scratch();
    if (!S) { set_msg(err, errlen, "b1 scratch: host allocation failed"); return 1; }
    hipError_t e = hipSuccess;
    S->st = stream;
    S->own_stream = own;
    if ((own && (e = hipStreamCreateWithFlags(&S->st, hipStreamNonBlocking)) != hipSuccess) ||
        (e = hipEventCreate(&S->e0)) != hipSuccess || (e = hipEventCreate(&S->ep)) != hipSuccess ||
        (e = hipEventCreate(&S->ea)) != hipSuccess || (e = hipEventCreate(&S->ec)) != hipSuccess ||
        (e = hipEventCreate(&S->e1)) != hipSuccess || (e = S->meta.ensure(kMetaWords * 4)) != hipSuccess ||
        (e = S->pad.ensure(8192 + 256)) != hipSuccess ||
        (e = hipMemset(S->pad.p, 0, 8192)) != hipSuccess ||
        (e = hipMemset(S->pad.as<uint8_t>() + 8192, 127, 256)) != hipSuccess || (e = plan_lds_attr()) != hipSuccess) {
        set_err(err, errlen, "b1 scratch stream/events", e);
        m26s_b1_scratch_free(S);
        return 1;
    }
    meta_reset_kernel<<<1, 64, 0, S->st>>>(S->meta.as<uint32_t>());
    if ((e = hipGetLastError()) != hipSuccess || (e = hipDeviceSynchronize()) != hipSuccess) {
        set_err(err, errlen, "b1 scratch meta", e);
        m26s_b1_scratch_free(S);
        return 1;
    }
    *out = S;
    return 0;
}

#define M26S_CK(expr, what) do { if ((e = (expr)) != hipSuccess) { set_err(err, errlen, what, e); return 2; } } while (0)

template <int NT>
void launch_ffn(const m26s_b1_layer* L, m26s_b1_scratch* S, const PlanView& pv, const uint8_t* x, size_t xp,
                const uint8_t* xs, size_t xsp, uint32_t chunk_cap, uint64_t routes) {
    const uint8_t* zero = S->pad.as<uint8_t>();
    Fc1Args f1{L->prepared, L->lay, pv, x, xp, xs, xsp, zero, zero + 8192, S->dq.as<uint8_t>(), S->dqs.as<uint8_t>(),
               S->taps ? S->tap_gate.as<float>() : nullptr, S->taps ? S->tap_up.as<float>() : nullptr,
               S->taps ? S->tap_h.as<float>() : nullptr, nullptr, nullptr, nullptr, nullptr};
    fc1_kernel<NT><<<dim3(L->lay.inter / 128, chunk_cap), 256, 0, S->st>>>(f1);
    (void)hipEventRecord(S->ea, S->st);
    Fc2Args f2{L->prepared, L->lay, pv, S->dq.as<uint8_t>(), S->dqs.as<uint8_t>(), zero, zero + 8192,
               S->y.as<float>(), uint32_t(routes), nullptr, nullptr, nullptr, 0};
    fc2_kernel<NT><<<dim3(16 / kFc2Blocks, chunk_cap), 256, 0, S->st>>>(f2);
    (void)hipEventRecord(S->ec, S->st);
}

// Prefill-size calls: workgroups that share each chunk's activation tiles through LDS, two per compute unit.
void launch_tiles(const m26s_b1_layer* L, m26s_b1_scratch* S, const PlanView& pv, const uint8_t* x, size_t xp,
                  const uint8_t* xs, size_t xsp, uint32_t chunk_cap, uint64_t routes) {
    const uint8_t* zero = S->pad.as<uint8_t>();
    const uint32_t inter = L->lay.inter;
    // Full-intermediate layers hand FC2's large chunks to the persistent stream kernel (b1_stream.h).
    const bool stream = S->stream_fc2 && inter == kStreamSteps * 128 && compute_units >= 8;
    gather_scales_kernel<<<chunk_cap, 256, 0, S->st>>>(pv, xs, xsp, S->xg.as<uint32_t>(), S->rowbad.as<uint32_t>(),
                                                     S->xrows.as<int32_t>(), S->yrows.as<int32_t>(),
                                                     stream ? S->big.as<int32_t>() : nullptr);
    Fc1Args f1{L->prepared, L->lay, pv, x, xp, xs, xsp, zero, zero + 8192, S->dq.as<uint8_t>(), S->dqs.as<uint8_t>(),
               S->taps ? S->tap_gate.as<float>() : nullptr, S->taps ? S->tap_up.as<float>() : nullptr,
               S->taps ? S->tap_h.as<float>() : nullptr, S->xg.as<uint8_t>(), S->rowbad.as<uint32_t>(), S->xrows.as<int32_t>(),
               S->dg.as<uint8_t>()};
    fc1_tile_kernel<<<tile_grid(inter / 128, chunk_cap), kTileThreads, kTileLdsBytes, S->st>>>(f1);
    (void)hipEventRecord(S->ea, S->st);
    Fc2Args f2{L->prepared, L->lay, pv, S->dq.as<uint8_t>(), S->dqs.as<uint8_t>(), zero, zero + 8192,
               S->y.as<float>(), uint32_t(routes), S->dg.as<uint8_t>(), S->yrows.as<int32_t>(), S->rowbad.as<uint32_t>(), 0};
    if (stream) {
        fc2_stream_kernel<<<compute_units / 8 * 8, kStreamThreads, kStreamLdsBytes, S->st>>>(StreamArgs{f2, S->big.as<BigChunk>()});
        f2.skip_from = kStreamFromGroups;
    }
    fc2_tile_kernel<<<tile_grid(kHidden / 256, chunk_cap), kTileThreads, kTileLdsBytes, S->st>>>(f2);
    (void)hipEventRecord(S->ec, S->st);
}

// Enqueue plan -> FC1(+quantizer) -> FC2 -> reduce on device-resident inputs. No host wait.
int enqueue(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* x, size_t xp, const uint8_t* xs, size_t xsp,
            const int32_t* ids, const float* w, uint32_t rows, uint16_t* bf16_out, float* partial, char* err,
            size_t errlen) {
    hipError_t e;
    const uint32_t cap = capacity_class(rows), nt = tiles_for(rows), inter = L->lay.inter;
    const uint64_t routes = uint64_t(rows) * kTopk, route_cap = uint64_t(cap) * kTopk;
    const uint64_t gcap = group_bound(routes), ccap = chunk_bound(routes, nt);
    M26S_CK(S->inv.ensure(route_cap * 4), "b1 inv alloc");
    M26S_CK(S->orig.ensure(route_cap * 4), "b1 orig alloc");
    M26S_CK(S->gw.ensure(route_cap * 4), "b1 gw alloc");
    M26S_CK(S->groups.ensure(route_cap * sizeof(Group)), "b1 groups alloc");
    M26S_CK(S->chunks.ensure(route_cap * sizeof(Chunk)), "b1 chunks alloc");
    // Eight groups of slack behind the intermediate and one spare row behind y: the stream kernel reads
    // all eight tiles of a chunk whatever its group count, and parks the rows that hold no token.
    M26S_CK(S->dq.ensure((gcap + 8) * 16 * inter), "b1 dq alloc");
    M26S_CK(S->dqs.ensure(gcap * 16 * inter / 32), "b1 dqs alloc");
    M26S_CK(S->y.ensure((routes + 1) * kHidden * 4), "b1 y alloc");
    if (nt > 2) {
        M26S_CK(S->xg.ensure(ccap * gathered_scale_bytes(kHidden)), "b1 gathered input scales alloc");
        M26S_CK(S->dg.ensure(ccap * gathered_scale_bytes(inter)), "b1 gathered intermediate scales alloc");
        // The tile kernels fetch these beside their chunk record, before they know whether the chunk exists:
        // the tables cover the whole grid (chunk capacity rounded up to runs on eight XCDs).
        M26S_CK(S->rowbad.ensure((ccap + 8 * kTileRun) * 16 * 4), "b1 row verdict alloc");
        M26S_CK(S->xrows.ensure((ccap + 8 * kTileRun) * 128 * 4), "b1 chunk row table alloc");
        M26S_CK(S->yrows.ensure(ccap * 128 * 4), "b1 chunk route table alloc");
        M26S_CK(S->big.ensure((ccap + 1) * sizeof(BigChunk)), "b1 large chunk list alloc");
    }
    if (S->taps) {
        M26S_CK(S->tap_gate.ensure(gcap * 16 * inter * 4), "b1 gate tap alloc");
        M26S_CK(S->tap_up.ensure(gcap * 16 * inter * 4), "b1 up tap alloc");
        M26S_CK(S->tap_h.ensure(gcap * 16 * inter * 4), "b1 h tap alloc");
    }
    const PlanView pv{S->inv.as<int32_t>(), S->orig.as<int32_t>(), S->gw.as<float>(), S->groups.as<Group>(),
                      S->chunks.as<Chunk>(), S->meta.as<uint32_t>()};
    M26S_CK(hipEventRecord(S->e0, S->st), "b1 event 0");
    // Stage faults accumulate across enqueued calls until the next sync; only the plan words reset.
    if (rows > kWidePlanFrom) {  // several compute units share the scatter (b1_kernels.h, "Stage 1 for large calls")
        const void* before = S->planw.p;
        M26S_CK(S->planw.ensure(wide_plan_words(uint32_t(route_cap)) * 4), "b1 plan work alloc");
        if (S->planw.p != before) M26S_CK(hipMemsetAsync(S->planw.p, 0xff, 16, S->st), "b1 plan work arm");  // a new buffer: no fault yet
        const uint32_t wide = wide_plan_groups(uint32_t(routes));
        plan_count_kernel<<<wide, kPlanThreads, 0, S->st>>>(ids, w, rows, L->resident, S->planw.as<uint32_t>());
        plan_scan_kernel<<<1, kPlanThreads, 0, S->st>>>(uint32_t(routes), S->planw.as<uint32_t>(), pv, nt);
        plan_place_kernel<<<wide, kPlanThreads, 0, S->st>>>(ids, w, rows, S->planw.as<uint32_t>(), pv, S->taps);
    } else {
        plan_kernel<<<1, kPlanThreads, routes, S->st>>>(ids, w, rows, L->resident, pv, nt, 0, S->taps);
    }
    M26S_CK(hipGetLastError(), "b1 plan launch");
    M26S_CK(hipEventRecord(S->ep, S->st), "b1 event p");
    if (nt == 1) launch_ffn<1>(L, S, pv, x, xp, xs, xsp, uint32_t(ccap), routes);
    else if (nt == 2) launch_ffn<2>(L, S, pv, x, xp, xs, xsp, uint32_t(ccap), routes);
    else launch_tiles(L, S, pv, x, xp, xs, xsp, uint32_t(ccap), routes);
    M26S_CK(hipGetLastError(), "b1 fc launch");
    const uint64_t n4 = uint64_t(rows) * (kHidden / 4);
    const uint32_t blocks = uint32_t(n4 / 256 < 65536 ? (n4 + 255) / 256 : 65536);
    reduce_kernel<<<blocks, 256, 0, S->st>>>(S->y.as<float>(), w, rows, partial, bf16_out,
                                             S->meta.as<uint32_t>() + kReduceFault, S->meta.as<uint32_t>());
    M26S_CK(hipGetLastError(), "b1 reduce launch");
    M26S_CK(hipEventRecord(S->e1, S->st), "b1 event 1");
    S->last_rows = rows;
    S->last_inter = inter;
    return 0;
}

// Wait, read the eight meta words, translate them (b1_serve.cu:365-368, 551-562) and clear them.
int finish(m26s_b1_scratch* S, uint32_t* meta_out, char* err, size_t errlen) {
    hipError_t e;
    uint32_t m[kMetaWords];
    M26S_CK(hipMemcpyAsync(m, S->meta.p, sizeof m, hipMemcpyDeviceToHost, S->st), "b1 meta download");
    M26S_CK(hipStreamSynchronize(S->st), "b1 compute sync");
    meta_reset_kernel<<<1, 64, 0, S->st>>>(S->meta.as<uint32_t>());
    M26S_CK(hipGetLastError(), "b1 meta reset");
    if (meta_out) std::memcpy(meta_out, m, sizeof m);
    if (m[kPlanFault]) { set_msg(err, errlen, "b1 plan: invalid routes (id/residency/weight/duplicate)"); return 3; }
    if (S->last_rows && !m[kGroupCount]) { set_msg(err, errlen, "b1 plan: bad group count"); return 3; }
    if (err && errlen) {
        if (m[kFc1Fault]) std::snprintf(err, errlen, "b1 fc1 fault %u (groups %u)", m[kFc1Fault], m[kGroupCount]);
        else if (m[kQuantFault])
            std::snprintf(err, errlen, "b1 quantizer fault %u at word %u (groups %u)", m[kQuantFault] & 1 ? 1u : 2u,
                          m[kQuantWhere], m[kGroupCount]);
        else if (m[kFc2Fault]) std::snprintf(err, errlen, "b1 fc2 fault %u (groups %u)", m[kFc2Fault], m[kGroupCount]);
        else if (m[kReduceFault]) std::snprintf(err, errlen, "b1 reduce fault %u (groups %u)", m[kReduceFault], m[kGroupCount]);
    }
    return (m[kFc1Fault] | m[kQuantFault] | m[kFc2Fault] | m[kReduceFault]) ? 4 : 0;
}

void report(m26s_b1_scratch* S, float* ms, float host_front, float host_total, uint32_t groups) {
    if (!ms) return;
    float plan = 0, gpu = 0, ph[3] = {0, 0, 0};
    (void)hipEventElapsedTime(&plan, S->e0, S->ep);
    (void)hipEventElapsedTime(&gpu, S->ep, S->e1);
    (void)hipEventElapsedTime(&ph[0], S->ep, S->ea);
    (void)hipEventElapsedTime(&ph[1], S->ea, S->ec);
    (void)hipEventElapsedTime(&ph[2], S->ec, S->e1);
    ms[0] = host_front + plan;
    ms[1] = gpu;
    ms[2] = host_total - host_front - plan - gpu;
    if (ms[2] < 0) ms[2] = 0;
    ms[3] = float(groups);
    ms[4] = ph[0];
    ms[5] = 0.0f;  // the intermediate quantizer runs inside FC1
    ms[6] = ph[1];
    ms[7] = ph[2];
}

bool layer_usable(const m26s_b1_layer* L, char* err, size_t errlen) {
    if (L->all_normal) return true;
    set_msg(err, errlen, "b1 ffn: layer holds weight scale bytes outside [2,252]; no conforming path for them yet");
    return false;
}

}  // namespace

extern "C" {

int m26s_b1_layer_new(const uint8_t* canonical_dev, uint64_t canonical_bytes, uint32_t rank, m26s_b1_layer** out,
                      char* err, size_t errlen) {
    if (!canonical_dev || canonical_bytes != uint64_t(kExperts) * kImageBytes || rank >= 4 || !out) {
        set_msg(err, errlen, "b1 layer: bad canonical extent/rank");
        return 1;
    }
    Canonical c{{canonical_dev, nullptr, nullptr, nullptr}, 1};
    return layer_build(c, kRankI, out, err, errlen);
}

int m26s_b1_layer_new_full(const uint8_t* const rank_images_dev[4], uint64_t bytes_each, m26s_b1_layer** out,
                           char* err, size_t errlen) {
    if (!rank_images_dev || !out || bytes_each != uint64_t(kExperts) * kImageBytes || !rank_images_dev[0] ||
        !rank_images_dev[1] || !rank_images_dev[2] || !rank_images_dev[3]) {
        set_msg(err, errlen, "b1 layer: bad canonical extent/rank");
        return 1;
    }
    Canonical c{{rank_images_dev[0], rank_images_dev[1], rank_images_dev[2], rank_images_dev[3]}, 4};
    return layer_build(c, 4 * kRankI, out, err, errlen);
}

int m26s_b1_layer_all_normal(const m26s_b1_layer* L) { return L && L->all_normal ? 1 : 0; }
uint32_t m26s_b1_layer_intermediate(const m26s_b1_layer* L) { return L ? L->lay.inter : 0; }

int m26s_b1_layer_view(const m26s_b1_layer* L, const uint8_t** prepared_dev, uint64_t* image_bytes, uint32_t* layout_tag) {
    if (!L || !prepared_dev || !image_bytes || !layout_tag) return 1;
    *prepared_dev = L->prepared;
    *image_bytes = L->lay.bytes();
    *layout_tag = M26S_B1_LAYOUT_G950_V1;
    return 0;
}

void m26s_b1_layer_free(m26s_b1_layer* L) {
    if (!L) return;
    if (L->prepared) (void)hipFree(L->prepared);
    if (L->resident) (void)hipFree(L->resident);
    delete L;
}

int m26s_b1_scratch_new(m26s_b1_scratch** out, char* err, size_t errlen) {
    return scratch_build(nullptr, true, out, err, errlen);
}
int m26s_b1_scratch_new_on(void* hip_stream, m26s_b1_scratch** out, char* err, size_t errlen) {
    return scratch_build(static_cast<hipStream_t>(hip_stream), false, out, err, errlen);
}

void m26s_b1_scratch_free(m26s_b1_scratch* S) {
    if (!S) return;
    for (hipEvent_t ev : {S->e0, S->ep, S->ea, S->ec, S->e1})
        if (ev) (void)hipEventDestroy(ev);
    if (S->own_stream && S->st) (void)hipStreamDestroy(S->st);
    delete S;
}

int m26s_b1_ffn(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* payload, size_t payload_pitch,
                const uint8_t* scales, size_t scales_pitch, const int32_t* ids, const float* weights, uint32_t rows,
                uint16_t* bf16_out, float* ms, char* err, size_t errlen) {
    if (!L || !S || !rows || rows > kMaxRows || payload_pitch < 4096 || scales_pitch < 128 || !payload || !scales ||
        !ids || !weights || !bf16_out) {
        set_msg(err, errlen, "b1 ffn: bad rows/handles/pitch");
        return 1;
    }
    if (!layer_usable(L, err, errlen)) return 4;
    hipError_t e;
    const auto t0 = std::chrono::steady_clock::now();
    const uint64_t routes = uint64_t(rows) * kTopk;
    M26S_CK(S->x.ensure(size_t(rows) * 4096), "b1 x alloc");
    M26S_CK(S->xs.ensure(size_t(rows) * 128), "b1 xs alloc");
    M26S_CK(S->iw.ensure(routes * 8), "b1 ids/w alloc");
    M26S_CK(S->bf16.ensure(size_t(rows) * 4096 * 2), "b1 bf16 alloc");
    M26S_CK(hipMemcpy2DAsync(S->x.p, 4096, payload, payload_pitch, 4096, rows, hipMemcpyHostToDevice, S->st), "b1 x upload");
    M26S_CK(hipMemcpy2DAsync(S->xs.p, 128, scales, scales_pitch, 128, rows, hipMemcpyHostToDevice, S->st), "b1 xs upload");
    S->hiw.resize(routes * 8);  // ids then weights: one upload (b1_serve.cu:344-347)
    std::memcpy(S->hiw.data(), ids, routes * 4);
    std::memcpy(S->hiw.data() + routes * 4, weights, routes * 4);
    M26S_CK(hipMemcpyAsync(S->iw.p, S->hiw.data(), routes * 8, hipMemcpyHostToDevice, S->st), "b1 ids/w upload");
    const auto t1 = std::chrono::steady_clock::now();
    int rc = enqueue(L, S, S->x.as<uint8_t>(), 4096, S->xs.as<uint8_t>(), 128, S->iw.as<int32_t>(),
                     reinterpret_cast<const float*>(S->iw.as<uint8_t>() + routes * 4), rows, S->bf16.as<uint16_t>(),
                     nullptr, err, errlen);
    if (rc) return rc;
    M26S_CK(hipMemcpyAsync(bf16_out, S->bf16.p, size_t(rows) * 4096 * 2, hipMemcpyDeviceToHost, S->st), "b1 bf16 download");
    uint32_t m[kMetaWords] = {};
    rc = finish(S, m, err, errlen);
    const auto t2 = std::chrono::steady_clock::now();
    report(S, ms, std::chrono::duration<float, std::milli>(t1 - t0).count(),
           std::chrono::duration<float, std::milli>(t2 - t0).count(), m[kGroupCount]);
    return rc;
}

int m26s_b1_ffn_enqueue(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* payload_dev, size_t payload_pitch,
                        const uint8_t* scales_dev, size_t scales_pitch, const int32_t* ids_dev, const float* weights_dev,
                        uint32_t rows, uint16_t* bf16_out_dev, float* partial_dev, char* err, size_t errlen) {
    if (!L || !S || !rows || rows > kMaxRows || payload_pitch < 4096 || scales_pitch < 128 || !payload_dev ||
        !scales_dev || !ids_dev || !weights_dev || !bf16_out_dev || (reinterpret_cast<uintptr_t>(payload_dev) & 15) ||
        (payload_pitch & 15) || (reinterpret_cast<uintptr_t>(scales_dev) & 3) || (scales_pitch & 3)) {
        set_msg(err, errlen, "b1 ffn: bad rows/handles/pitch");
        return 1;
    }
    if (!layer_usable(L, err, errlen)) return 4;
    return enqueue(L, S, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev, rows, bf16_out_dev,
                   partial_dev, err, errlen);
}

int m26s_b1_scratch_sync(m26s_b1_scratch* S, char* err, size_t errlen) {
    if (!S) { set_msg(err, errlen, "b1 sync: bad handle"); return 1; }
    return finish(S, nullptr, err, errlen);
}

int m26s_b1_ffn_dev(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* payload_dev, size_t payload_pitch,
                    const uint8_t* scales_dev, size_t scales_pitch, const int32_t* ids_dev, const float* weights_dev,
                    uint32_t rows, uint16_t* bf16_out_dev, float* partial_dev, float* ms, char* err, size_t errlen) {
    const auto t0 = std::chrono::steady_clock::now();
    int rc = m26s_b1_ffn_enqueue(L, S, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev, rows,
                                 bf16_out_dev, partial_dev, err, errlen);
    if (rc) return rc;
    uint32_t m[kMetaWords] = {};
    rc = finish(S, m, err, errlen);
    const auto t2 = std::chrono::steady_clock::now();
    report(S, ms, 0.0f, std::chrono::duration<float, std::milli>(t2 - t0).count(), m[kGroupCount]);
    return rc;
}

int m26s_b1_plan_dev(const int32_t* ids_dev, const float* weights_dev, uint32_t rows, uint32_t capacity,
                     const uint8_t* resident_dev, int32_t* inverse_dev, int32_t* original_routes_dev,
                     float* grouped_weights_dev, void* groups_dev, uint32_t* group_count_dev, uint32_t* fault_dev,
                     char* err, size_t errlen) {
    if ((capacity != 256 && capacity != 2048 && capacity != 4096 && capacity != 8192) || rows > capacity ||
        !resident_dev || !inverse_dev || !original_routes_dev || !grouped_weights_dev || !groups_dev ||
        !group_count_dev || !fault_dev || (rows && (!ids_dev || !weights_dev))) {
        set_msg(err, errlen, "b1 plan: bad capacity/rows/pointers");
        return 1;
    }
    hipError_t e;
    Dev meta, chunks;
    M26S_CK(plan_lds_attr(), "b1 plan lds");
    M26S_CK(meta.ensure(kMetaWords * 4), "b1 plan meta alloc");
    M26S_CK(chunks.ensure(uint64_t(capacity) * kTopk * sizeof(Chunk)), "b1 plan chunks alloc");
    M26S_CK(hipMemset(meta.p, 0, kMetaWords * 4), "b1 plan meta clear");
    const PlanView pv{inverse_dev, original_routes_dev, grouped_weights_dev, static_cast<Group*>(groups_dev),
                      chunks.as<Chunk>(), meta.as<uint32_t>()};
    uint32_t m[kMetaWords];
    plan_kernel<<<1, kPlanThreads, uint64_t(rows) * kTopk, 0>>>(ids_dev, weights_dev, rows, resident_dev, pv, 1,
                                                                 capacity * kTopk, true);
    M26S_CK(hipGetLastError(), "b1 plan launch");
    M26S_CK(hipMemcpy(m, meta.p, sizeof m, hipMemcpyDeviceToHost), "b1 plan meta download");
    M26S_CK(hipMemcpy(fault_dev, &m[kPlanFault], 4, hipMemcpyHostToDevice), "b1 plan fault store");
    if (m[kPlanFault]) return 0;  // a rejected plan changes nothing but the fault word
    M26S_CK(hipMemcpy(group_count_dev, &m[kGroupCount], 4, hipMemcpyHostToDevice), "b1 plan count store");
    return 0;
}

int m26s_b1_quantize_dev(const float* h_dev, uint64_t elements, uint8_t* payload_dev, uint8_t* scales_dev,
                         uint32_t* faults_dev, char* err, size_t errlen) {
    if (elements % 32 || (elements && (!h_dev || !payload_dev || !scales_dev || !faults_dev))) {
        set_msg(err, errlen, "b1 quantize: bad extent/pointers");
        return 1;
    }
    if (!elements) return 0;
    hipError_t e;
    const uint64_t blocks = elements / 32, need = (blocks + 7) / 8;
    quantize_kernel<<<uint32_t(need < 65535 ? need : 65535), 256>>>(h_dev, blocks, payload_dev, scales_dev, faults_dev);
    M26S_CK(hipGetLastError(), "b1 quantize launch");
    M26S_CK(hipDeviceSynchronize(), "b1 quantize sync");
    return 0;
}

int m26s_b1_reduce_dev(const float* y_dev, const float* weights_dev, uint32_t rows, float* partial_dev,
                       uint16_t* bf16_dev, uint32_t* fault_dev, char* err, size_t errlen) {
    if (rows > kMaxRows || !fault_dev || (rows && (!y_dev || !weights_dev || !bf16_dev))) {
        set_msg(err, errlen, "b1 reduce: bad rows/pointers");
        return 1;
    }
    hipError_t e;
    M26S_CK(hipMemset(fault_dev, 0, 4), "b1 reduce fault clear");
    if (!rows) return 0;
    const uint64_t n4 = uint64_t(rows) * (kHidden / 4);
    reduce_kernel<<<uint32_t(n4 / 256 < 65536 ? (n4 + 255) / 256 : 65536), 256>>>(y_dev, weights_dev, rows, partial_dev,
                                                                                bf16_dev, fault_dev, nullptr);
    M26S_CK(hipGetLastError(), "b1 reduce launch");
    M26S_CK(hipDeviceSynchronize(), "b1 reduce sync");
    return 0;
}

void m26s_b1_scratch_set_stream(m26s_b1_scratch* S, int on) { if (S) S->stream_fc2 = on != 0; }
void m26s_b1_scratch_set_taps(m26s_b1_scratch* S, int on) { if (S) S->taps = on != 0; }

int m26s_b1_scratch_view(const m26s_b1_scratch* S, int which, void** dev_ptr, size_t* bytes) {
    if (!S || !dev_ptr || !bytes) return 1;
    const Dev* table[] = {&S->inv, &S->orig, &S->gw, &S->groups, &S->meta, &S->dq, &S->dqs, &S->y,
                          &S->tap_gate, &S->tap_up, &S->tap_h, &S->chunks};
    if (which < 0 || which >= int(sizeof table / sizeof table[0]) || !table[which]->p) return 1;
    *dev_ptr = table[which]->p;
    *bytes = table[which]->n;
    return 0;
}

int m26s_b1_copy_to_host(void* dst_host, const void* src_dev, size_t bytes) {
    return hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost) == hipSuccess ? 0 : 2;
}
int m26s_b1_copy_to_device(void* dst_dev, const void* src_host, size_t bytes) {
    return hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice) == hipSuccess ? 0 : 2;
}
void* m26s_b1_device_alloc(size_t bytes) {
    void* p = nullptr;
    return hipMalloc(&p, bytes ? bytes : 1) == hipSuccess ? p : nullptr;
}
void m26s_b1_device_free(void* dev_ptr) { if (dev_ptr) (void)hipFree(dev_ptr); }

}  // extern "C"
