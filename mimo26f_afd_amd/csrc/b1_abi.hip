// C ABI of the gfx950 routed-expert FFN: handles, the per-call workspace, launch schedule, fault decode.
// Keeps the contract of crates/mimo26-spark/kernels/b1_serve.cu:214-574 of the reference (names,
// argument meaning, return codes, the ms[8] phase report). What is behind it is this library's own:
// every per-call array is carved out of one grow-only slab by a layout function of (rows, intermediate),
// there is no host round trip between the planner and the GEMMs (grids are sized by capacity and idle
// workgroups leave on the device-side counts), the intermediate quantizer is fused into FC1, and a
// layer with exceptional weight scales runs the conforming arm of b1_conform.h.
#include <hip/hip_runtime.h>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/m26s_b1.h"
#include "b1_conform.h"
#include "b1_tile.h"

using namespace m26g;

namespace {

// ---- the error channel of one call ------------------------------------------------------------------
// The first failure of a call decides its return code and its message; `text` is the caller's buffer.
class Outcome {
public:
    Outcome(char* text, size_t room) : text_(text), room_(room) {}
    int fail(int rc, const char* fmt, ...) __attribute__((format(printf, 3, 4))) {
        if (text_ && room_) {
            va_list ap;
            va_start(ap, fmt);
            std::vsnprintf(text_, room_, fmt, ap);
            va_end(ap);
        }
        return rc;
    }
    // 0 when the runtime call succeeded, else return code 2 with "<step>: <runtime message>".
    int runtime(hipError_t e, const char* step) { return e == hipSuccess ? 0 : fail(2, "%s: %s", step, hipGetErrorString(e)); }

private:
    char* text_;
    size_t room_;
};
#define M26G_TRY(out, call, step)                         \
    do {                                                  \
        if (const int rc_ = (out).runtime((call), step)) return rc_; \
    } while (0)

// ---- sizes ---------------------------------------------------------------------------------------------
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

// ---- the workspace of one call --------------------------------------------------------------------------
// Everything a call needs beyond its inputs and outputs, as pointers into one slab. `Fixed` survives from
// call to call (the fault words accumulate until the next sync; the zero row and the unit scales are
// written once); the rest is per call and may move when the slab grows.
struct Fixed {
    uint32_t* meta;      // kMetaWords fault / count words; 64 bytes on, four 64-bit words of the tile launches' clock record
    uint8_t* zero_row;   // 8192 zero bytes: the activation row of a padded tile row
    uint8_t* unit_scales;  // 256 bytes of 127
};
constexpr size_t kFixedBytes = 256 + 8192 + 256;
__host__ __device__ inline Fixed fixed_at(uint8_t* base) {
    return Fixed{reinterpret_cast<uint32_t*>(base), base + 256, base + 256 + 8192};
}
__global__ void fixed_init_kernel(uint8_t* base) {  // a kernel, not a memset: a caller may be recording a graph
    for (uint32_t i = threadIdx.x; i < kFixedBytes; i += blockDim.x)  // meta word kQuantWhere starts at "no block"
        base[i] = i >= 256 + 8192 ? uint8_t(127) : (i / 4 == kQuantWhere ? uint8_t(0xff) : uint8_t(0));
}

__global__ void arm_plan_work_kernel(uint32_t* work) {
    if (threadIdx.x < 4) work[threadIdx.x] = 0xffffffffu;
}

struct Shape {
    uint32_t rows, inter;
    bool taps, host_io, conforming;
    bool fused;   // the combine runs inside FC2 (completion counts per token and 64 columns), not as a launch of its own
    bool y_bf16;  // per-route rows kept as BF16 bits
    bool guards;  // every array is followed (and the first preceded) by a red zone of 0xa5 bytes
};
constexpr int kMaxZones = 32;
constexpr uint8_t kGuardByte = 0xa5;
struct Zone { uint64_t at, bytes; };  // relative to the slab
struct Workspace {
    uint32_t* plan_work;  // the wide planner's histograms (its header word is armed when the slab moves)
    int32_t *inverse, *original;
    float* grouped_weights;
    Group* groups;
    Chunk* chunks;
    uint8_t *dq, *dqs;
    float* y;
    uint32_t* done;    // fused combine: [rows][64] completion counts
    uint8_t *xg, *dg;  // tile schedule: activation scales in MFMA lane order
    uint32_t* rowbad;
    int32_t *xrows, *yrows;
    float *tap_gate, *tap_up, *tap_h;
    uint8_t *x, *xs;  // host entry: staged inputs and output
    int32_t* ids;
    float* weights;
    uint16_t* bf16;
    size_t bytes[20];  // extents of the views m26s_b1_scratch_view hands out, by its `which`
    size_t total;
    uint32_t tiles, chunk_cap, group_cap;
    uint64_t routes, route_cap;
    Zone zone[kMaxZones];
    int zones;
};
constexpr size_t kPlanWorkBytes = wide_plan_words(kMaxRows * kTopk) * 4;

// Lays the per-call arrays out behind `base` (which may be null: then only the sizes are wanted).
Workspace carve(uint8_t* base, const Shape& s) {
    Workspace w{};
    size_t at = 0;
    auto zone = [&](size_t from, size_t upto) {
        if (w.zones < kMaxZones) w.zone[w.zones++] = Zone{from, upto - from};
    };
    if (s.guards) zone(0, at = 256);
    auto take = [&](size_t bytes) {
        uint8_t* p = base ? base + at : nullptr;
        const size_t end = at + ((bytes + 3) & ~size_t(3));
        at += (bytes + 255) & ~size_t(255);
        if (s.guards) zone(end, at += 256);  // from the array's last word to 256 bytes past its padded end
        return p;
    };
    w.tiles = tiles_for(s.rows);
    w.routes = uint64_t(s.rows) * kTopk;
    w.route_cap = uint64_t(capacity_class(s.rows)) * kTopk;
    w.group_cap = uint32_t(group_bound(w.routes));
    w.chunk_cap = uint32_t(chunk_bound(w.routes, w.tiles));
    const uint64_t I = s.inter, gcap = w.group_cap, ccap = w.chunk_cap;
    // The tile kernels ask for their chunk record, row table and row verdicts before they know whether the
    // chunk exists: those tables cover the whole grid (chunk capacity rounded up to runs on eight XCDs).
    const uint64_t grid_chunks = ccap + 8 * kTileRunMax;
    w.plan_work = reinterpret_cast<uint32_t*>(take(kPlanWorkBytes));
    w.inverse = reinterpret_cast<int32_t*>(take(w.bytes[0] = w.route_cap * 4));
    w.original = reinterpret_cast<int32_t*>(take(w.bytes[1] = w.route_cap * 4));
    w.grouped_weights = reinterpret_cast<float*>(take(w.bytes[2] = w.route_cap * 4));
    w.groups = reinterpret_cast<Group*>(take(w.bytes[3] = gcap * sizeof(Group)));
    w.chunks = reinterpret_cast<Chunk*>(take(w.bytes[11] = grid_chunks * sizeof(Chunk)));
    w.dq = take(w.bytes[5] = gcap * 16 * I);
    w.dqs = take(w.bytes[6] = gcap * 16 * I / 32);
    w.y = reinterpret_cast<float*>(take(w.bytes[7] = w.routes * kHidden * (s.y_bf16 ? 2 : 4)));
    if (s.fused) w.done = reinterpret_cast<uint32_t*>(take(size_t(s.rows) * kDoneBlocks * 4));
    if (w.tiles > 2 && !s.conforming) {
        w.xg = take(ccap * gathered_scale_bytes(kHidden));
        w.dg = take(ccap * gathered_scale_bytes(s.inter));
        w.rowbad = reinterpret_cast<uint32_t*>(take(grid_chunks * 16 * 4));
        w.xrows = reinterpret_cast<int32_t*>(take(grid_chunks * 128 * 4));
        w.yrows = reinterpret_cast<int32_t*>(take(ccap * 128 * 4));
    }
    if (s.taps) {
        w.tap_gate = reinterpret_cast<float*>(take(w.bytes[8] = gcap * 16 * I * 4));
        w.tap_up = reinterpret_cast<float*>(take(w.bytes[9] = gcap * 16 * I * 4));
        w.tap_h = reinterpret_cast<float*>(take(w.bytes[10] = gcap * 16 * I * 4));
    }
    if (s.host_io) {
        w.x = take(size_t(s.rows) * kHidden);
        w.xs = take(size_t(s.rows) * (kHidden / 32));
        w.ids = reinterpret_cast<int32_t*>(take(w.routes * 4));
        w.weights = reinterpret_cast<float*>(take(w.routes * 4));
        w.bf16 = reinterpret_cast<uint16_t*>(take(size_t(s.rows) * kHidden * 2));
    }
    w.total = at;
    return w;
}

// Red zones (test aid): filled before every call when the scratch asks for them, read back by
// m26s_b1_scratch_check_guards. The counterpart of the reference's guarded test buffers
// (crates/mimo26-expert/tests/b1_core/primitive.cu:23-40).
struct ZoneTable { Zone zone[kMaxZones]; int zones; };
__global__ void fill_zones_kernel(uint8_t* base, ZoneTable t) {
    if (int(blockIdx.x) >= t.zones) return;
    const Zone z = t.zone[blockIdx.x];
    for (uint64_t i = threadIdx.x; i < z.bytes; i += blockDim.x) base[z.at + i] = kGuardByte;
}

// Kernels whose dynamic LDS passes 64 KB need the limit raised once per process.
std::atomic<bool> lds_ready{false};  // idempotent: threads that race set the same attributes
using TileS = PrefillTile;
hipError_t raise_lds_limits() {
    if (lds_ready) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(plan_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(kMaxRows * kTopk));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fc1_tile_kernel<TileS>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(TileS::kLdsBytes));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fc2_tile_kernel<TileS, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(TileS::kLdsBytes));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(fc2_tile_kernel<TileS, true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, int(TileS::kLdsBytes));
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
    hipStream_t stream = nullptr;
    bool own_stream = false;
    hipEvent_t begun = nullptr, planned = nullptr, fc1_done = nullptr, fc2_done = nullptr, ended = nullptr;
    uint8_t* fixed = nullptr;  // kFixedBytes
    uint8_t* slab = nullptr;
    size_t slab_bytes = 0;
    Workspace last{};  // of the latest call, for the views
    bool taps = false, fused_combine = false, y_bf16 = false, guards = false, scope_timing = false;
    uint32_t last_rows = 0;
    uint8_t* bounce = nullptr;  // page-locked host staging for callers whose own arrays are pageable
    size_t bounce_bytes = 0;
};

namespace {

// The slab only grows. Growing it frees the old one, which waits for the device: calls still in flight on it finish first.
int fit_slab(m26s_b1_scratch* S, size_t bytes, bool& grew, Outcome& out) {
    grew = false;
    if (bytes <= S->slab_bytes) return 0;
    if (S->slab) (void)hipFree(S->slab);
    S->slab = nullptr;
    S->slab_bytes = 0;
    M26G_TRY(out, hipMalloc(reinterpret_cast<void**>(&S->slab), bytes), "b1 workspace alloc");
    S->slab_bytes = bytes;
    grew = true;
    return 0;
}

Shape shape_of(const m26s_b1_layer* L, const m26s_b1_scratch* S, uint32_t rows, bool host_io) {
    const bool conforming = !L->all_normal;
    return Shape{rows, L->lay.inter, S->taps, host_io, conforming, S->fused_combine && !conforming, S->y_bf16, S->guards};
}

// Sizes the slab for the call and lays the call's arrays out in it (S->last).
int ready_workspace(m26s_b1_scratch* S, const Shape& shape, Outcome& out) {
    bool grew = false;
    if (const int rc = fit_slab(S, carve(nullptr, shape).total, grew, out)) return rc;
    S->last = carve(S->slab, shape);
    if (grew) {
        // The wide planner's first word is its fault key, armed to "none"; its scan re-arms it after every call.
        // A kernel, not a memset: the stream may be the caller's, and the caller may be recording a graph.
        arm_plan_work_kernel<<<1, 64, 0, S->stream>>>(S->last.plan_work);
        M26G_TRY(out, hipGetLastError(), "b1 workspace arm");
    }
    return 0;
}

int layer_build(const Canonical& c, uint32_t inter, m26s_b1_layer** made, Outcome& out) {
    auto* L = new (std::nothrow) m26s_b1_layer();
    if (!L) return out.fail(2, "b1 layer: host allocation failed");
    L->lay.inter = inter;
    uint32_t* flag = nullptr;
    uint32_t abnormal = 1;
    const std::vector<uint8_t> present(kExperts, 1);  // expert id == slot: every expert of the pool is resident
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&L->prepared), L->lay.bytes() * kExperts);
    const char* step = "b1 layer prepared alloc";
    if (e == hipSuccess) { step = "b1 layer metadata"; e = hipMalloc(reinterpret_cast<void**>(&L->resident), kExperts); }
    if (e == hipSuccess) e = hipMemcpy(L->resident, present.data(), kExperts, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&flag), 4);
    if (e == hipSuccess) e = hipMemset(flag, 0, 4);
    if (e == hipSuccess) {
        step = "b1 prepare";
        prepare_kernel<<<dim3(inter / 8, kExperts), 256>>>(c, L->prepared, L->lay, flag);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpy(&abnormal, flag, 4, hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (flag) (void)hipFree(flag);
    if (e != hipSuccess) {
        m26s_b1_layer_free(L);
        return out.runtime(e, step);
    }
    L->all_normal = abnormal == 0;
    *made = L;
    return 0;
}

int scratch_build(hipStream_t stream, bool own, m26s_b1_scratch** made, Outcome& out) {
    if (!made) return out.fail(1, "b1 scratch: null out");
    auto* S = new (std::nothrow) m26s_b1_scratch();
    if (!S) return out.fail(1, "b1 scratch: host allocation failed");
    S->stream = stream;
    S->own_stream = own;
    // The reference's opt-in switch for BF16 per-route rows (crates/mimo26-spark/kernels/b1_serve.cu:402-405).
    const char* y_mode = std::getenv("MIMO26_B1_Y");
    S->y_bf16 = y_mode && std::strcmp(y_mode, "bf16") == 0;
    hipError_t e = own ? hipStreamCreateWithFlags(&S->stream, hipStreamNonBlocking) : hipSuccess;
    for (hipEvent_t* ev : {&S->begun, &S->planned, &S->fc1_done, &S->fc2_done, &S->ended})
        if (e == hipSuccess) e = hipEventCreate(ev);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&S->fixed), kFixedBytes);
    if (e == hipSuccess) e = raise_lds_limits();
    if (e == hipSuccess) {
        fixed_init_kernel<<<1, 256, 0, S->stream>>>(S->fixed);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(S->stream);
    if (e != hipSuccess) {
        m26s_b1_scratch_free(S);
        return out.fail(1, "b1 scratch stream/events: %s", hipGetErrorString(e));
    }
    *made = S;
    return 0;
}

// What one call launches on, whoever owns the memory: the scratch handle's slab or the static workspace.
struct Launch {
    hipStream_t stream;
    Fixed fixed;
    Workspace ws;
    bool taps, y_bf16;
    hipEvent_t planned, fc1_done, fc2_done;  // null: not timed
};

void mark(hipEvent_t ev, hipStream_t st) { if (ev) (void)hipEventRecord(ev, st); }

PlanView plan_view(const Launch& k) {
    return PlanView{k.ws.inverse, k.ws.original, k.ws.grouped_weights, k.ws.groups, k.ws.chunks, k.fixed.meta, k.ws.done};
}

Fc1Args fc1_args(const m26s_b1_layer* L, const Launch& k, const uint8_t* x, size_t xp, const uint8_t* xs, size_t xsp) {
    return Fc1Args{L->prepared, L->lay, plan_view(k), x, xp, xs, xsp, k.fixed.zero_row, k.fixed.unit_scales, k.ws.dq, k.ws.dqs,
                   k.taps ? k.ws.tap_gate : nullptr, k.taps ? k.ws.tap_up : nullptr, k.taps ? k.ws.tap_h : nullptr,
                   k.ws.xg, k.ws.rowbad, k.ws.xrows, k.ws.dg, reinterpret_cast<unsigned long long*>(k.fixed.meta + 16)};
}
Fc2Args fc2_args(const m26s_b1_layer* L, const Launch& k, const float* w, uint16_t* bf16_out, float* partial) {
    return Fc2Args{L->prepared, L->lay, plan_view(k), k.ws.dq, k.ws.dqs, k.fixed.zero_row, k.fixed.unit_scales, k.ws.y,
                   uint32_t(k.ws.routes), k.ws.dg, k.ws.yrows, k.ws.rowbad, reinterpret_cast<unsigned long long*>(k.fixed.meta + 16),
                   w, bf16_out, partial, k.y_bf16};
}

// Decode-size calls: every wave streams its own weight block from HBM, activations from L2.
// The waves of these kernels share nothing, so the workgroup is only the unit the dispatcher hands out. Below
// 32 tokens a launch is a round or two of workgroups, and one-wave workgroups fill the compute units evenly
// where four-wave ones leave the last round part empty (per call, one wave against four: 8 tokens 58.7 / 64.2 us,
// 16 tokens 95.6 / 102.4, 24 tokens 130 / 134; one expert's 16 rows at a rank's share 36.8 / 41.6). At 32 tokens
// the two are within 1 % of each other either way (full intermediate 168 / 171, 256 experts of a rank's share with
// one row each 136.2 / 135.1), and from 96 tokens on the four-wave form is the faster by half a percent.
constexpr uint64_t kNarrowRoutes = 32 * kTopk;
template <int NT>
void launch_direct(const m26s_b1_layer* L, const Launch& k, const Fc1Args& f1, const Fc2Args& f2) {
    const uint32_t waves = k.ws.routes < kNarrowRoutes ? 1 : 4;
    fc1_kernel<NT><<<dim3(L->lay.inter / (32 * waves), k.ws.chunk_cap), 64 * waves, 0, k.stream>>>(f1);
    mark(k.fc1_done, k.stream);
    fc2_kernel<NT><<<dim3(kHidden / (64 * waves), k.ws.chunk_cap), 64 * waves, 0, k.stream>>>(f2);
    mark(k.fc2_done, k.stream);
}
// Prefill-size calls: workgroups that share each chunk's activation tiles through LDS, one of eight waves per compute unit.
void launch_tiles(const m26s_b1_layer* L, const Launch& k, const Fc1Args& f1, const Fc2Args& f2) {
    gather_scales_kernel<<<k.ws.chunk_cap, 256, 0, k.stream>>>(f1.plan, f1.xs, f1.xs_pitch, reinterpret_cast<uint32_t*>(k.ws.xg),
                                                              k.ws.rowbad, k.ws.xrows, k.ws.yrows);
    fc1_tile_kernel<TileS><<<tile_grid(L->lay.inter / (32 * TileS::kWaves), k.ws.chunk_cap, kFc1Run), TileS::kThreads, TileS::kLdsBytes, k.stream>>>(f1);
    mark(k.fc1_done, k.stream);
    const dim3 grid2(tile_grid(kHidden / (64 * TileS::kWaves), k.ws.chunk_cap, kFc2Run));
    if (L->lay.inter == kRankI) fc2_tile_kernel<TileS, true><<<grid2, TileS::kThreads, TileS::kLdsBytes, k.stream>>>(f2);
    else fc2_tile_kernel<TileS, false><<<grid2, TileS::kThreads, TileS::kLdsBytes, k.stream>>>(f2);
    mark(k.fc2_done, k.stream);
}
// Layers with exceptional weight scales: decode-then-multiply, group by group.
void launch_conforming(const m26s_b1_layer* L, const Launch& k, const Fc1Args& f1, const Fc2Args& f2) {
    fc1_conform_kernel<<<dim3(L->lay.inter / kConformColumns, k.ws.group_cap), kConformColumns, 0, k.stream>>>(f1);
    mark(k.fc1_done, k.stream);
    fc2_conform_kernel<<<dim3(kHidden / kConformColumns, k.ws.group_cap), kConformColumns, 0, k.stream>>>(f2);
    mark(k.fc2_done, k.stream);
}

// plan -> FC1 (+ quantizer) -> FC2 -> combine on device-resident inputs. Launches only.
hipError_t launch_ffn(const m26s_b1_layer* L, const Launch& k, const uint8_t* x, size_t xp, const uint8_t* xs, size_t xsp,
                      const int32_t* ids, const float* w, uint32_t rows, uint16_t* bf16_out, float* partial) {
    const PlanView pv = plan_view(k);
    const uint32_t nt = k.ws.tiles, routes = uint32_t(k.ws.routes);
    if (rows > kWidePlanFrom) {  // several compute units share the scatter (b1_kernels.h, "Stage 1 for large calls")
        const uint32_t wide = wide_plan_groups(routes);
        plan_count_kernel<<<wide, kPlanThreads, 0, k.stream>>>(ids, w, rows, L->resident, k.ws.plan_work, k.ws.done);
        plan_scan_kernel<<<1, kPlanThreads, 0, k.stream>>>(routes, k.ws.plan_work, pv, nt);
        plan_place_kernel<<<wide, kPlanThreads, 0, k.stream>>>(ids, w, rows, k.ws.plan_work, pv, k.taps);
    } else {
        plan_kernel<<<1, kPlanThreads, routes, k.stream>>>(ids, w, rows, L->resident, pv, nt, 0, k.taps);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    mark(k.planned, k.stream);
    const Fc1Args f1 = fc1_args(L, k, x, xp, xs, xsp);
    const Fc2Args f2 = fc2_args(L, k, w, bf16_out, partial);
    if (!L->all_normal) launch_conforming(L, k, f1, f2);
    else if (nt == 1) launch_direct<1>(L, k, f1, f2);
    else if (nt == 2) launch_direct<2>(L, k, f1, f2);
    else launch_tiles(L, k, f1, f2);
    if ((e = hipGetLastError()) != hipSuccess || k.ws.done) return e;  // with completion counts FC2 has summed the rows itself
    const uint64_t n4 = uint64_t(rows) * (kHidden / 4);
    const uint32_t blocks = uint32_t(n4 / 256 < 65536 ? (n4 + 255) / 256 : 65536);
    if (k.y_bf16) reduce_kernel<true><<<blocks, 256, 0, k.stream>>>(k.ws.y, w, rows, partial, bf16_out, k.fixed.meta + kReduceFault, k.fixed.meta);
    else reduce_kernel<false><<<blocks, 256, 0, k.stream>>>(k.ws.y, w, rows, partial, bf16_out, k.fixed.meta + kReduceFault, k.fixed.meta);
    return hipGetLastError();
}

// Sizes the scratch for the call, then launches it. Faults of all calls since the last sync accumulate in the meta words.
// `timed` brackets the call and its stages with the scratch's events (for the ms[8] report); an untimed call puts
// nothing but its kernels on the stream: every event is one more packet the GPU's front end works through between two kernels.
int enqueue(const m26s_b1_layer* L, m26s_b1_scratch* S, bool host_io, bool timed, const uint8_t* x, size_t xp, const uint8_t* xs,
            size_t xsp, const int32_t* ids, const float* w, uint32_t rows, uint16_t* bf16_out, float* partial, Outcome& out) {
    if (const int rc = ready_workspace(S, shape_of(L, S, rows, host_io), out)) return rc;
    S->last_rows = rows;
    if (S->guards) {
        ZoneTable t{};
        t.zones = S->last.zones;
        std::memcpy(t.zone, S->last.zone, sizeof t.zone);
        fill_zones_kernel<<<kMaxZones, 256, 0, S->stream>>>(S->slab, t);
        M26G_TRY(out, hipGetLastError(), "b1 red zones");
    }
    const Launch k{S->stream, fixed_at(S->fixed), S->last, S->taps, S->y_bf16, timed ? S->planned : nullptr,
                   timed && !S->scope_timing ? S->fc1_done : nullptr, timed ? S->fc2_done : nullptr};
    if (host_io) {  // the inputs were staged into the slab by the caller of this function
        x = S->last.x, xp = kHidden, xs = S->last.xs, xsp = kHidden / 32, ids = S->last.ids, w = S->last.weights;
        bf16_out = S->last.bf16;
    }
    if (timed) M26G_TRY(out, hipEventRecord(S->begun, S->stream), "b1 event");
    M26G_TRY(out, launch_ffn(L, k, x, xp, xs, xsp, ids, w, rows, bf16_out, partial), "b1 launch");
    if (timed) M26G_TRY(out, hipEventRecord(S->ended, S->stream), "b1 event");
    return 0;
}

// Wait, read the meta words, translate them (b1_serve.cu:365-368, 551-562) and clear them.
int finish(m26s_b1_scratch* S, uint32_t* meta_out, Outcome& out) {
    uint32_t m[kMetaWords];
    M26G_TRY(out, hipMemcpyAsync(m, S->fixed, sizeof m, hipMemcpyDeviceToHost, S->stream), "b1 meta download");
    M26G_TRY(out, hipStreamSynchronize(S->stream), "b1 compute sync");
    meta_reset_kernel<<<1, 64, 0, S->stream>>>(reinterpret_cast<uint32_t*>(S->fixed));
    M26G_TRY(out, hipGetLastError(), "b1 meta reset");
    if (meta_out) std::memcpy(meta_out, m, sizeof m);
    const bool called = S->last_rows != 0;  // a sync with nothing enqueued since the last one has nothing to report
    S->last_rows = 0;
    if (m[kPlanFault]) return out.fail(3, "b1 plan: invalid routes (id/residency/weight/duplicate)");
    if (called && !m[kGroupCount]) return out.fail(3, "b1 plan: bad group count");
    if (m[kFc1Fault]) return out.fail(4, "b1 fc1 fault %u (groups %u)", m[kFc1Fault], m[kGroupCount]);
    if (m[kQuantFault])
        return out.fail(4, "b1 quantizer fault %u at word %u (groups %u)", m[kQuantFault] & 1 ? 1u : 2u, m[kQuantWhere], m[kGroupCount]);
    if (m[kFc2Fault]) return out.fail(4, "b1 fc2 fault %u (groups %u)", m[kFc2Fault], m[kGroupCount]);
    if (m[kReduceFault]) return out.fail(4, "b1 reduce fault %u (groups %u)", m[kReduceFault], m[kGroupCount]);
    return 0;
}

// True for host memory the runtime knows as page-locked (hipHostMalloc or registered). Asking about a
// pageable pointer is an error to the runtime, which it would otherwise report at the next call: cleared here.
bool page_locked(const void* p) {
    hipPointerAttribute_t attr{};
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return attr.type == hipMemoryTypeHost;
}

using Clock = std::chrono::steady_clock;
float ms_between(Clock::time_point a, Clock::time_point b) { return std::chrono::duration<float, std::milli>(b - a).count(); }

// ms[8]: upload + plan, GPU compute, tail, group count, FC1 (with the fused quantizer), 0, FC2, combine.
void report(m26s_b1_scratch* S, float* ms, float host_front, float host_total, uint32_t groups) {
    if (!ms) return;
    float plan = 0, gpu = 0, fc1 = 0, fc2 = 0, combine = 0;
    (void)hipEventElapsedTime(&plan, S->begun, S->planned);
    (void)hipEventElapsedTime(&gpu, S->planned, S->ended);
    if (S->scope_timing) {  // one interval over both GEMM stages, no event between them
        (void)hipEventElapsedTime(&fc1, S->planned, S->fc2_done);
    } else {
        (void)hipEventElapsedTime(&fc1, S->planned, S->fc1_done);
        (void)hipEventElapsedTime(&fc2, S->fc1_done, S->fc2_done);
    }
    (void)hipEventElapsedTime(&combine, S->fc2_done, S->ended);
    const float tail = host_total - host_front - plan - gpu;
    const float v[8] = {host_front + plan, gpu, tail < 0 ? 0 : tail, float(groups), fc1, 0.0f, fc2, combine};
    std::memcpy(ms, v, sizeof v);
}

bool bad_call(const void* L, const void* S, uint32_t rows, size_t pp, size_t sp, const void* a, const void* b, const void* c,
              const void* d, const void* e) {
    return !L || !S || !rows || rows > kMaxRows || pp < kHidden || sp < kHidden / 32 || !a || !b || !c || !d || !e;
}

}  // namespace

// ---- a call that allocates nothing -----------------------------------------------------------------------
// The workspace of m26s_b1_ffn_static: a fixed array in the library's own device image, so that the call
// needs no allocation at all. Each GPU the library runs on holds its own copy at its own address from the
// moment the code object is loaded there until the process ends.
constexpr uint32_t kStaticRows = 128;            // the decode / verify batch of the benchmark configurations
constexpr size_t kStaticBytes = size_t(32) << 20;
static __device__ __align__(256) uint8_t scratch[kStaticBytes];

namespace {
constexpr int kStaticDevices = 64;
// The array's device address per GPU (the symbol itself is no address on the host). Threads that race on a
// GPU's first call look the same address up and store the same value.
std::atomic<uint8_t*> static_base[kStaticDevices];
// First kernel of every call on the static workspace: the count and fault words start from zero and the 256
// unit scale bytes are written again, so the array needs no one-time initialisation that a graph capture could
// swallow or another stream could overtake. The zero row is never written: the array starts as zeros when the
// code object is loaded.
__global__ void static_begin_kernel(uint8_t* base) {
    const Fixed f = fixed_at(base);
    if (threadIdx.x < kMetaWords) f.meta[threadIdx.x] = threadIdx.x == kQuantWhere ? 0xffffffffu : 0u;
    reinterpret_cast<uint32_t*>(f.unit_scales)[threadIdx.x] = 0x7f7f7f7fu;
}
__global__ void status_copy_kernel(uint32_t* __restrict__ out, const uint32_t* __restrict__ meta) {
    if (threadIdx.x < kMetaWords) out[threadIdx.x] = meta[threadIdx.x];
}
}  // namespace

extern "C" {

int m26s_b1_layer_new(const uint8_t* canonical_dev, uint64_t canonical_bytes, uint32_t rank, m26s_b1_layer** made,
                      char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (!canonical_dev || canonical_bytes != uint64_t(kExperts) * kImageBytes || rank >= 4 || !made)
        return out.fail(1, "b1 layer: bad canonical extent/rank");
    return layer_build(Canonical{{canonical_dev, nullptr, nullptr, nullptr}, 1}, kRankI, made, out);
}

int m26s_b1_layer_new_full(const uint8_t* const rank_images_dev[4], uint64_t bytes_each, m26s_b1_layer** made, char* err,
                           size_t errlen) {
    Outcome out(err, errlen);
    if (!rank_images_dev || !made || bytes_each != uint64_t(kExperts) * kImageBytes || !rank_images_dev[0] ||
        !rank_images_dev[1] || !rank_images_dev[2] || !rank_images_dev[3])
        return out.fail(1, "b1 layer: bad canonical extent/rank");
    return layer_build(Canonical{{rank_images_dev[0], rank_images_dev[1], rank_images_dev[2], rank_images_dev[3]}, 4},
                       4 * kRankI, made, out);
}

int m26s_b1_layer_all_normal(const m26s_b1_layer* L) { return L && L->all_normal ? 1 : 0; }
uint32_t m26s_b1_layer_intermediate(const m26s_b1_layer* L) { return L ? L->lay.inter : 0; }

int m26s_b1_layer_view(const m26s_b1_layer* L, const uint8_t** prepared_dev, uint64_t* image_bytes, uint32_t* layout_tag) {
    if (!L || !prepared_dev || !image_bytes || !layout_tag) return 1;
    *prepared_dev = L->prepared;
    *image_bytes = L->lay.bytes();
    *layout_tag = M26S_B1_LAYOUT_G950_V2;
    return 0;
}

void m26s_b1_layer_free(m26s_b1_layer* L) {
    if (!L) return;
    if (L->prepared) (void)hipFree(L->prepared);
    if (L->resident) (void)hipFree(L->resident);
    delete L;
}

int m26s_b1_scratch_new(m26s_b1_scratch** made, char* err, size_t errlen) {
    Outcome out(err, errlen);
    return scratch_build(nullptr, true, made, out);
}
int m26s_b1_scratch_new_on(void* hip_stream, m26s_b1_scratch** made, char* err, size_t errlen) {
    Outcome out(err, errlen);
    return scratch_build(static_cast<hipStream_t>(hip_stream), false, made, out);
}
void* m26s_b1_scratch_stream(const m26s_b1_scratch* S) { return S ? static_cast<void*>(S->stream) : nullptr; }

void m26s_b1_scratch_free(m26s_b1_scratch* S) {
    if (!S) return;
    for (hipEvent_t ev : {S->begun, S->planned, S->fc1_done, S->fc2_done, S->ended})
        if (ev) (void)hipEventDestroy(ev);
    if (S->slab) (void)hipFree(S->slab);
    if (S->fixed) (void)hipFree(S->fixed);
    if (S->bounce) (void)hipHostFree(S->bounce);
    if (S->own_stream && S->stream) (void)hipStreamDestroy(S->stream);
    delete S;
}

int m26s_b1_ffn(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* payload, size_t payload_pitch,
                const uint8_t* scales, size_t scales_pitch, const int32_t* ids, const float* weights, uint32_t rows,
                uint16_t* bf16_out, float* ms, char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (bad_call(L, S, rows, payload_pitch, scales_pitch, payload, scales, ids, weights, bf16_out))
        return out.fail(1, "b1 ffn: bad rows/handles/pitch");
    const auto t0 = Clock::now();
    // Stage the caller's host arrays into the slab: rows packed to 4096 / 128 bytes, ids and weights as they are.
    if (const int rc = ready_workspace(S, shape_of(L, S, rows, true), out)) return rc;
    const Workspace ws = S->last;
    const size_t routes = size_t(rows) * kTopk, out_bytes = size_t(rows) * kHidden * 2;
    // The reference's daemon hands over page-locked arrays (its registered receive ring and send slot) and those
    // are copied from and to directly. Pageable arrays go through a page-locked bounce buffer of the scratch:
    // left to the runtime, such copies are staged a piece at a time with a wait after each (2.9 against 0.6 ms
    // for a 128-row call, 158 against 7.7 ms for 8192 rows).
    const bool direct = page_locked(payload) && page_locked(scales) && page_locked(bf16_out);
    // The staged inputs lie in one run of the slab (rows, scales, ids, weights, each from a 256-byte boundary): the bounce
    // buffer mirrors that run, so one copy uploads all four.
    const size_t at_xs = size_t(ws.xs - ws.x), at_ids = size_t(reinterpret_cast<uint8_t*>(ws.ids) - ws.x),
                 at_w = size_t(reinterpret_cast<uint8_t*>(ws.weights) - ws.x), in_bytes = at_w + routes * 4;
    uint8_t* hx = nullptr;
    if (!direct) {
        const size_t need = in_bytes + out_bytes;
        if (need > S->bounce_bytes) {
            if (S->bounce) (void)hipHostFree(S->bounce);
            S->bounce = nullptr;
            S->bounce_bytes = 0;
            M26G_TRY(out, hipHostMalloc(reinterpret_cast<void**>(&S->bounce), need, hipHostMallocDefault), "b1 host staging alloc");
            S->bounce_bytes = need;
        }
        hx = S->bounce;
        for (uint32_t r = 0; r < rows; ++r) {
            std::memcpy(hx + size_t(r) * kHidden, payload + size_t(r) * payload_pitch, kHidden);
            std::memcpy(hx + at_xs + size_t(r) * (kHidden / 32), scales + size_t(r) * scales_pitch, kHidden / 32);
        }
        std::memcpy(hx + at_ids, ids, routes * 4);
        std::memcpy(hx + at_w, weights, routes * 4);
        M26G_TRY(out, hipMemcpyAsync(ws.x, hx, in_bytes, hipMemcpyHostToDevice, S->stream), "b1 input upload");
    } else {
        M26G_TRY(out, hipMemcpy2DAsync(ws.x, kHidden, payload, payload_pitch, kHidden, rows, hipMemcpyHostToDevice, S->stream), "b1 x upload");
        M26G_TRY(out, hipMemcpy2DAsync(ws.xs, kHidden / 32, scales, scales_pitch, kHidden / 32, rows, hipMemcpyHostToDevice, S->stream), "b1 xs upload");
        M26G_TRY(out, hipMemcpyAsync(ws.ids, ids, routes * 4, hipMemcpyHostToDevice, S->stream), "b1 ids upload");
        M26G_TRY(out, hipMemcpyAsync(ws.weights, weights, routes * 4, hipMemcpyHostToDevice, S->stream), "b1 weights upload");
    }
    const auto t1 = Clock::now();
    if (const int rc = enqueue(L, S, true, ms != nullptr, nullptr, 0, nullptr, 0, nullptr, nullptr, rows, nullptr, nullptr, out)) return rc;
    uint16_t* landing = direct ? bf16_out : reinterpret_cast<uint16_t*>(hx + in_bytes);
    M26G_TRY(out, hipMemcpyAsync(landing, S->last.bf16, out_bytes, hipMemcpyDeviceToHost, S->stream), "b1 bf16 download");
    uint32_t m[kMetaWords] = {};
    const int rc = finish(S, m, out);
    if (!direct && rc == 0) std::memcpy(bf16_out, landing, out_bytes);
    report(S, ms, ms_between(t0, t1), ms_between(t0, Clock::now()), m[kGroupCount]);
    return rc;
}

}  // extern "C"

namespace {
// The device-pointer call: argument checks, then the launches.
int enqueue_dev(const m26s_b1_layer* L, m26s_b1_scratch* S, bool timed, const uint8_t* payload_dev, size_t payload_pitch,
                const uint8_t* scales_dev, size_t scales_pitch, const int32_t* ids_dev, const float* weights_dev, uint32_t rows,
                uint16_t* bf16_out_dev, float* partial_dev, Outcome& out) {
    if (bad_call(L, S, rows, payload_pitch, scales_pitch, payload_dev, scales_dev, ids_dev, weights_dev, bf16_out_dev) ||
        (reinterpret_cast<uintptr_t>(payload_dev) & 15) || (payload_pitch & 15) ||
        (reinterpret_cast<uintptr_t>(scales_dev) & 3) || (scales_pitch & 3))
        return out.fail(1, "b1 ffn: bad rows/handles/pitch");
    return enqueue(L, S, false, timed, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev, rows,
                   bf16_out_dev, partial_dev, out);
}
}  // namespace

extern "C" {

int m26s_b1_ffn_enqueue(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* payload_dev, size_t payload_pitch,
                        const uint8_t* scales_dev, size_t scales_pitch, const int32_t* ids_dev, const float* weights_dev,
                        uint32_t rows, uint16_t* bf16_out_dev, float* partial_dev, char* err, size_t errlen) {
    Outcome out(err, errlen);
    return enqueue_dev(L, S, false, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev, rows,
                       bf16_out_dev, partial_dev, out);
}

int m26s_b1_scratch_sync(m26s_b1_scratch* S, char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (!S) return out.fail(1, "b1 sync: bad handle");
    return finish(S, nullptr, out);
}

int m26s_b1_ffn_dev(const m26s_b1_layer* L, m26s_b1_scratch* S, const uint8_t* payload_dev, size_t payload_pitch,
                    const uint8_t* scales_dev, size_t scales_pitch, const int32_t* ids_dev, const float* weights_dev,
                    uint32_t rows, uint16_t* bf16_out_dev, float* partial_dev, float* ms, char* err, size_t errlen) {
    const auto t0 = Clock::now();
    Outcome out(err, errlen);
    int rc = enqueue_dev(L, S, ms != nullptr, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev, rows,
                         bf16_out_dev, partial_dev, out);
    if (rc) return rc;
    uint32_t m[kMetaWords] = {};
    rc = finish(S, m, out);
    report(S, ms, 0.0f, ms_between(t0, Clock::now()), m[kGroupCount]);
    return rc;
}

int m26s_b1_plan_dev(const int32_t* ids_dev, const float* weights_dev, uint32_t rows, uint32_t capacity,
                     const uint8_t* resident_dev, int32_t* inverse_dev, int32_t* original_routes_dev,
                     float* grouped_weights_dev, void* groups_dev, uint32_t* group_count_dev, uint32_t* fault_dev,
                     char* err, size_t errlen) {
    Outcome out(err, errlen);
    if ((capacity != 256 && capacity != 2048 && capacity != 4096 && capacity != 8192) || rows > capacity ||
        !resident_dev || !inverse_dev || !original_routes_dev || !grouped_weights_dev || !groups_dev ||
        !group_count_dev || !fault_dev || (rows && (!ids_dev || !weights_dev)))
        return out.fail(1, "b1 plan: bad capacity/rows/pointers");
    // One allocation: the meta words, then the chunk table the planner also fills.
    uint8_t* work = nullptr;
    M26G_TRY(out, raise_lds_limits(), "b1 plan lds");
    M26G_TRY(out, hipMalloc(reinterpret_cast<void**>(&work), 256 + uint64_t(capacity) * kTopk * sizeof(Chunk)), "b1 plan work alloc");
    uint32_t m[kMetaWords] = {};
    hipError_t e = hipMemset(work, 0, 256);
    if (e == hipSuccess) {
        const PlanView pv{inverse_dev, original_routes_dev, grouped_weights_dev, static_cast<Group*>(groups_dev),
                          reinterpret_cast<Chunk*>(work + 256), reinterpret_cast<uint32_t*>(work), nullptr};
        plan_kernel<<<1, kPlanThreads, uint64_t(rows) * kTopk, 0>>>(ids_dev, weights_dev, rows, resident_dev, pv, 1,
                                                                     capacity * kTopk, true);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpy(m, work, sizeof m, hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemcpy(fault_dev, &m[kPlanFault], 4, hipMemcpyHostToDevice);
    // A rejected plan changes nothing but the fault word.
    if (e == hipSuccess && !m[kPlanFault]) e = hipMemcpy(group_count_dev, &m[kGroupCount], 4, hipMemcpyHostToDevice);
    (void)hipFree(work);
    return out.runtime(e, "b1 plan");
}

int m26s_b1_quantize_dev(const float* h_dev, uint64_t elements, uint8_t* payload_dev, uint8_t* scales_dev,
                         uint32_t* faults_dev, char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (elements % 32 || (elements && (!h_dev || !payload_dev || !scales_dev || !faults_dev)))
        return out.fail(1, "b1 quantize: bad extent/pointers");
    if (!elements) return 0;
    const uint64_t blocks = elements / 32, need = (blocks + 7) / 8;
    quantize_kernel<<<uint32_t(need < 65535 ? need : 65535), 256>>>(h_dev, blocks, payload_dev, scales_dev, faults_dev);
    M26G_TRY(out, hipGetLastError(), "b1 quantize launch");
    M26G_TRY(out, hipDeviceSynchronize(), "b1 quantize sync");
    return 0;
}

int m26s_b1_reduce_dev(const float* y_dev, const float* weights_dev, uint32_t rows, float* partial_dev,
                       uint16_t* bf16_dev, uint32_t* fault_dev, char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (rows > kMaxRows || !fault_dev || (rows && (!y_dev || !weights_dev || !bf16_dev)))
        return out.fail(1, "b1 reduce: bad rows/pointers");
    M26G_TRY(out, hipMemset(fault_dev, 0, 4), "b1 reduce fault clear");
    if (!rows) return 0;
    const uint64_t n4 = uint64_t(rows) * (kHidden / 4);
    reduce_kernel<false><<<uint32_t(n4 / 256 < 65536 ? (n4 + 255) / 256 : 65536), 256>>>(y_dev, weights_dev, rows, partial_dev,
                                                                                       bf16_dev, fault_dev, nullptr);
    M26G_TRY(out, hipGetLastError(), "b1 reduce launch");
    M26G_TRY(out, hipDeviceSynchronize(), "b1 reduce sync");
    return 0;
}

int m26s_b1_ffn_static(const m26s_b1_layer* L, const uint8_t* payload_dev, size_t payload_pitch, const uint8_t* scales_dev,
                       size_t scales_pitch, const int32_t* ids_dev, const float* weights_dev, uint32_t rows,
                       uint16_t* bf16_out_dev, uint32_t* status_dev, void* hip_stream, char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (bad_call(L, L, rows, payload_pitch, scales_pitch, payload_dev, scales_dev, ids_dev, weights_dev, bf16_out_dev) ||
        (reinterpret_cast<uintptr_t>(payload_dev) & 15) || (payload_pitch & 15) ||
        (reinterpret_cast<uintptr_t>(scales_dev) & 3) || (scales_pitch & 3))
        return out.fail(1, "b1 ffn: bad rows/handles/pitch");
    if (rows > kStaticRows)
        return out.fail(1, "b1 ffn static: %u rows exceed the %u rows the fixed workspace holds", rows, kStaticRows);
    const Shape shape{rows, L->lay.inter, false, false, !L->all_normal, false, false, false};
    if (carve(nullptr, shape).total + kFixedBytes > kStaticBytes)
        return out.fail(1, "b1 ffn static: the call needs more than the fixed workspace of %zu bytes", kStaticBytes);
    const hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    int device = -1;
    M26G_TRY(out, hipGetDevice(&device), "b1 ffn static device");
    if (device < 0 || device >= kStaticDevices) return out.fail(1, "b1 ffn static: device %d is beyond the %d this entry keeps track of", device, kStaticDevices);
    uint8_t* base = static_base[device].load(std::memory_order_acquire);
    if (!base) {  // first call on this GPU: find this GPU's copy of the array (a host-side look-up, nothing is enqueued)
        M26G_TRY(out, hipGetSymbolAddress(reinterpret_cast<void**>(&base), HIP_SYMBOL(scratch)), "b1 ffn static workspace address");
        if (!base) return out.fail(2, "b1 ffn static workspace address: null");
        static_base[device].store(base, std::memory_order_release);
    }
    const Launch k{stream, fixed_at(base), carve(base + kFixedBytes, shape), false, false, nullptr, nullptr, nullptr};
    // The array keeps what the last call left: the count and fault words start every call from zero.
    static_begin_kernel<<<1, 64, 0, stream>>>(base);
    M26G_TRY(out, hipGetLastError(), "b1 ffn static reset");
    M26G_TRY(out, launch_ffn(L, k, payload_dev, payload_pitch, scales_dev, scales_pitch, ids_dev, weights_dev, rows, bf16_out_dev, nullptr),
             "b1 ffn static launch");
    if (status_dev) {
        status_copy_kernel<<<1, 64, 0, stream>>>(status_dev, k.fixed.meta);
        M26G_TRY(out, hipGetLastError(), "b1 ffn static status");
    }
    return 0;
}

void m26s_b1_scratch_set_taps(m26s_b1_scratch* S, int on) { if (S) S->taps = on != 0; }

int m26s_b1_scratch_set_option(m26s_b1_scratch* S, int option, int value) {
    if (!S) return 1;
    const bool on = value != 0;
    switch (option) {
    case M26S_B1_OPT_TAPS: S->taps = on; return 0;
    case M26S_B1_OPT_FUSED_COMBINE: S->fused_combine = on; return 0;
    case M26S_B1_OPT_BF16_ROUTE_ROWS: S->y_bf16 = on; return 0;
    case M26S_B1_OPT_SCOPE_TIMING: S->scope_timing = on; return 0;
    case M26S_B1_OPT_GUARDS:
        if (S->guards != on) {  // the layout changes: the next call starts on a fresh slab, armed again
            if (hipStreamSynchronize(S->stream) != hipSuccess) return 2;
            if (S->slab) (void)hipFree(S->slab);
            S->slab = nullptr;
            S->slab_bytes = 0;
            S->last = Workspace{};
            S->guards = on;
        }
        return 0;
    default: return 1;
    }
}

int m26s_b1_scratch_check_guards(m26s_b1_scratch* S, char* err, size_t errlen) {
    Outcome out(err, errlen);
    if (!S || !S->guards || !S->slab || !S->last.zones) return out.fail(1, "b1 guards: not enabled, or no call made yet");
    M26G_TRY(out, hipStreamSynchronize(S->stream), "b1 guards sync");
    std::vector<uint8_t> host;
    for (int i = 0; i < S->last.zones; ++i) {
        const Zone z = S->last.zone[i];
        host.assign(z.bytes, 0);
        M26G_TRY(out, hipMemcpy(host.data(), S->slab + z.at, z.bytes, hipMemcpyDeviceToHost), "b1 guards download");
        for (uint64_t b = 0; b < z.bytes; ++b)
            if (host[b] != kGuardByte)
                return out.fail(4, "b1 guards: red zone %d damaged at slab offset %llu (byte %llu of %llu holds 0x%02x)", i,
                                static_cast<unsigned long long>(z.at + b), static_cast<unsigned long long>(b),
                                static_cast<unsigned long long>(z.bytes), host[b]);
    }
    return 0;
}

int m26s_b1_device_memory(size_t* free_bytes, size_t* total_bytes) {
    if (!free_bytes || !total_bytes) return 1;
    return hipMemGetInfo(free_bytes, total_bytes) == hipSuccess ? 0 : 2;
}

int m26s_b1_scratch_view(const m26s_b1_scratch* S, int which, void** dev_ptr, size_t* bytes) {
    if (!S || !dev_ptr || !bytes || !S->slab) return 1;
    const Workspace& w = S->last;
    void* const table[] = {w.inverse, w.original, w.grouped_weights, w.groups, S->fixed, w.dq, w.dqs, w.y,
                           w.tap_gate, w.tap_up, w.tap_h, w.chunks, S->fixed + 64};
    if (which < 0 || which >= int(sizeof table / sizeof table[0]) || !table[which]) return 1;
    *dev_ptr = table[which];
    *bytes = which == 4 ? size_t(kMetaWords) * 4 : which == 12 ? 32 : w.bytes[which];
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
