// Measurement aids: what this GPU sustains on the two rooflines the FFN is priced against
// (declared in include/m26_probe.h).
#include <hip/hip_runtime.h>
#include <vector>
#include <stdint.h>
#include <stdio.h>
#include "../../include/m26_probe.h"

namespace {
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

int fail(char* err, size_t errlen, int rc, const char* what, hipError_t e = hipSuccess) {
    if (err && errlen) {
        if (e != hipSuccess) snprintf(err, errlen, "probe: %s: %s", what, hipGetErrorString(e));
        else snprintf(err, errlen, "probe: %s", what);
    }
    return rc;
}

__device__ __forceinline__ uint32_t hash32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

__global__ void __launch_bounds__(256) fill_kernel(uint32_t* p, size_t words, uint32_t mask) {
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < words; i += stride) p[i] = hash32(uint32_t(i) + 1u) & mask;
}

// Grid-stride streaming read, eight 16-byte loads in flight per lane.
__global__ void __launch_bounds__(256) read_kernel(const v4i* __restrict__ p, size_t n, int* out) {
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    v4i acc = {0, 0, 0, 0};
    for (; i + 7 * stride < n; i += 8 * stride) {
        v4i v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    for (; i < n; i += stride) acc ^= __builtin_nontemporal_load(p + i);
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678) out[0] = 1;  // keeps the loads alive
}

// 32 independent accumulators per wave (4 weight tiles x 8 activation tiles, the tile kernels'
// shape); the accumulator is tied so no copy is issued between the MFMAs.
// `clock`, when given, receives from one workgroup in the middle of the grid what its first wave read before and
// after its loop: {shader-clock ticks, ticks of the fixed 100 MHz counter}.
__global__ void __launch_bounds__(256, 2) mfma_kernel(const v4i* w, const v8i* x, float* out, int iters, unsigned long long* clock) {
    const int lane = threadIdx.x & 63;
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    v4i a[4];
    v8i b[8];
#pragma unroll
    for (int t = 0; t < 4; ++t) a[t] = w[lane + 64 * t];
#pragma unroll
    for (int tt = 0; tt < 8; ++tt) b[tt] = x[lane + 64 * tt];
    const uint32_t sa = 0x7f7f7f7fu, sb = 0x7f7f7f7fu;
    v4f acc[4][8];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) acc[t][tt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int tt = 0; tt < 8; ++tt)
#pragma unroll
            for (int t = 0; t < 4; ++t)
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0] cbsz:4"
                             : "+a"(acc[t][tt]) : "v"(a[t]), "v"(b[tt]), "v"(sa), "v"(sb));
    }
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");  // the last MFMAs retire before their results are read
    if (clock && blockIdx.x == gridDim.x / 2 && threadIdx.x == 0) {
        clock[0] = __builtin_amdgcn_s_memtime() - t0;
        clock[1] = __builtin_amdgcn_s_memrealtime() - r0;
    }
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int tt = 0; tt < 8; ++tt) s += acc[t][tt].x;
    out[size_t(blockIdx.x) * blockDim.x + threadIdx.x] = s;
}

struct Events {
    hipEvent_t a = nullptr, b = nullptr;
    ~Events() { if (a) (void)hipEventDestroy(a); if (b) (void)hipEventDestroy(b); }
};
struct Buffer {
    void* p = nullptr;
    ~Buffer() { if (p) (void)hipFree(p); }
};
}  // namespace

#define M26P_TRY(call, what) do { hipError_t e_ = (call); if (e_ != hipSuccess) return fail(err, errlen, 2, what, e_); } while (0)

extern "C" int m26p_read_bandwidth(uint64_t bytes, int reps, void* stream, double* gbps, char* err, size_t errlen) {
    if (!gbps || reps < 1 || reps > 1000 || bytes < (64ull << 20) || (bytes & ((1ull << 20) - 1)))
        return fail(err, errlen, 1, "read_bandwidth: bytes must be a multiple of 1 MiB from 64 MiB up, reps 1..1000");
    hipStream_t s = static_cast<hipStream_t>(stream);
    Buffer data, flag;
    Events ev;
    M26P_TRY(hipMalloc(&data.p, bytes), "hipMalloc");
    M26P_TRY(hipMalloc(&flag.p, 4), "hipMalloc");
    M26P_TRY(hipEventCreate(&ev.a), "hipEventCreate");
    M26P_TRY(hipEventCreate(&ev.b), "hipEventCreate");
    fill_kernel<<<4096, 256, 0, s>>>(static_cast<uint32_t*>(data.p), bytes / 4, 0xffffffffu);
    const size_t n = bytes / 16;
    double best = 0.0;
    const int grids[3] = {4096, 16384, 65536};  // the best launch shape differs a little from part to part
    for (int r = 0; r <= 3 * reps; ++r) {  // repetition 0 warms up
        M26P_TRY(hipEventRecord(ev.a, s), "hipEventRecord");
        read_kernel<<<grids[r % 3], 256, 0, s>>>(static_cast<const v4i*>(data.p), n, static_cast<int*>(flag.p));
        M26P_TRY(hipEventRecord(ev.b, s), "hipEventRecord");
        M26P_TRY(hipEventSynchronize(ev.b), "read kernel");
        float ms = 0.f;
        M26P_TRY(hipEventElapsedTime(&ms, ev.a, ev.b), "hipEventElapsedTime");
        if (r && ms > 0.f && double(bytes) / (ms * 1e-3) / 1e9 > best) best = double(bytes) / (ms * 1e-3) / 1e9;
    }
    *gbps = best;
    return 0;
}

extern "C" int m26p_mfma_rate(int iters, int reps, void* stream, double* tflops, char* err, size_t errlen) {
    if (!tflops || iters < 1 || iters > 100000 || reps < 1 || reps > 1000)
        return fail(err, errlen, 1, "mfma_rate: iters 1..100000, reps 1..1000");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int grid = 2048, threads = 256;  // four workgroups' worth per compute unit, two resident at a time
    Buffer w, x, out;
    Events ev;
    M26P_TRY(hipMalloc(&w.p, 4 * 64 * 16), "hipMalloc");
    M26P_TRY(hipMalloc(&x.p, 8 * 64 * 32), "hipMalloc");
    M26P_TRY(hipMalloc(&out.p, size_t(grid) * threads * 4), "hipMalloc");
    M26P_TRY(hipEventCreate(&ev.a), "hipEventCreate");
    M26P_TRY(hipEventCreate(&ev.b), "hipEventCreate");
    fill_kernel<<<4, 256, 0, s>>>(static_cast<uint32_t*>(w.p), 4 * 64 * 4, 0xffffffffu);  // any nibble is a finite E2M1 code
    fill_kernel<<<16, 256, 0, s>>>(static_cast<uint32_t*>(x.p), 8 * 64 * 8, 0xf7f7f7f7u);  // bit 3 clear: no E4M3 NaN
    double best = 0.0;
    const double flops = double(grid) * (threads / 64) * double(iters) * 32.0 * (2.0 * 16 * 16 * 128);
    for (int r = 0; r <= reps; ++r) {
        M26P_TRY(hipEventRecord(ev.a, s), "hipEventRecord");
        mfma_kernel<<<grid, threads, 0, s>>>(static_cast<const v4i*>(w.p), static_cast<const v8i*>(x.p), static_cast<float*>(out.p), iters, nullptr);
        M26P_TRY(hipEventRecord(ev.b, s), "hipEventRecord");
        M26P_TRY(hipEventSynchronize(ev.b), "mfma kernel");
        float ms = 0.f;
        M26P_TRY(hipEventElapsedTime(&ms, ev.a, ev.b), "hipEventElapsedTime");
        if (r && ms > 0.f && flops / (ms * 1e-3) / 1e12 > best) best = flops / (ms * 1e-3) / 1e12;
    }
    *tflops = best;
    return 0;
}

extern "C" int m26p_mfma_sustained(int iters, int launches, void* stream, double* tflops_first, double* tflops_last,
                                   double* ghz_first, double* ghz_last, char* err, size_t errlen) {
    if (!tflops_first || !tflops_last || !ghz_first || !ghz_last || iters < 1 || iters > 100000 || launches < 2 || launches > 1000)
        return fail(err, errlen, 1, "mfma_sustained: iters 1..100000, launches 2..1000");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int grid = 2048, threads = 256;
    Buffer w, x, out, clock;
    M26P_TRY(hipMalloc(&w.p, 4 * 64 * 16), "hipMalloc");
    M26P_TRY(hipMalloc(&x.p, 8 * 64 * 32), "hipMalloc");
    M26P_TRY(hipMalloc(&out.p, size_t(grid) * threads * 4), "hipMalloc");
    M26P_TRY(hipMalloc(&clock.p, size_t(launches) * 16), "hipMalloc");
    std::vector<hipEvent_t> ev(size_t(launches) + 1, nullptr);
    struct Drop { std::vector<hipEvent_t>& e; ~Drop() { for (hipEvent_t v : e) if (v) (void)hipEventDestroy(v); } } drop{ev};
    for (hipEvent_t& e : ev) M26P_TRY(hipEventCreate(&e), "hipEventCreate");
    fill_kernel<<<4, 256, 0, s>>>(static_cast<uint32_t*>(w.p), 4 * 64 * 4, 0xffffffffu);
    fill_kernel<<<16, 256, 0, s>>>(static_cast<uint32_t*>(x.p), 8 * 64 * 8, 0xf7f7f7f7u);
    M26P_TRY(hipStreamSynchronize(s), "fill");
    M26P_TRY(hipEventRecord(ev[0], s), "hipEventRecord");
    for (int r = 0; r < launches; ++r) {  // back to back, nothing between them but an event
        mfma_kernel<<<grid, threads, 0, s>>>(static_cast<const v4i*>(w.p), static_cast<const v8i*>(x.p), static_cast<float*>(out.p), iters,
                                             static_cast<unsigned long long*>(clock.p) + 2 * r);
        M26P_TRY(hipEventRecord(ev[size_t(r) + 1], s), "hipEventRecord");
    }
    M26P_TRY(hipEventSynchronize(ev[size_t(launches)]), "mfma kernels");
    std::vector<unsigned long long> ticks(size_t(launches) * 2);
    M26P_TRY(hipMemcpy(ticks.data(), clock.p, ticks.size() * 8, hipMemcpyDeviceToHost), "hipMemcpy");
    const double flops = double(grid) * (threads / 64) * double(iters) * 32.0 * (2.0 * 16 * 16 * 128);
    auto rate = [&](int r, double* tf, double* ghz) -> hipError_t {
        float ms = 0.f;
        const hipError_t e = hipEventElapsedTime(&ms, ev[size_t(r)], ev[size_t(r) + 1]);
        *tf = ms > 0.f ? flops / (ms * 1e-3) / 1e12 : 0.0;
        *ghz = ticks[2 * size_t(r) + 1] ? double(ticks[2 * size_t(r)]) / double(ticks[2 * size_t(r) + 1]) * 0.1 : 0.0;
        return e;
    };
    M26P_TRY(rate(0, tflops_first, ghz_first), "hipEventElapsedTime");
    M26P_TRY(rate(launches - 1, tflops_last, ghz_last), "hipEventElapsedTime");
    return 0;
}
