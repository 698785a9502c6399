// C ABI of the coordinator-side kernels (include/m26c_glue.h): argument checks and launches.
#include "../../include/m26c_glue.h"
#include "glue_kernels.h"

namespace {

using namespace m26g;

constexpr int kThreads = 256;

int grid_for(long n) {
    long g = (n + kThreads - 1) / kThreads;
    if (g > 65535L * 8) g = 65535L * 8;
    return int(g < 1 ? 1 : g);
}

int launched() { return int(hipGetLastError()); }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// Launch shape of quantize_hidden_kernel: 32 blocks of a row per workgroup along x, rows along y, four rows per
// thread and step. Rows whose outputs are contiguous are one long array (x always is), cut into rows of 32
// blocks so that every thread still has its four loads in flight.
int launch_quantize(const float* x, long rows, long per_row, uint8_t* payload, size_t payload_pitch, uint8_t* scales,
                    size_t scales_pitch, float* scale_inv, void* stream) {
    const long total = rows * per_row;
    if ((!payload || payload_pitch == size_t(per_row) * 32) && scales_pitch == size_t(per_row)) {
        per_row = 32;
        rows = (total + 31) / 32;
        payload_pitch = 1024;
        scales_pitch = 32;
    }
    // About four workgroups per compute unit, each walking several sets of rows with the next set's loads in flight;
    // with fewer rows than that, a workgroup per row (a thread's other three rows fall past the end).
    const long pieces = (per_row + 31) / 32;
    if (pieces > 0x7fffffffL) return 1;
    long walkers = pieces >= 1024 ? 1 : 1024 / pieces;
    walkers = walkers < rows ? walkers : rows;
    quantize_hidden_kernel<<<dim3(unsigned(pieces), unsigned(walkers)), kThreads, 0, hipStream_t(stream)>>>(
        x, rows, per_row, total, payload, payload_pitch, scales, scales_pitch, scale_inv);
    return launched();
}

}  // namespace

extern "C" {

int m26c_router_topk(const float* logits, const float* bias, int rows, int n_experts, int top_k, int* idx_out,
                     float* w_out, void* stream) {
    if (rows <= 0) return 0;
    if (n_experts <= 0 || n_experts > 64 * kRouterPerLane || n_experts % 32 || top_k <= 0 || top_k > n_experts ||
        top_k > 64 || !logits || !bias || !idx_out || !w_out)
        return 1;
    const dim3 grid((rows + 3) / 4);
    hipStream_t st = hipStream_t(stream);
    const int per = (n_experts + 63) / 64;  // a lane's share, rounded up to a compiled size
    if (per <= 1) router_topk_kernel<1><<<grid, kThreads, 0, st>>>(logits, bias, rows, n_experts, top_k, idx_out, w_out);
    else if (per <= 2) router_topk_kernel<2><<<grid, kThreads, 0, st>>>(logits, bias, rows, n_experts, top_k, idx_out, w_out);
    else if (per <= 4) router_topk_kernel<4><<<grid, kThreads, 0, st>>>(logits, bias, rows, n_experts, top_k, idx_out, w_out);
    else if (per <= 8) router_topk_kernel<8><<<grid, kThreads, 0, st>>>(logits, bias, rows, n_experts, top_k, idx_out, w_out);
    else router_topk_kernel<kRouterPerLane><<<grid, kThreads, 0, st>>>(logits, bias, rows, n_experts, top_k, idx_out, w_out);
    return launched();
}

int m26c_quant_scales(const float* x, long n_blocks, unsigned char* scales, float* scale_inv, void* stream) {
    if (n_blocks <= 0) return 0;
    if (!x || !scales || !scale_inv) return 1;
    return launch_quantize(x, n_blocks, 1, nullptr, 0, scales, 1, scale_inv, stream);
}

int m26_quantize_hidden_fp8(const float* x, const float* scale_inv, uint8_t* payload, int64_t n_elem, void* stream) {
    if (n_elem <= 0) return 0;
    if (!x || !scale_inv || !payload) return 1;
    encode_hidden_kernel<<<grid_for(long((n_elem + 3) / 4)), kThreads, 0, hipStream_t(stream)>>>(x, scale_inv, payload, n_elem);
    return launched();
}

int m26c_quantize_hidden(const float* x, long rows, int cols, uint8_t* payload, size_t payload_pitch, uint8_t* scales,
                         size_t scales_pitch, void* stream) {
    if (rows <= 0) return 0;
    if (!x || !payload || !scales || cols <= 0 || cols % 32 || payload_pitch < size_t(cols) || scales_pitch < size_t(cols / 32) ||
        payload_pitch % 4)
        return 1;
    return launch_quantize(x, rows, cols / 32, payload, payload_pitch, scales, scales_pitch, nullptr, stream);
}

int m26c_frame_fill(const int* idx, const float* wts, const uint8_t* payload, const uint8_t* scales, int t, int topk,
                    int hid, uint8_t* routes, uint8_t* hidden, int pitch, void* stream) {
    if (t <= 0) return 0;
    if (!idx || !wts || !payload || !scales || !routes || !hidden || topk <= 0 || hid <= 0 || hid % 256 ||
        pitch < hid + hid / 32 || pitch % 8 || (reinterpret_cast<uintptr_t>(payload) & 15) ||
        (reinterpret_cast<uintptr_t>(scales) & 7) || (reinterpret_cast<uintptr_t>(hidden) & 7) ||
        (reinterpret_cast<uintptr_t>(routes) & 3))
        return 1;
    const int row_groups = (t + 3) / 4;                                   // one wave per hidden row
    const long route_groups = (long(t) * topk + kThreads - 1) / kThreads;  // one lane per route entry
    if (row_groups + route_groups > 0x7fffffffL) return 1;
    frame_fill_kernel<<<unsigned(row_groups + route_groups), kThreads, 0, hipStream_t(stream)>>>(idx, wts, payload, scales, t, topk, hid,
                                                                                              routes, hidden, pitch, row_groups);
    return launched();
}

int m26c_rank_sum_bf16(const uint16_t* p0, const uint16_t* p1, const uint16_t* p2, const uint16_t* p3, float* out,
                       long n, void* stream) {
    if (n <= 0) return 0;
    if (!p0 || !p1 || !p2 || !p3 || !out) return 1;
    if (aligned16(p0) && aligned16(p1) && aligned16(p2) && aligned16(p3) && aligned16(out))
        rank_sum_bf16_kernel<true><<<grid_for((n + 7) / 8), kThreads, 0, hipStream_t(stream)>>>(p0, p1, p2, p3, out, n);
    else
        rank_sum_bf16_kernel<false><<<grid_for(n), kThreads, 0, hipStream_t(stream)>>>(p0, p1, p2, p3, out, n);
    return launched();
}

int m26c_add_inplace(float* h, const float* a, long n, void* stream) {
    if (n <= 0) return 0;
    if (!h || !a) return 1;
    if (aligned16(h) && aligned16(a))
        add_inplace_kernel<true><<<grid_for((n + 7) / 8), kThreads, 0, hipStream_t(stream)>>>(h, a, n);
    else
        add_inplace_kernel<false><<<grid_for(n), kThreads, 0, hipStream_t(stream)>>>(h, a, n);
    return launched();
}

int m26c_f32_to_bf16(const float* x, uint16_t* y, long n, void* stream) {
    if (n <= 0) return 0;
    if (!x || !y) return 1;
    if (aligned16(x) && aligned16(y))
        f32_to_bf16_kernel<true><<<grid_for((n + 7) / 8), kThreads, 0, hipStream_t(stream)>>>(x, y, n);
    else
        f32_to_bf16_kernel<false><<<grid_for(n), kThreads, 0, hipStream_t(stream)>>>(x, y, n);
    return launched();
}

}  // extern "C"
