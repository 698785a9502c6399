// C entry points around the reference's own B1 host units, so the checker can be compared
// with them from Python. TEST INFRASTRUCTURE ONLY. Compiled together with the reference's
// group_plan.cu, route_reduce.cu and quant_v1.cu (as plain C++) from where they lie; no
// reference source is copied into this repository.
#include "group_plan.cuh"
#include "quant_v1.cuh"
#include "route_reduce.cuh"
#include "mimo26_expert_bits.h"
extern "C" {
// crates/mimo26-expert/kernels/include/mimo26_expert_bits.h:29
uint32_t ref_mxfp4_bits(uint32_t nibble, uint32_t scale) { return m26x_decode_bits(nibble, scale, 0); }
// crates/mimo26-expert/kernels/b1/quant_v1.cu:25 ; returns the Status
uint32_t ref_quant_v1(const float* h, uint64_t elements, uint8_t* payload, uint8_t* scales, uint32_t* faults) {
    const uint64_t blocks = elements / 32;
    return static_cast<uint32_t>(m26b1::quantize_host({h, elements}, {payload, scales, faults, elements, blocks, blocks}));
}
// crates/mimo26-expert/kernels/b1/group_plan.cu:80
uint32_t ref_plan(uint32_t capacity, uint32_t rows, const int32_t* ids, const float* weights, const uint8_t* resident,
                  int32_t* inverse, int32_t* original_routes, float* grouped_weights, void* groups,
                  uint32_t* group_count, uint32_t* fault) {
    const uint64_t cap = uint64_t(capacity) * 8;
    m26b1::PlanInput in{capacity, rows, ids, weights, uint64_t(rows) * 8, resident, 256};
    m26b1::PlanStorage out{inverse, original_routes, grouped_weights, static_cast<m26b1::Group*>(groups),
                           group_count, fault, cap, cap};
    return static_cast<uint32_t>(m26b1::plan_host(in, out));
}
// crates/mimo26-expert/kernels/b1/route_reduce.cu:75
uint32_t ref_reduce(const float* y, const float* w, uint32_t rows, float* partial, uint16_t* bf16, uint32_t* fault) {
    const uint64_t n = uint64_t(rows) * 4096;
    return static_cast<uint32_t>(m26b1::reduce_host({rows, y, w, n * 8, uint64_t(rows) * 8}, {partial, bf16, n, n, fault}));
}
}
