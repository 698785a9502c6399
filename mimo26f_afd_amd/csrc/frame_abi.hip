// Frame adapter (declared in include/m26w_frame.h): the L4 checksum on the host and the gathering of
// a request frame's routes on the device.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include "../../include/m26w_frame.h"

namespace {
struct CrcTables {
    uint32_t t[8][256];
    CrcTables() {
        for (uint32_t i = 0; i < 256; ++i) {
            uint32_t c = i;
            for (int k = 0; k < 8; ++k) c = (c >> 1) ^ ((c & 1u) ? 0x82F63B78u : 0u);
            t[0][i] = c;
        }
        for (uint32_t i = 0; i < 256; ++i)
            for (int s = 1; s < 8; ++s) t[s][i] = (t[s - 1][i] >> 8) ^ t[0][t[s - 1][i] & 0xffu];
    }
};

// One thread per row: descriptor -> its eight route entries -> ids / weights, with the checks of
// crates/mimo26-spark/src/serve.rs:219-232. Entries are read bytewise-safe: a descriptor is 40
// bytes and an entry 12, so neither is 8-byte aligned in general.
__global__ void __launch_bounds__(256) request_routes_kernel(const uint8_t* __restrict__ desc, const uint8_t* __restrict__ routes,
                                                             uint32_t rows, uint32_t route_count, int32_t* __restrict__ ids,
                                                             float* __restrict__ weights, uint32_t* __restrict__ fault) {
    const uint32_t row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    const uint32_t* d = reinterpret_cast<const uint32_t*>(desc + size_t(row) * 40);  // 40 * row is a multiple of 4
    const uint32_t offset = d[7], count = d[8];
    uint32_t code = 0;
    if (count != 8) code = 1;
    else if (uint64_t(offset) + 8 > route_count) code = 2;
    else {
        const uint32_t* r = reinterpret_cast<const uint32_t*>(routes + size_t(offset) * 12);
        for (int j = 0; j < 8; ++j) {
            if (r[3 * j] != row) code = 3;
            ids[size_t(row) * 8 + j] = int32_t(r[3 * j + 1]);
            weights[size_t(row) * 8 + j] = __uint_as_float(r[3 * j + 2]);
        }
    }
    if (code) atomicMin(fault, (row << 2) | code);
}

__global__ void arm_fault_kernel(uint32_t* fault) { *fault = 0xffffffffu; }
__global__ void settle_fault_kernel(uint32_t* fault) { if (*fault == 0xffffffffu) *fault = 0; }
}  // namespace

// The table walk: eight bytes per step through eight 256-entry tables. The fallback where the host has no
// CRC32C instruction, and the checker the instruction path is compared with (crates/mimo26-wire/src/
// crc32c.rs:37-46 keeps its byte-wise walk for the same two purposes).
extern "C" uint32_t m26w_crc32c_update_portable(uint32_t state, const uint8_t* data, size_t n) {
    static const CrcTables tables;
    const uint32_t (*t)[256] = tables.t;
    uint32_t c = state;
    while (n && (reinterpret_cast<uintptr_t>(data) & 7u)) { c = (c >> 8) ^ t[0][(c ^ *data++) & 0xffu]; --n; }
    while (n >= 8) {
        uint64_t w;
        memcpy(&w, data, 8);
        w ^= c;
        c = t[7][w & 0xff] ^ t[6][(w >> 8) & 0xff] ^ t[5][(w >> 16) & 0xff] ^ t[4][(w >> 24) & 0xff] ^
            t[3][(w >> 32) & 0xff] ^ t[2][(w >> 40) & 0xff] ^ t[1][(w >> 48) & 0xff] ^ t[0][w >> 56];
        data += 8;
        n -= 8;
    }
    while (n--) c = (c >> 8) ^ t[0][(c ^ *data++) & 0xffu];
    return c;
}

namespace {
// The x86-64 CRC32C instruction (SSE4.2; the reference's update_sse42, crc32c.rs:48-66) retires eight bytes
// every three cycles on one dependency chain and one a cycle over three independent ones, so long inputs
// are walked as three stripes side by side and the three states are joined afterwards: appending m bytes to
// a message multiplies its state by x^(8m) modulo the polynomial, a linear map over GF(2) that four
// 256-entry tables apply to a 32-bit state.
constexpr size_t kStripe = 4096;  // bytes per stripe; a frame's hidden rows alone are 4224 bytes each

struct ShiftTables {
    uint32_t z[4][256];  // state -> state after kStripe further zero bytes (on raw states, no inversion)
    static uint32_t times(const uint32_t (&mat)[32], uint32_t vec) {
        uint32_t sum = 0;
        for (int i = 0; vec; vec >>= 1, ++i)
            if (vec & 1u) sum ^= mat[i];
        return sum;
    }
    ShiftTables() {
        uint32_t op[32], sq[32];
        op[0] = 0x82F63B78u;  // one zero bit: bit 0 leaves and brings the polynomial in, the others move down
        for (int i = 1; i < 32; ++i) op[i] = 1u << (i - 1);
        size_t bits = 1;
        while (bits < kStripe * 8) {  // kStripe * 8 is a power of two: square up to it
            for (int i = 0; i < 32; ++i) sq[i] = times(op, op[i]);
            memcpy(op, sq, sizeof op);
            bits *= 2;
        }
        for (uint32_t b = 0; b < 256; ++b)
            for (int k = 0; k < 4; ++k) z[k][b] = times(op, b << (8 * k));
    }
    uint32_t shift(uint32_t c) const { return z[0][c & 0xff] ^ z[1][(c >> 8) & 0xff] ^ z[2][(c >> 16) & 0xff] ^ z[3][c >> 24]; }
};
static_assert((kStripe & (kStripe - 1)) == 0 && kStripe % 8 == 0, "a stripe is a power of two of whole words");

#if defined(__x86_64__)
__attribute__((target("sse4.2"))) uint32_t crc32c_hw(uint32_t state, const uint8_t* data, size_t n) {
    static const ShiftTables tables;
    uint64_t c = state;
    while (n && (reinterpret_cast<uintptr_t>(data) & 7u)) { c = __builtin_ia32_crc32qi(uint32_t(c), *data++); --n; }
    while (n >= 3 * kStripe) {
        uint64_t c1 = 0, c2 = 0;  // a stripe that starts from state 0 contributes its state unchanged: the map is linear
        const uint8_t* p = data;
        for (size_t i = 0; i < kStripe; i += 8, p += 8) {
            uint64_t w0, w1, w2;
            memcpy(&w0, p, 8);
            memcpy(&w1, p + kStripe, 8);
            memcpy(&w2, p + 2 * kStripe, 8);
            c = __builtin_ia32_crc32di(c, w0);
            c1 = __builtin_ia32_crc32di(c1, w1);
            c2 = __builtin_ia32_crc32di(c2, w2);
        }
        c = tables.shift(uint32_t(c)) ^ uint32_t(c1);
        c = tables.shift(uint32_t(c)) ^ uint32_t(c2);
        data += 3 * kStripe;
        n -= 3 * kStripe;
    }
    while (n >= 8) {
        uint64_t w;
        memcpy(&w, data, 8);
        c = __builtin_ia32_crc32di(c, w);
        data += 8;
        n -= 8;
    }
    while (n--) c = __builtin_ia32_crc32qi(uint32_t(c), *data++);
    return uint32_t(c);
}
#endif
}  // namespace

extern "C" uint32_t m26w_crc32c_update(uint32_t state, const uint8_t* data, size_t n) {
#if defined(__x86_64__)
    static const bool hw = __builtin_cpu_supports("sse4.2");
    if (hw) return crc32c_hw(state, data, n);
#endif
    return m26w_crc32c_update_portable(state, data, n);
}

extern "C" int m26w_request_routes_dev(const uint8_t* descriptors_dev, const uint8_t* routes_dev, uint32_t rows,
                                       uint32_t route_count, int32_t* ids_dev, float* weights_dev, uint32_t* fault_dev,
                                       void* stream) {
    if (!descriptors_dev || !routes_dev || !ids_dev || !weights_dev || !fault_dev || rows == 0) return 1;
    if ((reinterpret_cast<uintptr_t>(descriptors_dev) | reinterpret_cast<uintptr_t>(routes_dev)) & 3u) return 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    arm_fault_kernel<<<1, 1, 0, s>>>(fault_dev);
    request_routes_kernel<<<(rows + 255) / 256, 256, 0, s>>>(descriptors_dev, routes_dev, rows, route_count, ids_dev, weights_dev, fault_dev);
    settle_fault_kernel<<<1, 1, 0, s>>>(fault_dev);
    return int(hipGetLastError());
}

extern "C" int m26w_stage_rows_dev(uint8_t* aligned_dst_dev, const uint8_t* rows_dev, size_t bytes, void* stream) {
    if (!aligned_dst_dev || !rows_dev || !bytes || (reinterpret_cast<uintptr_t>(aligned_dst_dev) & 15u)) return 1;
    return int(hipMemcpyAsync(aligned_dst_dev, rows_dev, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
}
