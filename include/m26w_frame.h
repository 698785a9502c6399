/* Frame adapter of the gfx950 expert-FFN library: what the expert daemon does between a DS41RTE3 v3
 * request frame and the FFN call (crates/mimo26-spark/src/serve.rs:206-248), for frames in host
 * memory (as the reference receives them) and for frames that already lie in device memory. */
#ifndef M26W_FRAME_H
#define M26W_FRAME_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* CRC32C (Castagnoli, reflected polynomial 0x82F63B78) update over host bytes, the L4 frame checksum
 * of crates/mimo26-wire/src/crc32c.rs:107-140 (the host's CRC32C instruction where it has one, as there:
 * crc32c.rs:48-66, 86-104): pass state = 0xFFFFFFFF first, chain the returned
 * state over further segments, and invert the last one. m26w_crc32c_update(~0, "123456789", 9)
 * inverted is 0xE3069283. */
uint32_t m26w_crc32c_update(uint32_t state, const uint8_t* data, size_t n);

/* The same function by table look-ups only: what m26w_crc32c_update falls back to on a host without a
 * CRC32C instruction, exported so that the instruction path can be compared with it (the reference keeps
 * its byte-wise table walk beside update_sse42 for the same purpose, crc32c.rs:37-46, 203-216). */
uint32_t m26w_crc32c_update_portable(uint32_t state, const uint8_t* data, size_t n);

/* The route gathering of serve_b1_view (serve.rs:219-232) on the device, for a request frame whose
 * body lies in device memory: `descriptors_dev` = rows x 40-byte row descriptors, `routes_dev` =
 * route_count x 12-byte route entries (crates/mimo26-wire/src/layout.rs:100-118). Writes the
 * token-major ids_dev[rows * 8] and weights_dev[rows * 8] the FFN takes. *fault_dev (one uint32,
 * device) receives 0, or the lowest value of (row << 2 | code) over the rows that break the
 * contract: code 1 = the row does not carry 8 routes, 2 = its route range leaves the route array,
 * 3 = one of its routes names another row. Launches on `stream` (hipStream_t, NULL = default) and
 * does not wait. Returns 0, 1 for a bad argument, or a hipError_t. */
int m26w_request_routes_dev(const uint8_t* descriptors_dev, const uint8_t* routes_dev, uint32_t rows,
                            uint32_t route_count, int32_t* ids_dev, float* weights_dev, uint32_t* fault_dev,
                            void* stream);


/* The FFN reads hidden rows in place with 16-byte loads; a frame's rows start 128 + 136 * rows bytes
 * into it, which is a multiple of 8 only. For a device-resident frame whose rows do not start on a
 * 16-byte boundary this copies them (device to device, on `stream`, not waited for) to an aligned
 * buffer of the caller's. Returns 0, 1 for a bad argument, or a hipError_t. */
int m26w_stage_rows_dev(uint8_t* aligned_dst_dev, const uint8_t* rows_dev, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif
