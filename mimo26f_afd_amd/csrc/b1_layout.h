// Geometry and the gfx950 prepared-weight layout of the routed-expert FFN (B1, E-W4A8-v1).
//
// Canonical input is the reference's quarter-slice image v2
// (crates/mimo26-expert/src/slice.rs:33-53, kernels/include/mimo26_slice_layout.h:5-21):
// per expert-rank 3,342,336 bytes, rows K-contiguous, low nibble = even k, one E8M0 byte per
// 32 k. The reference permutes it once into an NVIDIA fragment order
// (kernels/b1/prepared.cuh:63-88); here it is permuted once into the operand order of
// CDNA4's v_mfma_scale_f32_16x16x128_f8f6f4. Nibbles and scale bytes are never changed.
//
// MFMA operand facts this layout relies on (measured on MI355X, FP4 operand as SrcA):
//   FP4 operand: lane l holds row (l % 16), k = 32*(l / 16) + p for its 32 nibbles p
//                (4 VGPRs, low nibble first);
//   FP8 operand: lane l holds row (l % 16), bytes 0..15 = k 16*(l/16)..+15 and bytes
//                16..31 = k 64 + 16*(l/16)..+15 (8 VGPRs);
//   scales     : for both operands the E8M0 byte given by lane l scales k-block (l / 16),
//                i.e. k in [32*(l/16), 32*(l/16)+32), of row (l % 16);
//   result     : lane l holds D[4*(l/16) + r][l % 16], r = 0..3.
//
// Prepared expert image ("G950" version 2, I = intermediate columns held, 512 or 2048). Column blocks (32
// intermediate columns of gate + up, or 64 output columns of down) come in sets of eight, and inside a set the
// k-step is the outer index: the eight blocks' fragments of one k-step lie back to back, 32 KB. A workgroup of
// the prefill schedule owns one set and reads those 32 KB per k-step as one run; a workgroup of the decode
// schedule owns half a set and reads 16 KB, its neighbour the other 16.
//   w13 payload  [set = I/256][ks = 32][cb % 8][t = 4][lane = 64][16 B]   tile t: 0,1 = gate rows
//   w13 scales   [cb = I/32][q  = 8 ][t = 4][lane = 64][ 4 B]                     cb*32 + 16*(t&1) + lane%16,
//   w2  payload  [set = 8    ][ks = I/128][ob % 8][t = 4][lane = 64][16 B]         2,3 = the same up rows;
//   w2  scales   [ob = 64  ][q  = I/512][t = 4][lane = 64][ 4 B]   w2 tile t = down rows ob*64 + 16*t + lane%16
// A payload cell is the 16 canonical bytes of k-block 4*ks + lane/16 of its row; a scale cell
// packs, in byte b, the scale of k-block 4*(4*q + b) + lane/16, so one dword serves four
// consecutive k-steps through the MFMA's scale byte select.
// (Version 1 kept every block's k-steps together, [cb][ks]: a wave streamed one contiguous run of 128 or 64 KB.
// A bare streaming kernel whose workgroups read their four waves' k-steps back to back reaches 6.8-6.9 TB/s
// where one contiguous run per wave reaches 6.2-6.4; the decode step became 1.5 % shorter with this order (same box,
// interleaved runs).)
#pragma once
#include <stdint.h>
#include <stddef.h>

namespace m26g {
constexpr uint32_t kHidden = 4096, kExperts = 256, kTopk = 8, kRankI = 512;
constexpr uint64_t kImageBytes = 3342336;
constexpr uint64_t kGatePayload = 0, kGateScales = 1048576, kUpPayload = 1114112, kUpScales = 2162688,
                   kDownPayload = 2228224, kDownScales = 3276800;
constexpr uint32_t kMaxRows = 8192;  // rows per call (the reference caps a call at 4096)

// One k-step of a set of eight column blocks, and where a block's fragments of k-step 0 start inside a payload
// region of `ksteps` k-steps.
constexpr uint32_t kSetBlocks = 8, kStepBytes = kSetBlocks * 4096;
__host__ __device__ constexpr uint64_t block_payload(uint32_t block, uint32_t ksteps) {
    return uint64_t(block / kSetBlocks) * ksteps * kStepBytes + (block % kSetBlocks) * 4096;
}

// Byte offsets of the four regions inside one prepared expert image.
struct Prepared {
    uint32_t inter;  // 512 or 2048
    __host__ __device__ uint64_t w13() const { return 0; }
    __host__ __device__ uint64_t s13() const { return uint64_t(inter) * 4096; }
    __host__ __device__ uint64_t w2() const { return s13() + uint64_t(inter) * 256; }
    __host__ __device__ uint64_t s2() const { return w2() + uint64_t(inter) * 2048; }
    __host__ __device__ uint64_t bytes() const { return s2() + uint64_t(inter) * 128; }
};

// The reference's plan records (kernels/b1/group_plan.cuh:5-9, b1_fc1_m64.cuh:22-24).
struct Group {
    int32_t expert, rows, route_base;
    int32_t input_rows[16];
};
static_assert(sizeof(Group) == 76, "Group is 19 int32");
struct Chunk {
    int32_t first_group, groups;
    int32_t expert;    // the groups' expert, so a kernel can address the weights one load after its index
    int32_t reserved;  // zero
};
static_assert(sizeof(Chunk) == 16, "Chunk is four int32");

// meta words written by the planner and the stage kernels; one small device array per scratch.
enum Meta : uint32_t {
    kGroupCount = 0,
    kPlanFault = 1,   // the reference planner's Status value, 0 = ok
    kChunkCount = 2,
    kFc1Fault = 3,    // metadata faults of the FC1 launch
    kQuantFault = 4,  // 1 nonfinite intermediate (or input scale outside 105..247), 2 overflow
    kQuantWhere = 5,  // lowest faulting K32 block index
    kFc2Fault = 6,
    kReduceFault = 7,
    kMetaWords = 8
};
}  // namespace m26g
