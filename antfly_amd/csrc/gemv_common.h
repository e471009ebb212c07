// Pieces shared by the decode GEMV kernels (one row: gemv_kernels.hip; two to eight rows:
// gemv_batch_kernels.hip).
#pragma once

#include <hip/hip_runtime.h>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <int kType>
struct GemvFormat;
template <>
struct GemvFormat<2> {  // Q4_0: lane = block, 16 B of nibbles
    static constexpr int kLanesPerBlock = 1;
    static constexpr int kQuantBytes = 16;
    static constexpr int kSteps = 2;
    static constexpr int kCols = 4;
    typedef u32x4 TileScales;  // steps 0..1 x columns 0..3
};
template <>
struct GemvFormat<8> {  // Q8_0: lane = half block, 16 B of int8
    static constexpr int kLanesPerBlock = 2;
    static constexpr int kQuantBytes = 32;
    static constexpr int kSteps = 4;
    static constexpr int kCols = 2;
    typedef u32x2 TileScales;  // steps 2 * (lane & 1) + {0, 1} x columns 0..1; the other two steps are the neighbour lane's
};
constexpr int kSliceBlocks = kTileSliceBlocks;  // 4096 values
static_assert(kSliceBlocks == 128, "a wavefront's K slice is one tile of the scale layout");

// A lane's entry of the wavefront-tile copy of the scales, and the scale of (step j, column c)
// out of it.  Q8_0: the two lanes of a block hold two steps each and exchange them.
template <int kType>
struct LaneScales;
template <>
struct LaneScales<2> {
    u32x4 w;
    __device__ __forceinline__ void exchange() {}
    __device__ __forceinline__ float get(int j, int c, int) const {
        const int i = j * 4 + c;
        const uint32_t word = i / 2 == 0 ? w.x : (i / 2 == 1 ? w.y : (i / 2 == 2 ? w.z : w.w));
        return half_bits_to_f32(static_cast<uint16_t>((i & 1) ? word >> 16 : word & 0xFFFFu));
    }
};
template <>
struct LaneScales<8> {
    u32x2 w, other;
    __device__ __forceinline__ void exchange() {
        other.x = static_cast<uint32_t>(dpp_move<kDppXor1>(static_cast<int>(w.x)));
        other.y = static_cast<uint32_t>(dpp_move<kDppXor1>(static_cast<int>(w.y)));
    }
    __device__ __forceinline__ float get(int j, int c, int half) const {
        const u32x2 src = (j >> 1) == half ? w : other;
        const uint32_t word = (j & 1) ? src.y : src.x;
        return half_bits_to_f32(static_cast<uint16_t>(c ? word >> 16 : word & 0xFFFFu));
    }
};

// LDS image of the quantized activations.
//   Q4_0: two planes per row so that a lane's two 16-byte reads are unit-stride
//         across lanes: plane 0 holds values 0..15 of every block, plane 1 holds
//         values 16..31 (matching low / high nibbles) -- or, with kNibblePlanes,
//         the high nibbles and the low nibbles of all 32 values (see below).
//   Q8_0: natural order; lane (block, half) reads 16 bytes at 16*lane.
// Quantizes one 32-value block held by one thread (8 float4) and stores it.
// Same arithmetic as ops/native_compute.zig:23799-23832: f32 scale = max|x|/127,
// one reciprocal, round half away from zero, clamp to +-127, zero block -> scale 1.
// kNibblePlanes (Q4_0 only): instead of int8 values, LDS gets the high nibbles h = q >> 4
// (signed, -8..7) and the low nibbles l = q & 15 (unsigned) of the block, each packed
// eight to a word in the order of the weight nibbles (bits 8t..8t+3 = value 4d+t, bits
// 8t+4..8t+7 = value 16+4d+t of word d), and sum_row gets -8 * sum(l): with weight
// nibbles n (value n - 8, which is n ^ 8 read as a signed nibble)
//   dot(q, n - 8) = 16 * dot_i4(h, n ^ 8) + dot_u4(l, n) - 8 * sum(l).
template <int kType, bool kNibblePlanes = false>
__device__ __forceinline__ void quantize_block_to_lds(const float4 (&v)[8], int block, int kb, int* q_row,
                                                      float* scale_row, int* sum_row) {
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        m = fmaxf(fmaxf(m, fmaxf(fabsf(v[i].x), fabsf(v[i].y))), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
    const float s = act_scale(m);
    const float inv = m == 0.0f ? 0.0f : 1.0f / s;
    int p[8];
    int total = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int q0 = act_quant(v[i].x, inv), q1 = act_quant(v[i].y, inv);
        const int q2 = act_quant(v[i].z, inv), q3 = act_quant(v[i].w, inv);
        p[i] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
        total = dot4(p[i], 0x01010101, total);
    }
    if (kType == 2 && kNibblePlanes) {
        int h[4], l[4];
        uint32_t lsum = 0;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t a = static_cast<uint32_t>(p[d]), b = static_cast<uint32_t>(p[4 + d]);
            l[d] = static_cast<int>((a & 0x0F0F0F0Fu) | ((b & 0x0F0F0F0Fu) << 4));
            h[d] = static_cast<int>(((a >> 4) & 0x0F0F0F0Fu) | (b & 0xF0F0F0F0u));
            lsum = dot8_u4(static_cast<uint32_t>(l[d]), 0x11111111u, lsum);
        }
        reinterpret_cast<int4*>(q_row)[block] = make_int4(h[0], h[1], h[2], h[3]);
        reinterpret_cast<int4*>(q_row + kb * 4)[block] = make_int4(l[0], l[1], l[2], l[3]);
        scale_row[block] = s;
        sum_row[block] = -8 * static_cast<int>(lsum);
        return;
    }
    const int4 lo = make_int4(p[0], p[1], p[2], p[3]), hi = make_int4(p[4], p[5], p[6], p[7]);
    if (kType == 2) {
        // two planes: values 0..15 of every block, then values 16..31 (low / high nibbles)
        reinterpret_cast<int4*>(q_row)[block] = lo;
        reinterpret_cast<int4*>(q_row + kb * 4)[block] = hi;
    } else {
        reinterpret_cast<int4*>(q_row)[2 * block] = lo;
        reinterpret_cast<int4*>(q_row)[2 * block + 1] = hi;
    }
    scale_row[block] = s;
    sum_row[block] = total;
}

constexpr int pow2_at_least(int n) { return n <= 1 ? 1 : (n <= 2 ? 2 : (n <= 4 ? 4 : (n <= 8 ? 8 : 16))); }

// Arguments of the fused GEMV that only some calls use; they follow the sixteen preloaded
// dwords in the kernel-argument segment and are loaded from memory on the paths that need
// them (block dots, argmax keys, a bias / activation / residual epilogue), never on the plain
// Y = X * W^T path.
struct GemvExtras {
    int* dots;
    unsigned long long* keys;
    Epilogue ep_a;  // bias / activation / residual of each matrix (linear, linearPair ...,
    Epilogue ep_b;  // ops/ops.zig:1728, :915)
};
constexpr uint32_t kGemvHasEpilogueA = 1u << 24, kGemvHasEpilogueB = 1u << 25;
constexpr uint32_t kGemvReadyCounter = 1u << 26;  // wait for the quantizing wavefronts through a counter in LDS, not at a barrier


// Compute units of the current device (cached).
int gemv_compute_units();

}  // namespace afhip
