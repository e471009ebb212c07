// Fused-dequant GEMV for decode and speculative-verify rows (rows = 1..8) on the
// PREPARED weight layout, activation-quantized route
// (ops/native_compute.zig:23834-23870 for Q4_0, :29084-29145 for Q8_0).
//
// The kernel is bound by HBM, and at these sizes (one call streams 18-33 MB in a
// few microseconds) by how early the bytes are requested.  So it is "single
// shot": a wavefront requests every weight byte it will ever use as its first
// instructions, and only then does anything else.
//
//   * work unit: kCols consecutive output columns x one K-slice of 4096 values.
//     A slice is kSteps wavefront-wide steps of 16 bytes per lane (Q4_0: lane =
//     block, 2 steps; Q8_0: lane = half block, 4 steps), 1 KiB contiguous per
//     load instruction.
//   * a workgroup is kGroups x slices wavefronts; slices = ceil(in_dim / 4096).
//   * prologue (after the weight requests are out): the workgroup quantizes
//     X[rows, in_dim] into LDS -- the activation quantizer of
//     ops/native_compute.zig:23799-23832, fused.  The first activation loads are
//     issued before the weight loads so that they return first.
//   * each lane accumulates (sx*sw)*f32(dot) for its blocks in f32; the
//     wavefront reduces with DPP; K-slices are combined through LDS in slice
//     order.  The summation order is fixed, so results are run-to-run identical.
#include <hip/hip_runtime.h>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int kType>
struct GemvFormat;
template <>
struct GemvFormat<2> {  // Q4_0: lane = block, 16 B of nibbles
    static constexpr int kLanesPerBlock = 1;
    static constexpr int kQuantBytes = 16;
    static constexpr int kSteps = 2;
};
template <>
struct GemvFormat<8> {  // Q8_0: lane = half block, 16 B of int8
    static constexpr int kLanesPerBlock = 2;
    static constexpr int kQuantBytes = 32;
    static constexpr int kSteps = 4;
};
constexpr int kSliceBlocks = 128;  // 4096 values

// LDS image of the quantized activations.
//   Q4_0: two planes per row so that a lane's two 16-byte reads are unit-stride
//         across lanes: plane 0 holds values 0..15 of every block, plane 1 holds
//         values 16..31 (matching low / high nibbles).
//   Q8_0: natural order; lane (block, half) reads 16 bytes at 16*lane.
// Quantizes one 32-value block held by one thread (8 float4) and stores it.
// Same arithmetic as ops/native_compute.zig:23799-23832: f32 scale = max|x|/127,
// one reciprocal, round half away from zero, clamp to +-127, zero block -> scale 1.
template <int kType>
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

// Workgroups hold at most 1024 threads for 1-2 rows and 512 beyond that (more
// registers per lane for the extra accumulators).
constexpr int gemv_max_threads(int rows) { return rows <= 2 ? 1024 : 512; }

template <int kType, int kRows, int kCols, bool kWriteDots>
__global__ __launch_bounds__(gemv_max_threads(kRows)) void gemv_fused_kernel(float* __restrict__ dst, int* __restrict__ dots, const float* __restrict__ input,
                                  const uint8_t* __restrict__ weight, int in_dim, int out_dim, int slices) {
    using F = GemvFormat<kType>;
    constexpr int kLpb = F::kLanesPerBlock;
    constexpr int kBlocksPerStep = kWave / kLpb;
    constexpr int kSteps = F::kSteps;

    extern __shared__ __align__(16) unsigned char lds[];
    const int kb = in_dim >> 5;
    const int row_dwords = in_dim >> 2;
    int* qx = reinterpret_cast<int*>(lds);                                           // [kRows][in_dim] bytes
    float* sx = reinterpret_cast<float*>(lds + static_cast<size_t>(kRows) * in_dim);  // [kRows][kb]
    int* sumx = reinterpret_cast<int*>(sx + kRows * kb);                              // [kRows][kb]
    float* partial = reinterpret_cast<float*>(sumx + kRows * kb);                     // [waves][kRows*kCols]

    const size_t blocks = static_cast<size_t>(out_dim) * kb;
    const u32x4* qs = reinterpret_cast<const u32x4*>(weight);
    const uint16_t* ds = reinterpret_cast<const uint16_t*>(weight + blocks * F::kQuantBytes);

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    // wavefront-uniform values live in scalar registers, so column base addresses
    // are scalar and each load is "scalar base + one 32-bit lane offset"
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int half = lane & (kLpb - 1);
    const int lane_block = lane / kLpb;
    const int slice = wave % slices;
    const int groups_per_wg = waves / slices;
    const int group = blockIdx.x * groups_per_wg + wave / slices;
    const int o0 = group * kCols;
    const bool active = o0 < out_dim;

    // ---- 1. first activation requests, then every weight byte this wavefront needs
    const int x_blocks = kRows * kb;  // one thread quantizes one block
    float4 xpre[8];
    {
        const int xb = tid < x_blocks ? tid : 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) xpre[i] = reinterpret_cast<const float4*>(input)[xb * 8 + i];
    }

    u32x4 wq[kSteps][kCols];
    uint16_t wd[kSteps][kCols];
    int blk[kSteps];
    bool ok[kSteps];
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
        const int b = slice * kSliceBlocks + j * kBlocksPerStep + lane_block;
        ok[j] = active && b < kb;
        blk[j] = b < kb ? b : kb - 1;  // lanes past the row end re-read its last block and contribute nothing
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
        const int o = min(o0 + c, out_dim - 1);  // likewise for columns past the end
        const u32x4* qcol = qs + static_cast<size_t>(o) * kb * kLpb;
        const uint16_t* dcol = ds + static_cast<size_t>(o) * kb;
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            wq[j][c] = __builtin_nontemporal_load(qcol + blk[j] * kLpb + half);
            wd[j][c] = __builtin_nontemporal_load(dcol + blk[j]);
        }
    }

    // ---- 2. quantize X into LDS, one thread per block
    if (tid < x_blocks) {
        const int r = tid / kb, b = tid - r * kb;
        quantize_block_to_lds<kType>(xpre, b, kb, qx + r * row_dwords, sx + r * kb, sumx + r * kb);
    }
    for (int xb = tid + static_cast<int>(blockDim.x); xb < x_blocks; xb += blockDim.x) {
        float4 v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = reinterpret_cast<const float4*>(input)[xb * 8 + i];
        const int r = xb / kb, b = xb - r * kb;
        quantize_block_to_lds<kType>(v, b, kb, qx + r * row_dwords, sx + r * kb, sumx + r * kb);
    }
    __syncthreads();

    // ---- 3. block dots and scaled accumulation
    float acc[kRows][kCols];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int c = 0; c < kCols; ++c) acc[r][c] = 0.0f;

#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
        const int b = blk[j];
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            const float s = ok[j] ? sx[r * kb + b] : 0.0f;
            int a[8];
            int sm = 0;
            if (kType == 2) {
                const int4 a0 = reinterpret_cast<const int4*>(qx + r * row_dwords)[b];
                const int4 a1 = reinterpret_cast<const int4*>(qx + r * row_dwords + (row_dwords >> 1))[b];
                a[0] = a0.x; a[1] = a0.y; a[2] = a0.z; a[3] = a0.w;
                a[4] = a1.x; a[5] = a1.y; a[6] = a1.z; a[7] = a1.w;
                sm = sumx[r * kb + b];
            } else {
                const int4 a0 = reinterpret_cast<const int4*>(qx + r * row_dwords)[b * 2 + half];
                a[0] = a0.x; a[1] = a0.y; a[2] = a0.z; a[3] = a0.w;
            }
#pragma unroll
            for (int c = 0; c < kCols; ++c) {
                const u32x4 w = wq[j][c];
                int dot;
                if (kType == 2) {
                    // nibbles stay unsigned: dot(qx, n - 8) = dot(qx, n) - 8 * sum(qx)
                    dot = -8 * sm;
                    dot = dot4(static_cast<int>(w.x & 0x0F0F0F0Fu), a[0], dot);
                    dot = dot4(static_cast<int>(w.y & 0x0F0F0F0Fu), a[1], dot);
                    dot = dot4(static_cast<int>(w.z & 0x0F0F0F0Fu), a[2], dot);
                    dot = dot4(static_cast<int>(w.w & 0x0F0F0F0Fu), a[3], dot);
                    dot = dot4(static_cast<int>((w.x >> 4) & 0x0F0F0F0Fu), a[4], dot);
                    dot = dot4(static_cast<int>((w.y >> 4) & 0x0F0F0F0Fu), a[5], dot);
                    dot = dot4(static_cast<int>((w.z >> 4) & 0x0F0F0F0Fu), a[6], dot);
                    dot = dot4(static_cast<int>((w.w >> 4) & 0x0F0F0F0Fu), a[7], dot);
                } else {
                    dot = dot4(static_cast<int>(w.x), a[0], 0);
                    dot = dot4(static_cast<int>(w.y), a[1], dot);
                    dot = dot4(static_cast<int>(w.z), a[2], dot);
                    dot = dot4(static_cast<int>(w.w), a[3], dot);
                    dot += dpp_move<kDppXor1>(dot);  // both lanes of the pair hold the block dot
                }
                if (kWriteDots && ok[j] && half == 0 && o0 + c < out_dim)
                    dots[(static_cast<size_t>(r) * out_dim + o0 + c) * kb + b] = dot;
                const float tscale = s * half_bits_to_f32(wd[j][c]);
                const float term = tscale * static_cast<float>(dot);
                acc[r][c] += (kLpb == 1 || half == 0) ? term : 0.0f;
            }
            // keep one row's activations live at a time: without this fence the
            // scheduler hoists every row's LDS reads and spills registers
            if (kRows > 2) __builtin_amdgcn_sched_barrier(0);
        }
    }

    // ---- 4. wavefront reduction, then K-slices in slice order
    if (slices == 1) {
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int c = 0; c < kCols; ++c) {
                const float total = wave_sum(acc[r][c]);
                if (lane == 0 && o0 + c < out_dim && dst) dst[static_cast<size_t>(r) * out_dim + o0 + c] = total;
            }
        return;
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int c = 0; c < kCols; ++c) {
            const float total = wave_sum(acc[r][c]);
            if (lane == 0) partial[wave * (kRows * kCols) + r * kCols + c] = total;
        }
    __syncthreads();
    const int cells = groups_per_wg * kRows * kCols;
    for (int i = threadIdx.x; i < cells; i += blockDim.x) {
        const int gi = i / (kRows * kCols), rc = i - gi * (kRows * kCols);
        const int r = rc / kCols, c = rc - r * kCols;
        const int o = (blockIdx.x * groups_per_wg + gi) * kCols + c;
        float total = 0.0f;
        for (int s = 0; s < slices; ++s) total += partial[(gi * slices + s) * (kRows * kCols) + rc];
        if (o < out_dim && dst) dst[static_cast<size_t>(r) * out_dim + o] = total;
    }
}

// ---------------------------------------------------------------- launchers

namespace {

template <int kType, int kRows, int kCols>
hipError_t launch_gemv_cols(hipStream_t stream, float* dst, int* dots, const float* input, const uint8_t* weight,
                            int in_dim, int out_dim, const GemvTuning& tune) {
    const int kb = in_dim / 32;
    const int slices = (kb + kSliceBlocks - 1) / kSliceBlocks;
    if (slices > 16) return hipErrorInvalidValue;  // callers route in_dim > 65536 elsewhere
    int waves = (tune.threads < gemv_max_threads(kRows) ? tune.threads : gemv_max_threads(kRows)) / 64;
    if (waves < slices) waves = slices;
    waves = waves / slices * slices;  // whole column groups per workgroup
    const int groups_per_wg = waves / slices;
    const size_t lds = gemv_fused_lds_bytes(kRows, in_dim);
    auto kernel = dots ? gemv_fused_kernel<kType, kRows, kCols, true> : gemv_fused_kernel<kType, kRows, kCols, false>;
    // Raising the dynamic-LDS limit is sticky per kernel: do it once, outside any
    // stream capture a caller may open later.
    static size_t lds_limit = 64 * 1024;
    if (lds > lds_limit) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
        if (e != hipSuccess) return e;
        lds_limit = 128 * 1024;
    }
    const int groups = (out_dim + kCols - 1) / kCols;
    const int grid = (groups + groups_per_wg - 1) / groups_per_wg;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(waves * 64), lds, stream, dst, dots, input, weight, in_dim, out_dim,
                       slices);
    return hipGetLastError();
}

template <int kType, int kRows>
hipError_t launch_gemv_rows(hipStream_t stream, float* dst, int* dots, const float* input, const uint8_t* weight,
                            int in_dim, int out_dim, const GemvTuning& tune) {
    constexpr int kCols = kType == 2 ? (kRows <= 4 ? 4 : 2) : 2;
    if constexpr (kRows <= 2) {
        if (tune.wide)
            return launch_gemv_cols<kType, kRows, 2 * kCols>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
    }
    return launch_gemv_cols<kType, kRows, kCols>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
}

template <int kType>
hipError_t launch_gemv(hipStream_t stream, float* dst, int* dots, const float* input, const uint8_t* weight, int rows,
                       int in_dim, int out_dim, const GemvTuning& tune) {
    switch (rows) {
        case 1: return launch_gemv_rows<kType, 1>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 2: return launch_gemv_rows<kType, 2>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 3: return launch_gemv_rows<kType, 3>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 4: return launch_gemv_rows<kType, 4>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 5: return launch_gemv_rows<kType, 5>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 6: return launch_gemv_rows<kType, 6>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 7: return launch_gemv_rows<kType, 7>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        case 8: return launch_gemv_rows<kType, 8>(stream, dst, dots, input, weight, in_dim, out_dim, tune);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// quantized X (int8 + f32 scale + i32 sum per block) plus one partial-sum slot
// of up to 8 rows x 4 columns for each of up to 16 wavefronts
size_t gemv_fused_lds_bytes(int rows, int in_dim) {
    return static_cast<size_t>(rows) * in_dim + static_cast<size_t>(rows) * (in_dim / 32) * 8 + 16 * 64 * 4;
}

int gemv_fused_max_in_dim() { return 16 * kSliceBlocks * 32; }

hipError_t launch_gemv_fused(hipStream_t stream, int tensor_type, float* dst, int* dots, const float* input,
                             const uint8_t* weight_prepared, int rows, int in_dim, int out_dim,
                             const GemvTuning& tune) {
    if (tensor_type == 2) return launch_gemv<2>(stream, dst, dots, input, weight_prepared, rows, in_dim, out_dim, tune);
    return launch_gemv<8>(stream, dst, dots, input, weight_prepared, rows, in_dim, out_dim, tune);
}

}  // namespace afhip
