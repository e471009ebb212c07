// Fused-dequant GEMV for two to eight rows (small batches, speculative-decoding verify) on the
// PREPARED weight layout, activation-quantized route (ops/native_compute.zig:23834-23870 for
// Q4_0, :29084-29145 for Q8_0).  One launch: the activation quantizer
// (ops/native_compute.zig:23799-23832) runs inside it.
//
//   * work unit of a wavefront: kCols output columns x one K slice of 128 blocks, every weight
//     byte requested at once, as in the one-row kernel (gemv_kernels.hip).
//   * a workgroup is `waves` such wavefronts on ONE K slice (blockIdx.y), so it stages and
//     quantizes only its 4096-value slice of X.  A matrix with a longer K is shared out over
//     blockIdx.y; the slices' sums go to partial[slice][row][column] and a second kernel adds
//     them in slice order (launch_splitk_reduce), so the result does not depend on timing.
//   * staging X: coalesced 16-byte loads (eight lanes per 128-byte line) into LDS, the
//     chunks of a block XOR-swizzled by the block index; then one thread per block reads its
//     32 values back without bank conflicts and quantizes them (the 8-lanes-per-block form
//     costs 2.5 times the vector instructions per value).  The quantized image overwrites
//     the staging area once every thread holds its values in registers.
//   * Q4_0 block dot without unpacking and without touching the weights: with the
//     activation q = 16 h + l - 128 (h, l unsigned nibbles of q + 128) and weight nibbles n
//     (value n - 8):
//       dot(q, n - 8) = 16 (dot_u4(n, h) - 8 sum(n)) + dot_u4(n, l) - 8 sum(q)
//     sum(n) is four dot instructions per weight block, once for all rows; sum(q) comes with
//     the quantized activations.  Eight v_dot8_u32_u4 and four more instructions per
//     (block, column, row).
//   * rows are walked in passes of up to four (sixteen accumulators per lane), the weights
//     stay in registers across passes.
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include "device_common.h"
#include "gemv_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

constexpr int kRawRowBytes = kSliceBlocks * 128;  // staging: one row of one K slice as f32
constexpr int kQRowBytes = kSliceBlocks * 32;     // quantized image of the same

// Quantizes one 32-value block (ops/native_compute.zig:23799-23832: f32 scale = max|x| / 127, one
// reciprocal, round half away from zero, clamp to +-127, zero block -> scale 1) and stores it in
// the image the main loop reads: Q8_0 natural int8 order; Q4_0 two planes of unsigned nibbles of
// q + 128 (h at block * 16, l at 2048 + block * 16, packed in the order of the weight nibbles:
// bits 8t..8t+3 = value 4d+t, bits 8t+4..8t+7 = value 16+4d+t of word d); sum = -8 * sum(q).
template <int kType>
__device__ __forceinline__ void quantize_block_image(const float4 (&v)[8], int block, unsigned char* q_row, float* scale_row,
                                                     int* sum_row) {
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
        m = fmaxf(fmaxf(m, fmaxf(fabsf(v[i].x), fabsf(v[i].y))), fmaxf(fabsf(v[i].z), fabsf(v[i].w)));
    const float s = act_scale(m);
    const float inv = m == 0.0f ? 0.0f : 1.0f / s;
    uint32_t p[8];
    int total = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int q0 = act_quant(v[i].x, inv), q1 = act_quant(v[i].y, inv);
        const int q2 = act_quant(v[i].z, inv), q3 = act_quant(v[i].w, inv);
        p[i] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | (static_cast<uint32_t>(q3 & 0xFF) << 24);
        total = dot4(static_cast<int>(p[i]), 0x01010101, total);
    }
    if (kType == 2) {
        uint32_t h[4], l[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const uint32_t a = p[d] ^ 0x80808080u, b = p[4 + d] ^ 0x80808080u;  // q + 128 per byte
            l[d] = (a & 0x0F0F0F0Fu) | ((b & 0x0F0F0F0Fu) << 4);
            h[d] = ((a >> 4) & 0x0F0F0F0Fu) | (b & 0xF0F0F0F0u);
        }
        reinterpret_cast<uint4*>(q_row)[block] = make_uint4(h[0], h[1], h[2], h[3]);
        reinterpret_cast<uint4*>(q_row + kQRowBytes / 2)[block] = make_uint4(l[0], l[1], l[2], l[3]);
        sum_row[block] = -8 * total;
    } else {
        reinterpret_cast<uint4*>(q_row)[2 * block] = make_uint4(p[0], p[1], p[2], p[3]);
        reinterpret_cast<uint4*>(q_row)[2 * block + 1] = make_uint4(p[4], p[5], p[6], p[7]);
        sum_row[block] = total;
    }
    scale_row[block] = s;
}

constexpr uint32_t kBatchHasEpilogueA = 1u << 28, kBatchHasEpilogueB = 1u << 29;
constexpr uint32_t kBatchReadyCounter = 1u << 30;  // wait for the quantizing wavefronts through a counter in LDS (below)

// blockDim = (64, waves); grid = (column chunks, K slices).
//   shape: waves | stagger << 8 | kBatchHasEpilogue*
//   extras.dots (kWriteDots): int32 [kRows][out_dim][kb] block dots instead of Y
//   partial != nullptr (more than one K slice): sums of slice s go to
//     partial[((matrix * slices + s) * kRows + r) * out_dim + o] instead of Y
template <int kType, int kRows, bool kWriteDots>
__global__ __launch_bounds__(1024) void gemv_batch_kernel(
    const uint8_t* __restrict__ weight_a, const uint8_t* __restrict__ weight_b, const float* __restrict__ input,
    float* __restrict__ dst_a, float* __restrict__ dst_b, uint32_t tile_off16, int kb, int out_dim, uint32_t shape,
    float* __restrict__ partial, GemvExtras extras) {
    using F = GemvFormat<kType>;
    constexpr int kCols = F::kCols;
    constexpr int kLpb = F::kLanesPerBlock;
    constexpr int kBlocksPerStep = kWave / kLpb;
    constexpr int kSteps = F::kSteps;
    constexpr int kWords = kType == 2 ? 8 : 4;
    static_assert(kRows >= 1 && kRows <= 8, "rows per launch");

    extern __shared__ __align__(16) unsigned char lds[];

    const int waves = shape & 0xFF, stagger = (shape >> 8) & 0xFF;
    const int groups_each = (out_dim + kCols - 1) / kCols;
    const int in_dim = kb << 5;
    const int lane = threadIdx.x;  // blockDim.x == 64
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int tid = wave * kWave + lane;
    const int threads = waves * kWave;
    const int slice = blockIdx.y;
    const int slices = gridDim.y;
    const int kb_s = min(kSliceBlocks, kb - slice * kSliceBlocks);  // blocks of this slice, 1..128
    const int half = lane & (kLpb - 1);
    const int lane_block = lane / kLpb;
    const int group_all = blockIdx.x * waves + wave;
    const bool second = weight_b != nullptr && group_all >= groups_each;
    const int group = second ? group_all - groups_each : group_all;
    const uint8_t* weight = second ? weight_b : weight_a;
    const u32x4* qs = reinterpret_cast<const u32x4*>(weight);
    const int o0 = group * kCols;
    const bool active = group < groups_each && o0 < out_dim;
    typedef typename F::TileScales TileScales;
    const TileScales* tile_scales = reinterpret_cast<const TileScales*>(weight + (static_cast<size_t>(tile_off16) << 4)) +
                                    (static_cast<size_t>(min(group, groups_each - 1)) * ((kb + kSliceBlocks - 1) / kSliceBlocks) + slice) * kWave;

    // ---- 1. requests: X (coalesced), then the weights.
    // Two forms.  With the counter (kBatchReadyCounter: the host sets it when the workgroup has wavefronts that do not
    // quantize and LDS holds image and staging side by side, up to seven rows) the first 2 * kRows wavefronts are the
    // quantizers: wavefront w takes the 64 blocks [64 w, +64) of the slice's kRows x 128 (half a row: 8 KB contiguous)
    // straight into 8 KB of LDS of its own with eight global_load_lds (slot 64 i + l of load i = chunk slot l % 8 of
    // block 8 i + l / 8, which receives chunk (l % 8) ^ ((block >> 1) & 7): conflict-free per-thread reads later);
    // one early barrier puts every request for X ahead of every weight request in the memory pipeline's queue (and
    // publishes the cleared counter); the quantizers wait for X alone, then everybody requests weights.  Nobody waits
    // at a barrier behind the weight requests: a wavefront is through those only when the pipeline has accepted them,
    // for the last wavefronts of a unit halfway into the stream.
    // Without the counter: every wavefront fetches a share of X into registers, and three barriers follow (staging
    // written, staging read, image written: the image lies over the staging area).
    const bool ready_counter = (shape & kBatchReadyCounter) != 0;  // wave-uniform
    constexpr uint32_t kCounterOff = kRows * (kQRowBytes + kSliceBlocks * 8);
    uint32_t* ready = reinterpret_cast<uint32_t*>(lds + kCounterOff);
    const bool quantizer = ready_counter && wave < 2 * kRows;
    const uint32_t stage_byte = kCounterOff + 16 + static_cast<uint32_t>(wave) * 8192;
    // staging units of the other form: unit q = row (q >> 4), 64 chunks [64 (q & 15), +64) of that row's slice
    constexpr int kUnits = kRows * 16;
    constexpr int kXPre = 8;  // units per wavefront requested ahead of the weights
    const u32x4* x4 = reinterpret_cast<const u32x4*>(input);
    u32x4 xv[kXPre];
    int xpos[kXPre];
    if (ready_counter) {
        if (tid == 0) *ready = 0;
        if (quantizer) {
            const int r = wave >> 1;
            uint32_t off[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int b = (wave & 1) * 64 + i * 8 + (lane >> 3), c = (lane & 7) ^ ((b >> 1) & 7);
                off[i] = static_cast<uint32_t>((static_cast<size_t>(r) * in_dim + (slice * kSliceBlocks + min(b, kb_s - 1)) * 32) * 4 + c * 16);
            }
            // (all offsets first, then nothing but the requests: the compiler does not count these loads, and a wait it
            // places for reasons of its own between them would wait for them)
            asm volatile("" : "+v"(off[0]), "+v"(off[1]), "+v"(off[2]), "+v"(off[3]), "+v"(off[4]), "+v"(off[5]), "+v"(off[6]), "+v"(off[7]));
            const uint32_t stage_lds = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + stage_byte);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(stage_lds + i * 1024), "v"(off[i]), "s"(input)
                             : "memory", "m0");
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (quantizer) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    } else {
#pragma unroll
        for (int i = 0; i < kXPre; ++i) {
            const int q = wave + i * waves;  // wave-uniform
            if (q < kUnits) {
                const int r = q >> 4, p = ((q & 15) << 6) + lane;  // chunk position p inside the row's staging area
                const int b = p >> 3, c = (p & 7) ^ (b & 7);      // block, 16-byte chunk of it that lives at p
                xpos[i] = r * kRawRowBytes + p * 16;
                xv[i] = x4[(static_cast<size_t>(r) * in_dim + (slice * kSliceBlocks + min(b, kb_s - 1)) * 32) / 4 + c];
            }
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // the activation requests stay ahead of the weight requests

    u32x4 wq[kSteps][kCols];
    LaneScales<kType> wd;
    int blk[kSteps];
    bool ok[kSteps];
    uint32_t lane_off[kSteps];
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
        const int b = j * kBlocksPerStep + lane_block;  // block inside the slice
        ok[j] = active && b < kb_s;
        blk[j] = b < kb_s ? b : kb_s - 1;
        lane_off[j] = static_cast<uint32_t>((slice * kSliceBlocks + blk[j]) * kLpb + half) * 16u;
    }
    for (int q = 0; q < wave * stagger; ++q) __builtin_amdgcn_s_sleep(1);
    wd.w = __builtin_nontemporal_load(tile_scales + lane);
#pragma unroll
    for (int u = 0; u < kCols * kSteps; ++u) {  // K step by K step: the order of consumption
        const int c = u % kCols, j = u / kCols;
        const int o = min(o0 + c, out_dim - 1);
        const uint8_t* qcol = reinterpret_cast<const uint8_t*>(qs + static_cast<size_t>(o) * kb * kLpb);
        wq[j][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(qcol + lane_off[j]));
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. stage X in LDS, quantize one block per thread (two for the first threads when
    // the workgroup has fewer threads than the slice has blocks), image over the staging area
    unsigned char* qimg = lds;                                                         // [kRows][4096]
    float* sx = reinterpret_cast<float*>(lds + kRows * kQRowBytes);                     // [kRows][128]
    int* sumx = reinterpret_cast<int*>(lds + kRows * kQRowBytes + kRows * kSliceBlocks * 4);  // [kRows][128]
    if (ready_counter) {
        if (quantizer) {
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const f32x4* stage = reinterpret_cast<const f32x4*>(lds + stage_byte);
            float4 v[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const f32x4 got = stage[lane * 8 + (c ^ ((lane >> 1) & 7))];
                v[c] = make_float4(got.x, got.y, got.z, got.w);
            }
            const int r = wave >> 1, b = (wave & 1) * 64 + lane;
            quantize_block_image<kType>(v, b, qimg + r * kQRowBytes, sx + r * kSliceBlocks, sumx + r * kSliceBlocks);
            // this wavefront's blocks are in LDS: say so (the fence names LDS only -- a general release would also wait
            // for the wavefront's own weight requests)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            if (lane == 0) __hip_atomic_fetch_add(ready, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        // (bounded all the same; the quantizers depend on nobody)
        for (int spin = 0; spin < (1 << 22) && __hip_atomic_load(ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < 2u * kRows; ++spin)
            __builtin_amdgcn_s_sleep(2);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    } else {
#pragma unroll
        for (int i = 0; i < kXPre; ++i)
            if (wave + i * waves < kUnits) *reinterpret_cast<u32x4*>(lds + xpos[i]) = xv[i];
        for (int q = wave + kXPre * waves; q < kUnits; q += waves) {  // small workgroups: the rest queues behind the weights
            const int r = q >> 4, p = ((q & 15) << 6) + lane;
            const int b = p >> 3, c = (p & 7) ^ (b & 7);
            *reinterpret_cast<u32x4*>(lds + r * kRawRowBytes + p * 16) =
                x4[(static_cast<size_t>(r) * in_dim + (slice * kSliceBlocks + min(b, kb_s - 1)) * 32) / 4 + c];
        }
        __syncthreads();
        constexpr int kXBlocks = kRows * kSliceBlocks;
        float4 raw0[8], raw1[8];
        const int id1 = tid + threads;
        const bool two = id1 < kXBlocks;
        auto read_block = [&](int id, float4 (&v)[8]) {
            const int r = id >> 7, b = id & (kSliceBlocks - 1);
            const unsigned char* base = lds + r * kRawRowBytes + b * 128;
#pragma unroll
            for (int c = 0; c < 8; ++c) v[c] = *reinterpret_cast<const float4*>(base + ((c ^ (b & 7)) << 4));
        };
        if (tid < kXBlocks) read_block(tid, raw0);
        if (two) read_block(id1, raw1);
        __syncthreads();
        auto quantize = [&](int id, const float4 (&v)[8]) {
            const int r = id >> 7, b = id & (kSliceBlocks - 1);
            quantize_block_image<kType>(v, b, qimg + r * kQRowBytes, sx + r * kSliceBlocks, sumx + r * kSliceBlocks);
        };
        if (tid < kXBlocks) quantize(tid, raw0);
        if (two) quantize(id1, raw1);
        __syncthreads();
    }
    wd.exchange();

    // ---- 3. block dots and scaled accumulation
    // Q4_0: -8 * sum of the weight nibbles of each of this lane's blocks (start of the h chain)
    int nsum[kSteps][kCols];
    if (kType == 2) {
#pragma unroll
        for (int j = 0; j < kSteps; ++j)
#pragma unroll
            for (int c = 0; c < kCols; ++c) {
                uint32_t t = dot8_u4(wq[j][c].x, 0x11111111u, 0);
                t = dot8_u4(wq[j][c].y, 0x11111111u, t);
                t = dot8_u4(wq[j][c].z, 0x11111111u, t);
                t = dot8_u4(wq[j][c].w, 0x11111111u, t);
                nsum[j][c] = -8 * static_cast<int>(t);
            }
    }
    const int kb_full = kb;
    auto run_pass = [&](auto row0_tag, auto rows_tag) {
        constexpr int kRow0 = decltype(row0_tag)::value, kN = decltype(rows_tag)::value;
        float acc[kN][kCols];
#pragma unroll
        for (int r = 0; r < kN; ++r)
#pragma unroll
            for (int c = 0; c < kCols; ++c) acc[r][c] = 0.0f;
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            int a[kN][kWords];
            float s[kN];
            int sm[kN];
            const int b = blk[j];
#pragma unroll
            for (int r = 0; r < kN; ++r) {
                const unsigned char* qrow = qimg + (kRow0 + r) * kQRowBytes;
                if (kType == 2) {
                    const int4 a0 = reinterpret_cast<const int4*>(qrow)[b];
                    const int4 a1 = reinterpret_cast<const int4*>(qrow + kQRowBytes / 2)[b];
                    a[r][0] = a0.x; a[r][1] = a0.y; a[r][2] = a0.z; a[r][3] = a0.w;
                    a[r][4 % kWords] = a1.x; a[r][5 % kWords] = a1.y; a[r][6 % kWords] = a1.z; a[r][7 % kWords] = a1.w;
                } else {
                    const int4 a0 = reinterpret_cast<const int4*>(qrow)[b * 2 + half];
                    a[r][0] = a0.x; a[r][1] = a0.y; a[r][2] = a0.z; a[r][3] = a0.w;
                }
                s[r] = ok[j] ? sx[(kRow0 + r) * kSliceBlocks + b] : 0.0f;
                sm[r] = sumx[(kRow0 + r) * kSliceBlocks + b];
            }
#pragma unroll
            for (int c = 0; c < kCols; ++c) {
                const u32x4 w = wq[j][c];
                const float sw = wd.get(j, c, half);
#pragma unroll
                for (int r = 0; r < kN; ++r) {
                    int dot;
                    if (kType == 2) {
                        uint32_t hi = dot8_u4(w.x, static_cast<uint32_t>(a[r][0]), static_cast<uint32_t>(nsum[j][c]));
                        hi = dot8_u4(w.y, static_cast<uint32_t>(a[r][1]), hi);
                        hi = dot8_u4(w.z, static_cast<uint32_t>(a[r][2]), hi);
                        hi = dot8_u4(w.w, static_cast<uint32_t>(a[r][3]), hi);
                        uint32_t lo = dot8_u4(w.x, static_cast<uint32_t>(a[r][4 % kWords]), static_cast<uint32_t>(sm[r]));
                        lo = dot8_u4(w.y, static_cast<uint32_t>(a[r][5 % kWords]), lo);
                        lo = dot8_u4(w.z, static_cast<uint32_t>(a[r][6 % kWords]), lo);
                        lo = dot8_u4(w.w, static_cast<uint32_t>(a[r][7 % kWords]), lo);
                        dot = static_cast<int>((hi << 4) + lo);
                    } else {
                        dot = dot4(static_cast<int>(w.x), a[r][0], 0);
                        dot = dot4(static_cast<int>(w.y), a[r][1], dot);
                        dot = dot4(static_cast<int>(w.z), a[r][2], dot);
                        dot = dot4(static_cast<int>(w.w), a[r][3], dot);
                        dot += dpp_move<kDppXor1>(dot);  // both lanes of the pair hold the block dot
                    }
                    if (kWriteDots && ok[j] && half == 0 && o0 + c < out_dim)
                        extras.dots[(static_cast<size_t>(kRow0 + r) * out_dim + o0 + c) * kb_full + slice * kSliceBlocks + b] = dot;
                    const float tscale = s[r] * sw;
                    const float term = tscale * static_cast<float>(dot);
                    acc[r][c] += (kLpb == 1 || half == 0) ? term : 0.0f;
                }
            }
        }
        if (kWriteDots) return;
        constexpr int kCells = kN * kCols;
        constexpr int kPadded = pow2_at_least(kCells);
        float red[kPadded];
#pragma unroll
        for (int i = 0; i < kPadded; ++i) red[i] = i < kCells ? acc[i / kCols][i % kCols] : 0.0f;
        wave_sum_transposed<kPadded>(red, lane);
        const int cell = lane & (kPadded - 1);
        const int cr = kRow0 + cell / kCols, cc = cell % kCols;
        if (!(active && lane < kPadded && cell < kCells && o0 + cc < out_dim)) return;
        const size_t at = static_cast<size_t>(cr) * out_dim + o0 + cc;
        if (partial != nullptr) {
            partial[(static_cast<size_t>(second ? slices : 0) + slice) * kRows * out_dim + at] = red[0];
            return;
        }
        float* dst = second ? dst_b : dst_a;
        float v = red[0];
        if (shape & (second ? kBatchHasEpilogueB : kBatchHasEpilogueA)) v = finish_output(second ? extras.ep_b : extras.ep_a, o0 + cc, at, v);
        dst[at] = v;
    };
    constexpr int kFirst = kRows <= 4 ? kRows : (kRows + 1) / 2;  // 5 -> 3 + 2, 6 -> 3 + 3, 7 -> 4 + 3, 8 -> 4 + 4
    run_pass(std::integral_constant<int, 0>{}, std::integral_constant<int, kFirst>{});
    if (kRows > kFirst) run_pass(std::integral_constant<int, kFirst>{}, std::integral_constant<int, (kRows > kFirst ? kRows - kFirst : 1)>{});
}

template <typename Kernel>
hipError_t allow_lds(Kernel kernel, size_t lds, std::atomic<size_t>* limit) {
    if (lds <= limit->load(std::memory_order_acquire)) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess) limit->store(160 * 1024, std::memory_order_release);
    return e;
}

template <int kType, int kRows, bool kDots>
hipError_t launch_rows(hipStream_t stream, float* dst_a, float* dst_b, int* dots, const float* input, const uint8_t* weight_a,
                       const uint8_t* weight_b, int in_dim, int out_dim, float* partial, const Epilogue& ep_a, const Epilogue& ep_b) {
    constexpr int kCols = GemvFormat<kType>::kCols;
    const int kb = in_dim / 32;
    const int slices = (kb + kSliceBlocks - 1) / kSliceBlocks;
    const int groups = (out_dim + kCols - 1) / kCols * (weight_b ? 2 : 1);
    const int waves = gemv_batch_waves(kRows, in_dim, groups);
    const int chunks = (groups + waves - 1) / waves;
    // the counter form: wavefronts that do not quantize, and LDS for image, scales, counter and staging side by side
    const bool ready_counter = kRows >= 2 && kRows <= 7 && waves > 2 * kRows;
    const size_t lds = ready_counter ? static_cast<size_t>(kRows) * (kQRowBytes + kSliceBlocks * 8 + kRawRowBytes) + 16
                                     : static_cast<size_t>(kRows) * kRawRowBytes;
    auto kernel = gemv_batch_kernel<kType, kRows, kDots>;
    static std::atomic<size_t> lds_limit{64 * 1024};
    if (hipError_t e = allow_lds(kernel, lds, &lds_limit); e != hipSuccess) return e;
    const size_t tile_off = tile_scales_offset(kType, static_cast<size_t>(out_dim) * kb);
    if ((tile_off >> 4) > 0xFFFFFFFFull) return hipErrorInvalidValue;
    auto has_epilogue = [](const Epilogue& e) { return e.bias != nullptr || e.residual != nullptr || e.activation != kActNone; };
    const bool split = slices > 1 && !kDots;
    if (split && partial == nullptr) return hipErrorInvalidValue;
    const int stagger = static_cast<long>(chunks) * slices <= gemv_compute_units() ? 1 : 0;
    const uint32_t shape = static_cast<uint32_t>(waves) | static_cast<uint32_t>(stagger) << 8 | (ready_counter ? kBatchReadyCounter : 0u) |
                           (!split && has_epilogue(ep_a) ? kBatchHasEpilogueA : 0u) | (!split && has_epilogue(ep_b) ? kBatchHasEpilogueB : 0u);
    const GemvExtras extras{dots, nullptr, ep_a, ep_b};
    hipLaunchKernelGGL(kernel, dim3(chunks, slices), dim3(64, waves), lds, stream, weight_a, weight_b, input, dst_a, dst_b,
                       static_cast<uint32_t>(tile_off >> 4), kb, out_dim, shape, split ? partial : nullptr, extras);
    if (hipError_t e = hipGetLastError(); e != hipSuccess || !split) return e;
    const size_t count = static_cast<size_t>(kRows) * out_dim;
    if (hipError_t e = launch_splitk_reduce(stream, dst_a, partial, count, out_dim, slices, ep_a); e != hipSuccess) return e;
    if (weight_b) return launch_splitk_reduce(stream, dst_b, partial + static_cast<size_t>(slices) * count, count, out_dim, slices, ep_b);
    return hipSuccess;
}

template <int kType>
hipError_t launch_type(hipStream_t stream, float* dst_a, float* dst_b, int* dots, const float* input, const uint8_t* weight_a,
                       const uint8_t* weight_b, int rows, int in_dim, int out_dim, float* partial, const Epilogue& ep_a,
                       const Epilogue& ep_b) {
    switch (rows) {
#define AFHIP_BATCH_ROWS(R)                                                                                                   \
    case R:                                                                                                                   \
        return dots ? launch_rows<kType, R, true>(stream, dst_a, dst_b, dots, input, weight_a, weight_b, in_dim, out_dim, partial, ep_a, ep_b) \
                    : launch_rows<kType, R, false>(stream, dst_a, dst_b, dots, input, weight_a, weight_b, in_dim, out_dim, partial, ep_a, ep_b);
        AFHIP_BATCH_ROWS(1) AFHIP_BATCH_ROWS(2) AFHIP_BATCH_ROWS(3) AFHIP_BATCH_ROWS(4)
        AFHIP_BATCH_ROWS(5) AFHIP_BATCH_ROWS(6) AFHIP_BATCH_ROWS(7) AFHIP_BATCH_ROWS(8)
#undef AFHIP_BATCH_ROWS
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

// Wavefronts per workgroup: enough threads to quantize the slice of X with at most two blocks
// per thread (rows * 128 blocks), at most 16, and -- beyond that minimum -- whatever spreads the
// column groups most evenly over the compute units (ties: the larger workgroup, which repeats
// the quantization less often).
int gemv_batch_waves(int rows, int in_dim, int groups) {
    const int slices = (in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks;
    const int units = gemv_compute_units();
    const int min_waves = rows < 2 ? 2 : rows;
    int best = 16;
    long best_cost = -1;
    for (int waves = 16; waves >= min_waves; --waves) {
        const long grid = static_cast<long>((groups + waves - 1) / waves) * slices;
        const long cost = (grid + units - 1) / units * (waves + 2 * rows);  // streaming share + the prologue every workgroup repeats
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = waves;
        }
    }
    return best;
}

size_t gemv_batch_partial_bytes(size_t rows, size_t in_dim, size_t out_dim, bool pair) {
    const size_t slices = (in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks;
    return slices > 1 ? slices * rows * out_dim * 4 * (pair ? 2 : 1) : 0;
}

hipError_t launch_gemv_batch(hipStream_t stream, int tensor_type, float* dst, int* dots, const float* input,
                             const uint8_t* weight_prepared, int rows, int in_dim, int out_dim, float* partial, float* dst_b,
                             const uint8_t* weight_b_prepared, const Epilogue& ep, const Epilogue& ep_b) {
    if (rows < 1 || rows > 8 || in_dim <= 0 || in_dim % 32 != 0) return hipErrorInvalidValue;
    if (weight_b_prepared != nullptr && dots != nullptr) return hipErrorInvalidValue;
    if ((in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks > 65535) return hipErrorInvalidValue;
    if (tensor_type == 2)
        return launch_type<2>(stream, dst, dst_b, dots, input, weight_prepared, weight_b_prepared, rows, in_dim, out_dim, partial, ep, ep_b);
    return launch_type<8>(stream, dst, dst_b, dots, input, weight_prepared, weight_b_prepared, rows, in_dim, out_dim, partial, ep, ep_b);
}

}  // namespace afhip
