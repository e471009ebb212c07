// Fused-dequant GEMV for decode and speculative-verify rows (rows = 1..8) on the
// PREPARED weight layout, activation-quantized route
// (ops/native_compute.zig:23834-23870 for Q4_0, :29084-29145 for Q8_0).
//
// The kernel is bound by HBM, and at these sizes (one call streams 18-33 MB in a
// few microseconds) by how early the bytes are requested.  So it is "single
// shot": a wavefront requests every weight byte it will ever use before it
// touches any of them.
//
//   * work unit: kCols consecutive output columns x one K-slice of 4096 values.
//     A slice is kSteps wavefront-wide steps of 16 bytes per lane (Q4_0: lane =
//     block, 2 steps; Q8_0: lane = half block, 4 steps), 1 KiB contiguous per
//     load instruction.
//   * a workgroup is kGroups x slices wavefronts; slices = ceil(in_dim / 4096).
//   * prologue: the workgroup quantizes X[rows, in_dim] into LDS -- the activation
//     quantizer of ops/native_compute.zig:23799-23832, fused.  Loads complete in
//     order, so a wavefront that quantizes asks for X before its weights: the
//     barrier after the prologue never waits for weight bytes.
//   * each lane accumulates (sx*sw)*f32(dot) for its blocks in f32, consuming its
//     weights in the order they were requested; the wavefront reduces with DPP;
//     K-slices are combined through LDS in slice order.  The summation order is
//     fixed, so results are run-to-run identical.
//   * the fp16 scales of a lane's blocks are one more load of the same width: the PREPARED
//     layout keeps a copy of the scales in wavefront-tile order (qmatmul_launch.h), so a
//     wavefront issues nine 1 KiB loads instead of eight plus eight 128-byte ones.  The
//     texture addresser takes a 64-lane load of any width in turn, and the requests of a
//     compute unit's wavefronts all queue there at the start of the kernel.
//   * a launch may serve two matrices of the same shape that share X (GemvTargets).
#include <hip/hip_runtime.h>

#include <atomic>

#include "device_common.h"
#include "gemv_common.h"
#include "qmatmul_launch.h"

namespace afhip {

// Where a GEMV launch reads its weights and writes its results: one matrix, or two of
// the same shape that share X (the engine's linearNoBiasPair, ops/ops.zig:909).  Column
// groups [0, groups_each) belong to the first matrix, [groups_each, 2*groups_each) to
// the second.
struct GemvTargets {
    float* dst_a;
    float* dst_b;
    const uint8_t* weight_a;
    const uint8_t* weight_b;  // null: one matrix
    int groups_each;
    Epilogue ep_a;  // bias / activation / residual of each matrix (linear, linearPair ...,
    Epilogue ep_b;  // ops/ops.zig:1728, :915)
};


// One to four rows of f32 activations, quantized in the prologue of every workgroup.
// kArgmax (one row, one matrix): no Y is written; the workgroup leaves the argmax key of
// its output columns in keys[blockIdx.x] instead.
// Launch shape: blockDim = (64 * slices, groups_per_wg): threadIdx.x / 64 is the K slice,
// threadIdx.y the column group inside the workgroup (no division in the kernel).  The
// leading arguments are everything the plain product needs, and fit the sixteen dwords
// that reach a wavefront in registers at launch (kernel-argument preload): no wavefront
// waits for a kernel-argument load from memory before its first request, or at all.  A
// kernel of this size is as long as its longest wavefront, and each of those starts with
// these instructions.
//   tile_off16: where the scales in tile order start inside a weight, in 16-byte units
//   shape:      slices | groups_per_wg << 8 | stagger << 16 | kGemvHasEpilogue*
//   kCompact:   one K slice (in_dim <= 4096), one matrix, at most one block of X per thread:
//               the instantiation carries none of the code of the other cases (the
//               instruction stream a wavefront walks is half as long)
//   kProbe:     timing diagnostics (afhip_launch_gemv_probe), results meaningless: bit 0 leaves
//               out the block dots (one xor per weight register keeps the loads alive), bit 1
//               the store of Y, bit 2 the activation prologue (no X is read, LDS is used as found)
//               bit 3 (alone): nothing is left out, but instead of Y every wavefront stores eight readings of the 100 MHz
//               clock at extras.dots[8 * (workgroup * wavefronts + wavefront)]: [0] entry, [1] past the wait for the
//               quantized activations (barrier or counter), [2] block dots done, [3] reduction done; quantizing
//               wavefronts of a counter launch also [4] past the barrier behind the requests for X, [5] X there,
//               [6] blocks quantized
constexpr int kProbeNoDots = 1, kProbeNoStore = 2, kProbeNoPrologue = 4, kProbeTimeline = 8;
template <int kType, int kRows, int kCols, bool kWriteDots, bool kArgmax = false, bool kCompact = false, int kProbe = 0, int kDefer = 0>
__device__ __forceinline__ void gemv_fused_body(
    const uint8_t* __restrict__ weight_a, const uint8_t* __restrict__ weight_b, const float* __restrict__ input,
    float* __restrict__ dst_a, float* __restrict__ dst_b, uint32_t tile_off16, int kb, int out_dim, uint32_t shape,
    const GemvExtras& extras) {
    const int slices = kCompact ? 1 : static_cast<int>(shape & 0xFF);
    const int groups_per_wg = (shape >> 8) & 0xFF, stagger = (shape >> 16) & 0xFF;
    const int groups_each = (out_dim + kCols - 1) / kCols;
    const size_t tile_off = static_cast<size_t>(tile_off16) << 4;
    static_assert(!kArgmax || (kRows == 1 && !kWriteDots), "argmax keys: one row, no block dots");
    static_assert(kCols == GemvFormat<kType>::kCols, "the scale tiles are laid out for this many columns per wavefront");
    using F = GemvFormat<kType>;
    constexpr int kLpb = F::kLanesPerBlock;
    constexpr int kBlocksPerStep = kWave / kLpb;
    constexpr int kSteps = F::kSteps;

    extern __shared__ __align__(16) unsigned char lds[];
    uint32_t stamp[8] = {0, 0, 0, 0, 0, 0, 0, 0};  // kProbeTimeline: 100 MHz clock readings, see below
    if (kProbe & kProbeTimeline) stamp[0] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
    const int in_dim = kb << 5;
    const int row_dwords = kb << 3;
    int* qx = reinterpret_cast<int*>(lds);                                           // [kRows][in_dim] bytes
    float* sx = reinterpret_cast<float*>(lds + static_cast<size_t>(kRows) * in_dim);  // [kRows][kb]
    int* sumx = reinterpret_cast<int*>(sx + kRows * kb);                              // [kRows][kb]
    float* partial = reinterpret_cast<float*>(sumx + kRows * kb);                     // [waves][kRows*kCols]

    // [0] = wavefronts that have finished quantizing their blocks of X; 16 bytes in front of the staging area
    const uint32_t flag_off = (static_cast<uint32_t>(kRows) * in_dim + static_cast<uint32_t>(kRows) * kb * 8 +
                               16 * (kRows < 4 ? 4 : kRows) * 16 + 15) & ~15u;
    uint32_t* ready = reinterpret_cast<uint32_t*>(lds + flag_off);
    // Several rows, and wavefronts that do not quantize (the host decides): the quantizers' blocks are waited for
    // through a counter in LDS instead of a barrier (below).
    // (one row of at most 4096 values never takes the counter: that instantiation does not carry its code)
    const bool ready_counter = !(kRows == 1 && kCompact) && (shape & kGemvReadyCounter) != 0;  // wave-uniform
    if (ready_counter && threadIdx.x == 0 && threadIdx.y == 0) *ready = 0;  // (the barrier that publishes it is further down)

    const int lane = threadIdx.x & (kWave - 1);
    // wavefront-uniform values live in scalar registers, so column base addresses
    // are scalar and each load is "scalar base + one 32-bit lane offset"
    const int slice = kCompact ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int group_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.y);
    const int wave = group_in_wg * slices + slice;  // flat wavefront index
    const int tid = wave * kWave + lane;
    const int waves = slices * groups_per_wg;
    const int threads = waves * kWave;
    const int half = lane & (kLpb - 1);
    const int lane_block = lane / kLpb;
    // column group -> matrix (wave-uniform), columns o0 .. o0 + kCols - 1 of it
    const int group_all = blockIdx.x * groups_per_wg + group_in_wg;
    const bool second = !kCompact && weight_b != nullptr && group_all >= groups_each;
    const int group = second ? group_all - groups_each : group_all;
    const uint8_t* weight = second ? weight_b : weight_a;
    const u32x4* qs = reinterpret_cast<const u32x4*>(weight);
    const int o0 = group * kCols;
    const bool active = group < groups_each && o0 < out_dim;
    // this wavefront's tile of the scales (an idle wavefront re-reads the last group's)
    typedef typename F::TileScales TileScales;
    const TileScales* tile_scales = reinterpret_cast<const TileScales*>(weight + tile_off) +
                                    (static_cast<size_t>(min(group, groups_each - 1)) * slices + slice) * kWave;

    // ---- 1. requests: first the activations (wavefronts that quantize a block per
    // thread), then every weight byte this wavefront needs.  Loads complete in order, so
    // the activation requests have to be the older ones: quantizing X -- which the whole
    // workgroup waits for at the barrier -- must not wait for the weights.
    const int x_blocks = kRows * kb;
    u32x4 wq[kSteps][kCols];
    LaneScales<kType> wd;
    int blk[kSteps];
    bool ok[kSteps];
    uint32_t lane_off[kSteps];  // byte offset of this lane's 16 bytes inside a column's quant bytes
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
        const int b = slice * kSliceBlocks + j * kBlocksPerStep + lane_block;
        ok[j] = active && b < kb;
        blk[j] = b < kb ? b : kb - 1;  // lanes past the row end re-read its last block and contribute nothing
        lane_off[j] = static_cast<uint32_t>(blk[j] * kLpb + half) * 16u;
    }
    // Request order = consumption order: the scales, then column by column for one or two
    // rows, K step by K step for more (the activations of a step are then in registers for
    // all columns).
    constexpr bool kStepMajor = kRows > 2;
    auto request_weights = [&]() {
        wd.w = __builtin_nontemporal_load(tile_scales + lane);
#pragma unroll
        for (int u = 0; u < kCols * kSteps; ++u) {
            const int c = kStepMajor ? u % kCols : u / kSteps;
            const int j = kStepMajor ? u / kCols : u % kSteps;
            const int o = min(o0 + c, out_dim - 1);  // columns past the end re-read the last one
            // scalar column base + unsigned 32-bit lane offset: the load takes its address as
            // "SGPR pair + VGPR offset", no 64-bit vector arithmetic between the requests
            const uint8_t* qcol = reinterpret_cast<const uint8_t*>(qs + static_cast<size_t>(o) * kb * kLpb);
            wq[j][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(qcol + lane_off[j]));
        }
    };
    // With more than one row several wavefronts quantize, and the memory pipeline serves requests in the order it
    // accepted them: a quantizer whose requests for X queued behind other wavefronts' weight requests gets X after
    // those kilobytes.  So nobody asks for weights before every quantizer has asked for X: one barrier, reached within
    // a few instructions by everybody (it also publishes the cleared counter).
    auto x_requests_first = [&]() {
        if (ready_counter) {
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            if (kProbe & kProbeTimeline) stamp[4] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
        }
    };
    if (!(kProbe & kProbeNoPrologue) && wave * kWave < x_blocks) {  // wave-uniform
        if (ready_counter) {
            // (The host sets the counter bit only when some wavefront does not quantize: one block a thread at most.)
            // A thread quantizes block `tid` but does not fetch it itself: the wavefront's 64 blocks come in as eight
            // contiguous kilobytes, straight into 8 KB of LDS of its own (global_load_lds: the bytes never are values
            // the compiler could touch before they have arrived), and each thread then picks up its block.  LDS slot
            // 64 i + l of load i is chunk slot l % 8 of block 8 i + l / 8; it receives that block's 16-byte chunk
            // (l % 8) ^ ((block >> 1) & 7), so that the per-thread reads that follow are conflict-free.  No other
            // wavefront touches the region: no barrier.  Then X alone is waited for (nothing else is outstanding: the
            // wait does not depend on where the compiler puts its own loads), the weights are requested, and the
            // quantization runs while they come.
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            const uint32_t stage_byte = flag_off + 16 + static_cast<uint32_t>(wave) * 8192;
            const uint32_t stage_lds = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)) + stage_byte);
            const int last_chunk = x_blocks * 8 - 1;
            uint32_t off[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int b = wave * 64 + i * 8 + (lane >> 3), c = (lane & 7) ^ ((b >> 1) & 7);
                off[i] = static_cast<uint32_t>(min(b * 8 + c, last_chunk)) * 16u;
            }
            // (all eight offsets first, then nothing but the requests: the compiler does not count these loads, and a
            // wait it places for reasons of its own between them -- before a vector register is overwritten, say --
            // would wait for them)
            asm volatile("" : "+v"(off[0]), "+v"(off[1]), "+v"(off[2]), "+v"(off[3]), "+v"(off[4]), "+v"(off[5]), "+v"(off[6]), "+v"(off[7]));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(stage_lds + i * 1024), "v"(off[i]), "s"(input)
                             : "memory", "m0");
            __builtin_amdgcn_sched_barrier(0);
            x_requests_first();
            asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            if (kProbe & kProbeTimeline) stamp[5] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
            __builtin_amdgcn_sched_barrier(0);
            if (kDefer == 0 || (kDefer == 1 && wave < 4)) request_weights();
            __builtin_amdgcn_sched_barrier(0);
            const f32x4* stage = reinterpret_cast<const f32x4*>(lds + stage_byte);
            float4 v[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const f32x4 got = stage[lane * 8 + (c ^ ((lane >> 1) & 7))];
                v[c] = make_float4(got.x, got.y, got.z, got.w);
            }
            if (tid < x_blocks) {
                const int r = tid / kb, b = tid - r * kb;
                quantize_block_to_lds<kType, true>(v, b, kb, qx + r * row_dwords, sx + r * kb, sumx + r * kb);
            }
        } else {
            const int xb = tid < x_blocks ? tid : x_blocks - 1;  // spare lanes of the last such wavefront repeat its last block
            const bool two = !kCompact && x_blocks > threads;    // uniform: a second block per thread
            const int xb1 = min(tid + threads, x_blocks - 1);
            float4 v[8], v1[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = reinterpret_cast<const float4*>(input)[xb * 8 + i];
            if (two) {
#pragma unroll
                for (int i = 0; i < 8; ++i) v1[i] = reinterpret_cast<const float4*>(input)[xb1 * 8 + i];
            }
            __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the weight requests
            x_requests_first();
            request_weights();
            __builtin_amdgcn_sched_barrier(0);
            const int r = xb / kb, b = xb - r * kb;
            quantize_block_to_lds<kType, true>(v, b, kb, qx + r * row_dwords, sx + r * kb, sumx + r * kb);
            if (two) {
                const int r1 = xb1 / kb, b1 = xb1 - r1 * kb;
                quantize_block_to_lds<kType, true>(v1, b1, kb, qx + r1 * row_dwords, sx + r1 * kb, sumx + r1 * kb);
            }
        }
        // more than two blocks per thread (not a shape the host sends here): these requests
        // queue behind the weights
        for (int xb2 = tid + 2 * threads; !kCompact && xb2 < x_blocks; xb2 += threads) {
            float4 v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = reinterpret_cast<const float4*>(input)[xb2 * 8 + i];
            const int r2 = xb2 / kb, b2 = xb2 - r2 * kb;
            quantize_block_to_lds<kType, true>(v, b2, kb, qx + r2 * row_dwords, sx + r2 * kb, sumx + r2 * kb);
        }
        if (kProbe & kProbeTimeline) stamp[6] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
        if (ready_counter) {
            // This wavefront's blocks are in LDS: say so.  The fence names LDS only -- a general release would also
            // wait for the wavefront's own weight requests to complete before the counter moves.
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
            if (lane == 0) __hip_atomic_fetch_add(ready, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            // With two quantizers to a SIMD on a launch that streams for microseconds, a quantizer asks for its weights
            // only now: a request is through when the memory pipeline has accepted it, and right after the barrier that
            // pipeline is taking the requests of all sixteen wavefronts -- a quantizer that joined the queue first began to
            // quantize up to a microsecond late, and every wavefront waits for the last quantizer.  Its own weights come
            // later this way, but the quantizers were the first to finish by a wide margin.  (kDefer: an instantiation of
            // its own, chosen by the host -- a flag tested here cost the launches that do not defer 3 %.  kDefer = 2: all
            // quantizers; 1, for five to seven of them: only those that are a SIMD's second one, wavefronts 4 and up.)
            __builtin_amdgcn_sched_barrier(0);
            if (kDefer == 2 || (kDefer == 1 && wave >= 4)) request_weights();
        }


    } else {
        // The requests of a unit's wavefronts queue at its one texture addresser.  Left alone
        // they interleave, every wavefront's last bytes arrive at the very end and all of them
        // finish their arithmetic at once; entering the queue one after the other, a wavefront
        // gets its bytes in a burst and only the last one still computes when the stream ends.
        x_requests_first();
        for (int q = 0; q < wave * stagger; ++q) __builtin_amdgcn_s_sleep(1);
        request_weights();
    }
    // No barrier here.  A wavefront is through its requests only when the memory pipeline has accepted them all,
    // which for the last wavefronts of a unit is halfway through the stream; a barrier would hold the first ones,
    // whose bytes are long there, until then, and all the arithmetic would be done in the second half.  Each
    // wavefront waits for the quantizers alone (they depend on nobody: the loop ends).
    if (!ready_counter) {
        __syncthreads();
    } else if (!(kProbe & kProbeNoPrologue)) {
        const uint32_t quantizers = static_cast<uint32_t>(min(waves, (x_blocks + kWave - 1) / kWave));
        // (bounded all the same: a wavefront that gave up would compute on what LDS holds and still end)
        for (int spin = 0; spin < (1 << 22) && __hip_atomic_load(ready, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < quantizers; ++spin)
            __builtin_amdgcn_s_sleep(2);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
    if (kProbe & kProbeTimeline) stamp[1] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
    wd.exchange();

    // ---- 3. block dots and scaled accumulation (the weights stay packed in registers)
    static_assert(kRows <= 4, "the accumulators of all rows and columns live in registers");
    constexpr int kWords = kType == 2 ? 8 : 4;
    constexpr int kCells = kRows * kCols;
    // one block of one column against one row's activations
    auto block_dot = [&](const u32x4& w, const int (&a)[kWords], int sm) {
        int dot;
        if (kProbe & kProbeNoDots) return static_cast<int>(w.x ^ w.y ^ w.z ^ w.w) + a[0];
        if (kType == 2) {
            // 4-bit dots on the packed nibbles, nothing is unpacked: a[0..3] = high
            // nibbles of the activations (signed), a[4..7] = low nibbles (unsigned),
            // sm = -8 * sum(low nibbles); see quantize_block_to_lds
            int hi = dot8_i4(static_cast<int>(w.x ^ 0x88888888u), a[0], 0);
            hi = dot8_i4(static_cast<int>(w.y ^ 0x88888888u), a[1], hi);
            hi = dot8_i4(static_cast<int>(w.z ^ 0x88888888u), a[2], hi);
            hi = dot8_i4(static_cast<int>(w.w ^ 0x88888888u), a[3], hi);
            uint32_t lo = dot8_u4(w.x, static_cast<uint32_t>(a[4 % kWords]), static_cast<uint32_t>(sm));
            lo = dot8_u4(w.y, static_cast<uint32_t>(a[5 % kWords]), lo);
            lo = dot8_u4(w.z, static_cast<uint32_t>(a[6 % kWords]), lo);
            lo = dot8_u4(w.w, static_cast<uint32_t>(a[7 % kWords]), lo);
            dot = (hi << 4) + static_cast<int>(lo);
        } else {
            dot = dot4(static_cast<int>(w.x), a[0], 0);
            dot = dot4(static_cast<int>(w.y), a[1], dot);
            dot = dot4(static_cast<int>(w.z), a[2], dot);
            dot = dot4(static_cast<int>(w.w), a[3], dot);
            dot += dpp_move<kDppXor1>(dot);  // both lanes of the pair hold the block dot
        }
        return dot;
    };
    // this lane's activations of block blk[j], row r: words, scale, -8 * sum(low nibbles)
    auto load_x = [&](int j, int r, int (&a)[kWords], float& s, int& sm) {
        const int b = blk[j];
        s = ok[j] ? sx[r * kb + b] : 0.0f;
        sm = 0;
        if (kType == 2) {
            const int4 a0 = reinterpret_cast<const int4*>(qx + r * row_dwords)[b];
            const int4 a1 = reinterpret_cast<const int4*>(qx + r * row_dwords + (row_dwords >> 1))[b];
            a[0] = a0.x; a[1] = a0.y; a[2] = a0.z; a[3] = a0.w;
            a[4 % kWords] = a1.x; a[5 % kWords] = a1.y; a[6 % kWords] = a1.z; a[7 % kWords] = a1.w;
            sm = sumx[r * kb + b];
        } else {
            const int4 a0 = reinterpret_cast<const int4*>(qx + r * row_dwords)[b * 2 + half];
            a[0] = a0.x; a[1] = a0.y; a[2] = a0.z; a[3] = a0.w;
        }
    };
    float acc[kRows][kCols];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
        for (int c = 0; c < kCols; ++c) acc[r][c] = 0.0f;
    auto accumulate = [&](int j, int c, int r, const int (&a)[kWords], float s, int sm) {
        const int dot = block_dot(wq[j][c], a, sm);
        if (kWriteDots && ok[j] && half == 0 && o0 + c < out_dim)
            extras.dots[(static_cast<size_t>(r) * out_dim + o0 + c) * kb + blk[j]] = dot;
        const float tscale = s * wd.get(j, c, half);
        const float term = tscale * static_cast<float>(dot);
        acc[r][c] += (kLpb == 1 || half == 0) ? term : 0.0f;
    };
    if (!kStepMajor) {
        // one or two rows: all activations of this lane's blocks go to registers, then the
        // weights are consumed column by column, in the order their loads were issued
        float sxr[kSteps][kRows];
        int ar[kSteps][kRows][kWords];
        int smr[kSteps][kRows];
#pragma unroll
        for (int j = 0; j < kSteps; ++j)
#pragma unroll
            for (int r = 0; r < kRows; ++r) load_x(j, r, ar[j][r], sxr[j][r], smr[j][r]);
#pragma unroll
        for (int c = 0; c < kCols; ++c)
#pragma unroll
            for (int j = 0; j < kSteps; ++j)
#pragma unroll
                for (int r = 0; r < kRows; ++r) accumulate(j, c, r, ar[j][r], sxr[j][r], smr[j][r]);
    } else {
        // three or four rows: K step by K step (the order of the requests), the step's
        // activations of all rows in registers for all columns
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            float sxr[kRows];
            int ar[kRows][kWords];
            int smr[kRows];
#pragma unroll
            for (int r = 0; r < kRows; ++r) load_x(j, r, ar[r], sxr[r], smr[r]);
#pragma unroll
            for (int c = 0; c < kCols; ++c)
#pragma unroll
                for (int r = 0; r < kRows; ++r) accumulate(j, c, r, ar[r], sxr[r], smr[r]);
        }
    }

    if (kProbe & kProbeTimeline) {
        asm volatile("" : "+v"(acc[0][0]));
        if (kRows * kCols > 1) asm volatile("" : "+v"(acc[kRows - 1][kCols - 1]));  // (never the same register twice in one statement)
        stamp[2] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
    }
    // ---- 4. wavefront reduction (all rows x columns at once)
    constexpr int kPadded = pow2_at_least(kCells);
    static_assert(kCells <= 16, "at most 16 accumulators per lane and reduction");
    float red[kPadded];
#pragma unroll
    for (int i = 0; i < kPadded; ++i) red[i] = i < kCells ? acc[i / kCols][i % kCols] : 0.0f;
    wave_sum_transposed<kPadded>(red, lane);
    const int cell = lane & (kPadded - 1);  // this lane holds the total of accumulator `cell`
    const int cr = cell / kCols, cc = cell % kCols;
    const bool mine = lane < kPadded && cell < kCells;
    if (slices == 1) {
        if (kArgmax) {
            // (`partial` is free here: one word per wavefront)
            const bool live = active && mine && o0 + cc < out_dim;
            const unsigned long long key = workgroup_max_key<kPadded>(
                live ? argmax_key(red[0], static_cast<uint32_t>(o0 + cc)) : 0ull, reinterpret_cast<unsigned long long*>(partial), tid,
                waves);
            if (tid == 0) extras.keys[blockIdx.x] = key;
            return;
        }
        float* dst = second ? dst_b : dst_a;
        if ((kProbe & kProbeNoStore) && red[0] != 1234.5f) return;  // (keeps the arithmetic alive)
        if (kProbe & kProbeTimeline) {
            stamp[3] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
            if (lane == 0 && red[0] != 1234.5f) {  // (keeps the arithmetic alive)
                uint32_t* o = reinterpret_cast<uint32_t*>(extras.dots) + (static_cast<size_t>(blockIdx.x) * waves + wave) * 8;
#pragma unroll
                for (int k = 0; k < 8; ++k) o[k] = stamp[k];
            }
            return;
        }
        if (active && mine && o0 + cc < out_dim && dst) {
            const size_t at = static_cast<size_t>(cr) * out_dim + o0 + cc;
            float v = red[0];
            if (shape & (second ? kGemvHasEpilogueB : kGemvHasEpilogueA)) v = finish_output(second ? extras.ep_b : extras.ep_a, o0 + cc, at, v);
            dst[at] = v;
        }
        return;
    }
    if (mine) partial[wave * kCells + cell] = red[0];
    // K-slices are combined in slice order
    __syncthreads();
    const int cells = groups_per_wg * kCells;
    unsigned long long key = 0;
    for (int i = tid; i < cells; i += threads) {
        const int gi = i / kCells, rc = i - gi * kCells;
        const int r = rc / kCols, c = rc - r * kCols;
        const int ga = blockIdx.x * groups_per_wg + gi;
        const bool sec = !kCompact && weight_b != nullptr && ga >= groups_each;
        const int g = sec ? ga - groups_each : ga;
        float* d = sec ? dst_b : dst_a;
        const int o = g * kCols + c;
        float total = 0.0f;
        for (int sl = 0; sl < slices; ++sl) total += partial[(gi * slices + sl) * kCells + rc];
        if (kArgmax) {
            if (g < groups_each && o < out_dim) {
                const unsigned long long k = argmax_key(total, static_cast<uint32_t>(o));
                if (k > key) key = k;
            }
        } else if (g < groups_each && o < out_dim && d) {
            if (shape & (sec ? kGemvHasEpilogueB : kGemvHasEpilogueA))
                total = finish_output(sec ? extras.ep_b : extras.ep_a, o, static_cast<size_t>(r) * out_dim + o, total);
            d[static_cast<size_t>(r) * out_dim + o] = total;
        }
    }
    if (kArgmax) {
        __syncthreads();  // every total has been read: the partial sums' memory becomes the key slots
        key = workgroup_max_key(key, reinterpret_cast<unsigned long long*>(partial), tid, waves);
        if (tid == 0) extras.keys[blockIdx.x] = key;
    }
    if (kProbe & kProbeTimeline) {  // (several K slices: the probe passes no result array, the readings go out here)
        stamp[3] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
        if (lane == 0) {
            uint32_t* o = reinterpret_cast<uint32_t*>(extras.dots) + (static_cast<size_t>(blockIdx.x) * waves + wave) * 8;
#pragma unroll
            for (int k = 0; k < 8; ++k) o[k] = stamp[k];
        }
    }
}

template <int kType, int kRows, int kCols, bool kWriteDots, bool kArgmax = false, bool kCompact = false, int kProbe = 0, int kDefer = 0>
__global__ __launch_bounds__(1024) void gemv_fused_kernel(
    const uint8_t* __restrict__ weight_a, const uint8_t* __restrict__ weight_b, const float* __restrict__ input,
    float* __restrict__ dst_a, float* __restrict__ dst_b, uint32_t tile_off16, int kb, int out_dim, uint32_t shape,
    GemvExtras extras) {
    gemv_fused_body<kType, kRows, kCols, kWriteDots, kArgmax, kCompact, kProbe, kDefer>(weight_a, weight_b, input, dst_a, dst_b, tile_off16,
                                                                                 kb, out_dim, shape, extras);
}

// =====================================================================
// Same work decomposition for any number of rows whose activations were quantized
// beforehand by quantize_activations_kernel (natural order: pre_q [rows][in_dim] int8,
// pre_scale / pre_sum [rows][in_dim/32]); they are copied into LDS.  The wavefront keeps
// its weights (unpacked once) in registers and walks the rows two at a time, so register
// use does not grow with the row count; `rows` is a run-time value bounded only by LDS.
// =====================================================================
template <int kType, int kCols, bool kWriteDots>
__device__ __forceinline__ void gemv_rows_body(const GemvTargets& tg, int* __restrict__ dots, const int4* __restrict__ pre_q,
                                               const float* __restrict__ pre_scale, const int* __restrict__ pre_sum, int rows,
                                               int in_dim, int out_dim, int slices) {
    using F = GemvFormat<kType>;
    constexpr int kLpb = F::kLanesPerBlock;
    constexpr int kBlocksPerStep = kWave / kLpb;
    constexpr int kSteps = F::kSteps;
    constexpr int kWords = kType == 2 ? 8 : 4;  // int8x4 words of weights per lane per step

    extern __shared__ __align__(16) unsigned char lds[];
    const int kb = in_dim >> 5;
    const int row_dwords = in_dim >> 2;
    int* qx = reinterpret_cast<int*>(lds);                                          // [rows][in_dim] bytes
    float* sx = reinterpret_cast<float*>(lds + static_cast<size_t>(rows) * in_dim);  // [rows][kb]
    int* sumx = reinterpret_cast<int*>(sx + rows * kb);                              // [rows][kb]
    float* partial = reinterpret_cast<float*>(sumx + rows * kb);                     // [waves][rows*kCols]

    const size_t blocks = static_cast<size_t>(out_dim) * kb;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = blockDim.x >> 6;
    const int half = lane & (kLpb - 1);
    const int lane_block = lane / kLpb;
    const int slice = wave % slices;
    const int groups_per_wg = waves / slices;
    // column group -> matrix (wave-uniform), columns o0 .. o0 + kCols - 1 of it
    const int group_all = blockIdx.x * groups_per_wg + wave / slices;
    const bool second = tg.weight_b != nullptr && group_all >= tg.groups_each;
    const int group = second ? group_all - tg.groups_each : group_all;
    const uint8_t* weight = second ? tg.weight_b : tg.weight_a;
    float* dst = second ? tg.dst_b : tg.dst_a;
    const u32x4* qs = reinterpret_cast<const u32x4*>(weight);
    const int o0 = group * kCols;
    const bool active = group < tg.groups_each && o0 < out_dim;
    static_assert(kCols == F::kCols, "the scale tiles are laid out for this many columns per wavefront");
    typedef typename F::TileScales TileScales;
    const TileScales* tile_scales =
        reinterpret_cast<const TileScales*>(weight + ((blocks * (F::kQuantBytes + 2) + 15) & ~static_cast<size_t>(15))) +
        (static_cast<size_t>(min(group, tg.groups_each - 1)) * slices + slice) * kWave;

    int wv[kSteps][kCols][kWords];
    float wd[kSteps][kCols];
    int blk[kSteps];
    bool ok[kSteps];
    uint32_t lane_off[kSteps];
#pragma unroll
    for (int j = 0; j < kSteps; ++j) {
        const int b = slice * kSliceBlocks + j * kBlocksPerStep + lane_block;
        ok[j] = active && b < kb;
        blk[j] = b < kb ? b : kb - 1;
        lane_off[j] = static_cast<uint32_t>(blk[j] * kLpb + half) * 16u;
    }
    {
        u32x4 raw[kSteps][kCols];
        LaneScales<kType> rawd;
        auto request_weights = [&]() {
            rawd.w = __builtin_nontemporal_load(tile_scales + lane);
#pragma unroll
            for (int c = 0; c < kCols; ++c) {
                const int o = min(o0 + c, out_dim - 1);
                const uint8_t* qcol = reinterpret_cast<const uint8_t*>(qs + static_cast<size_t>(o) * kb * kLpb);
#pragma unroll
                for (int j = 0; j < kSteps; ++j)
                    raw[j][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(qcol + lane_off[j]));
            }
        };

        {
            // ---- 1. requests for the quantized X (coalesced, 16 bytes = half a block per
            // thread) go out before the weight requests: loads complete in order, and the copy
            // into LDS (and with it the barrier) must not wait for every weight byte of the
            // wavefront.  kXPre units per thread are requested up front (all of X for up to 8
            // rows of 4096 values with 512 threads); larger inputs copy the rest afterwards.
            constexpr int kXPre = 4;
            const int row_int4 = in_dim >> 4;
            const int x_units = rows * row_int4;
            auto x_lds_index = [&](int u) {
                if (kType != 2) return u;
                const int r = u / row_int4, w = u - r * row_int4;
                return r * row_int4 + (w & 1) * (row_int4 >> 1) + (w >> 1);  // plane (w & 1), block (w >> 1)
            };
            int4 xq[kXPre];
            int xu[kXPre];
#pragma unroll
            for (int i = 0; i < kXPre; ++i) {
                xu[i] = min(tid + i * static_cast<int>(blockDim.x), x_units - 1);  // spare threads repeat the last unit
                xq[i] = pre_q[xu[i]];
            }
            const int su = min(tid, rows * kb - 1);
            const float xs0 = pre_scale[su];
            const int xm0 = pre_sum[su];
            __builtin_amdgcn_sched_barrier(0);  // keep these requests ahead of the weight requests
            request_weights();
#pragma unroll
            for (int i = 0; i < kXPre; ++i) reinterpret_cast<int4*>(qx)[x_lds_index(xu[i])] = xq[i];
            sx[su] = xs0;
            sumx[su] = xm0;
            for (int u = tid + kXPre * static_cast<int>(blockDim.x); u < x_units; u += blockDim.x)
                reinterpret_cast<int4*>(qx)[x_lds_index(u)] = pre_q[u];
            for (int u = tid + static_cast<int>(blockDim.x); u < rows * kb; u += blockDim.x) {
                sx[u] = pre_scale[u];
                sumx[u] = pre_sum[u];
            }
        }

        // X is complete in LDS once every wavefront is here; none of them has had to wait
        // for its weights yet
        __syncthreads();

        // unpack once; lanes that own no block get a zero scale
        rawd.exchange();
#pragma unroll
        for (int j = 0; j < kSteps; ++j)
#pragma unroll
            for (int c = 0; c < kCols; ++c) {
                const u32x4 w = raw[j][c];
                if (kType == 2) {
                    wv[j][c][0] = w.x & 0x0F0F0F0Fu; wv[j][c][1] = w.y & 0x0F0F0F0Fu;
                    wv[j][c][2] = w.z & 0x0F0F0F0Fu; wv[j][c][3] = w.w & 0x0F0F0F0Fu;
                    wv[j][c][4] = (w.x >> 4) & 0x0F0F0F0Fu; wv[j][c][5] = (w.y >> 4) & 0x0F0F0F0Fu;
                    wv[j][c][6] = (w.z >> 4) & 0x0F0F0F0Fu; wv[j][c][7] = (w.w >> 4) & 0x0F0F0F0Fu;
                } else {
                    wv[j][c][0] = w.x; wv[j][c][1] = w.y; wv[j][c][2] = w.z; wv[j][c][3] = w.w;
                }
                wd[j][c] = (ok[j] && (kLpb == 1 || half == 0)) ? rawd.get(j, c, half) : 0.0f;
            }
    }

    // ---- 3. two rows per pass
    const int cells = rows * kCols;
    for (int r0 = 0; r0 < rows; r0 += 2) {
        const int r1 = r0 + 1 < rows ? r0 + 1 : r0;  // odd row count: the last pass repeats its row
        float acc[2][kCols];
#pragma unroll
        for (int c = 0; c < kCols; ++c) acc[0][c] = acc[1][c] = 0.0f;
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
            const int b = blk[j];
#pragma unroll
            for (int rr = 0; rr < 2; ++rr) {
                const int r = rr == 0 ? r0 : r1;
                const float s = sx[r * kb + b];
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
                    int dot = kType == 2 ? -8 * sm : 0;  // unsigned nibbles: dot(qx, n - 8) = dot(qx, n) - 8 sum(qx)
#pragma unroll
                    for (int i = 0; i < kWords; ++i) dot = dot4(wv[j][c][i], a[i], dot);
                    if (kLpb == 2) dot += dpp_move<kDppXor1>(dot);
                    if (kWriteDots && ok[j] && half == 0 && o0 + c < out_dim && (rr == 0 || r1 != r0))
                        dots[(static_cast<size_t>(r) * out_dim + o0 + c) * kb + b] = dot;
                    const float tscale = s * wd[j][c];
                    acc[rr][c] += tscale * static_cast<float>(dot);
                }
            }
        }
        constexpr int kPadded = pow2_at_least(2 * kCols);
        float red[kPadded];
#pragma unroll
        for (int i = 0; i < kPadded; ++i) red[i] = i < 2 * kCols ? acc[i / kCols][i % kCols] : 0.0f;
        wave_sum_transposed<kPadded>(red, lane);
        const int cell = lane & (kPadded - 1);
        const int rr = cell / kCols, cc = cell - rr * kCols;
        const bool mine = lane < kPadded && cell < 2 * kCols && (rr == 0 || r1 != r0);
        const int r = rr == 0 ? r0 : r1;
        if (slices == 1) {
            if (active && mine && o0 + cc < out_dim && dst)
                dst[static_cast<size_t>(r) * out_dim + o0 + cc] =
                    finish_output(second ? tg.ep_b : tg.ep_a, o0 + cc, static_cast<size_t>(r) * out_dim + o0 + cc, red[0]);
        } else if (mine) {
            partial[wave * cells + r * kCols + cc] = red[0];
        }
    }
    if (slices == 1) return;
    __syncthreads();
    for (int i = tid; i < groups_per_wg * cells; i += blockDim.x) {
        const int gi = i / cells, rc = i - gi * cells;
        const int r = rc / kCols, c = rc - r * kCols;
        const int ga = blockIdx.x * groups_per_wg + gi;
        const bool sec = tg.weight_b != nullptr && ga >= tg.groups_each;
        const int g = sec ? ga - tg.groups_each : ga;
        float* d = sec ? tg.dst_b : tg.dst_a;
        const int o = g * kCols + c;
        float total = 0.0f;
        for (int sl = 0; sl < slices; ++sl) total += partial[(gi * slices + sl) * cells + rc];
        if (g < tg.groups_each && o < out_dim && d)
            d[static_cast<size_t>(r) * out_dim + o] =
                finish_output(sec ? tg.ep_b : tg.ep_a, o, static_cast<size_t>(r) * out_dim + o, total);
    }
}

// ---------------------------------------------------------------- launchers

int gemv_compute_units() {
    static const int cus = []() {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        return n;
    }();
    return cus;
}

template <int kType, int kCols, bool kWriteDots>
__global__ __launch_bounds__(512, 4) void gemv_rows_kernel(GemvTargets tg, int* __restrict__ dots,
                                                            const int4* __restrict__ pre_q,
                                                            const float* __restrict__ pre_scale,
                                                            const int* __restrict__ pre_sum, int rows, int in_dim,
                                                            int out_dim, int slices) {
    gemv_rows_body<kType, kCols, kWriteDots>(tg, dots, pre_q, pre_scale, pre_sum, rows, in_dim, out_dim, slices);
}

namespace {

int compute_units() { return gemv_compute_units(); }

// Wavefronts per workgroup: a multiple of `slices` (whole column groups), at most the
// requested size, chosen so that the workgroups spread evenly over the compute units.
// The busiest unit runs ceil(grid / units) workgroups, each `waves` wavefronts of weight
// streaming plus a prologue (X is quantized by every workgroup) that costs about as much
// as kPrologueWaves more; the size (of at least min_waves wavefronts) with the smallest
// such share wins, ties go to the larger workgroup.  A small matrix therefore gets small workgroups (one per unit), a
// large one gets large ones.  `exact` takes the requested size as it is (tuning runs).
int workgroup_waves(int requested_threads, int max_threads, int slices, int groups, bool exact, int min_waves = 1) {
    constexpr int kPrologueWaves = 2;
    int limit = (requested_threads < max_threads ? requested_threads : max_threads) / 64;
    if (limit < slices) limit = slices;
    limit = limit / slices * slices;
    if (exact) return limit;
    const int units = compute_units();
    int best = limit;
    long best_cost = -1;
    if (min_waves < 2) min_waves = 2;  // a lone wavefront per workgroup measured slower than two
    for (int waves = limit; waves >= slices && waves >= min_waves; waves -= slices) {
        const int groups_per_wg = waves / slices;
        const long grid = (groups + groups_per_wg - 1) / groups_per_wg;
        const long cost = (grid + units - 1) / units * (waves + kPrologueWaves);
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = waves;
        }
    }
    return best;
}

// Raising the dynamic-LDS limit is sticky per kernel: done once per kernel, outside
// any stream capture a caller may open later.
template <typename Kernel>
hipError_t allow_large_lds(Kernel kernel, size_t lds, std::atomic<size_t>* limit) {
    if (lds <= limit->load(std::memory_order_acquire)) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       160 * 1024);
    if (e == hipSuccess) limit->store(160 * 1024, std::memory_order_release);  // (two host threads may both get here: the call is idempotent)
    return e;
}

// Whether a fused launch waits for its quantizing wavefronts through the LDS counter (kGemvReadyCounter) instead of a
// barrier: only when some wavefront does not quantize, and for one row only when it is long (measured: a gain from
// K = 6144 on, a small loss on one row of 4096 values, whose two quantizers are done before the barrier matters).
bool use_ready_counter(int rows, int x_blocks, int waves) {
    return waves > (x_blocks + 63) / 64 && (rows >= 2 || x_blocks >= 192);
}
// Whether the quantizing wavefronts of a counter launch ask for their weights behind their quantization (see the kernel):
// where two of them share a SIMD (eight and more; Q8_0, whose wavefronts request twice the bytes, from six on) and the
// launch streams at least 24 MB of weights.  Measured (us, before -> after): Q4_0 four rows x 14336 columns 9.65 -> 9.0,
// two rows K = 11008 x 4096 columns 8.4 -> 7.8, Q8_0 three rows x 14336 columns 14.2 -> 13.45; below those bounds it
// costs: three rows (six quantizers) 8.6 -> 9.0, four rows x 4096 columns 6.0 -> 6.2, one row of 14336 values 7.75 -> 8.1.
// 0: nobody; 1: a SIMD's second quantizer (wavefronts 4 and up) -- five to seven quantizers of Q4_0: three rows x 11008
// columns 7.7 -> 7.15, 28672 columns 16.65 -> 15.9, a pair of 14336 16.9 -> 15.3, 14336 columns 8.7 -> 8.6 (all of them
// late: 8.6 -> 9.0); 2: all quantizers.
int defer_quantizer_weights(int tensor_type, bool ready_counter, int x_blocks, int waves, int in_dim, int out_dim, bool pair) {
    if (!ready_counter) return 0;
    const int quantizers = std::min(waves, (x_blocks + 63) / 64);
    const double bytes = static_cast<double>(out_dim) * (pair ? 2 : 1) * (in_dim / 32) * (tensor_type == 2 ? 18 : 34);
    if (bytes < 24.0e6) return 0;
    if (quantizers >= (tensor_type == 8 ? 6 : 8)) return 2;
    return tensor_type == 2 && quantizers >= 5 ? 1 : 0;
}

// LDS behind the fused kernel's own: 16 bytes of counter, the f32 staging of X (8 KB per quantizing wavefront), alignment
size_t ready_counter_lds_bytes(int x_blocks) { return 32 + static_cast<size_t>((x_blocks + 63) / 64) * 8192; }

template <int kType, int kRows, bool kDots, bool kArgmax = false>
hipError_t launch_fused(hipStream_t stream, const GemvTargets& tg0, int* dots, const float* input, int in_dim,
                        int out_dim, const GemvTuning& tune, unsigned long long* keys = nullptr, int* key_count = nullptr) {
    constexpr int kCols = kType == 2 ? 4 : 2;
    const int slices = (in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks;
    GemvTargets tg = tg0;
    tg.groups_each = (out_dim + kCols - 1) / kCols;
    const int groups = tg.groups_each * (tg.weight_b ? 2 : 1);
    // the prologue quantizes up to two blocks of X per thread ahead of the weight requests
    const int x_blocks = kRows * (in_dim / 32);
    int waves = workgroup_waves(tune.threads, 1024, slices, groups, tune.exact, (x_blocks + 127) / 128);
    // A matrix that takes several rounds of workgroups (a vocabulary): half-size workgroups,
    // two to a compute unit, so that one streams weights while the other is in its prologue.
    if (!tune.exact && waves > 8 && slices <= 8 && x_blocks <= 512 &&
        (groups + waves / slices - 1) / (waves / slices) > compute_units() * 3)
        waves = workgroup_waves(512, 512, slices, groups, true);  // many rounds: nothing to balance
    const int groups_per_wg = waves / slices;
    // Several rows, or one long row, and wavefronts that do not quantize: those wait for the quantizers through a
    // counter, not at a barrier (and X passes through 8 KB of LDS per quantizing wavefront on its way in).
    const bool ready_counter = use_ready_counter(kRows, x_blocks, waves);
    const size_t lds = gemv_fused_lds_bytes(kRows, in_dim) + (ready_counter ? ready_counter_lds_bytes(x_blocks) : 0);
    const bool compact = slices == 1 && tg.weight_b == nullptr && x_blocks <= waves * 64;
    auto kernel = compact ? gemv_fused_kernel<kType, kRows, kCols, kDots, kArgmax, true>
                          : gemv_fused_kernel<kType, kRows, kCols, kDots, kArgmax, false>;
    int defer = 0;
    if constexpr (kRows >= 2 && !kDots && !kArgmax) {  // (the instantiations that request a quantizer's weights late)
        defer = defer_quantizer_weights(kType, ready_counter, x_blocks, waves, in_dim, out_dim, tg.weight_b != nullptr);
        if (defer == 2)
            kernel = compact ? gemv_fused_kernel<kType, kRows, kCols, kDots, kArgmax, true, 0, 2>
                             : gemv_fused_kernel<kType, kRows, kCols, kDots, kArgmax, false, 0, 2>;
        if constexpr (kType == 2) {
            if (defer == 1)
                kernel = compact ? gemv_fused_kernel<kType, kRows, kCols, kDots, kArgmax, true, 0, 1>
                                 : gemv_fused_kernel<kType, kRows, kCols, kDots, kArgmax, false, 0, 1>;
        }
    }
    static std::atomic<size_t> lds_limit[6] = {{64 * 1024}, {64 * 1024}, {64 * 1024}, {64 * 1024}, {64 * 1024}, {64 * 1024}};
    if (hipError_t e = allow_large_lds(kernel, lds, &lds_limit[(compact ? 1 : 0) + 2 * defer]); e != hipSuccess) return e;
    const int grid = (groups + groups_per_wg - 1) / groups_per_wg;
    if (key_count) *key_count = grid;
    // one round of workgroups: the wavefronts of a unit enter its load queue one after the other
    const int stagger = grid <= compute_units() ? 1 : 0;
    const GemvExtras extras{dots, keys, tg.ep_a, tg.ep_b};
    auto has_epilogue = [](const Epilogue& e) { return e.bias != nullptr || e.residual != nullptr || e.activation != kActNone; };
    const size_t tile_off = tile_scales_offset(kType, static_cast<size_t>(out_dim) * (in_dim / 32));
    if ((tile_off >> 4) > 0xFFFFFFFFull || slices > 255 || groups_per_wg > 255) return hipErrorInvalidValue;
    const uint32_t shape = static_cast<uint32_t>(slices) | static_cast<uint32_t>(groups_per_wg) << 8 |
                           static_cast<uint32_t>(stagger) << 16 | (ready_counter ? kGemvReadyCounter : 0u) | (has_epilogue(tg.ep_a) ? kGemvHasEpilogueA : 0u) |
                           (has_epilogue(tg.ep_b) ? kGemvHasEpilogueB : 0u);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * slices, groups_per_wg), lds, stream, tg.weight_a, tg.weight_b, input, tg.dst_a,
                       tg.dst_b, static_cast<uint32_t>(tile_off >> 4), in_dim / 32, out_dim, shape, extras);
    return hipGetLastError();
}

template <int kType, bool kDots>
hipError_t launch_rows(hipStream_t stream, const GemvTargets& tg0, int* dots, const GemvActivations& pre,
                       int rows, int in_dim, int out_dim, const GemvTuning& tune) {
    constexpr int kCols = kType == 2 ? 4 : 2;
    const int slices = (in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks;
    GemvTargets tg = tg0;
    tg.groups_each = (out_dim + kCols - 1) / kCols;
    const int groups = tg.groups_each * (tg.weight_b ? 2 : 1);
    // 8 wavefronts; several of these workgroups share a unit, and smaller ones for small matrices measured no better
    const int waves = workgroup_waves(tune.threads, 512, slices, groups, true);
    const int groups_per_wg = waves / slices;
    const size_t lds = gemv_fused_lds_bytes(rows, in_dim);
    auto kernel = gemv_rows_kernel<kType, kCols, kDots>;
    static std::atomic<size_t> lds_limit{64 * 1024};
    if (hipError_t e = allow_large_lds(kernel, lds, &lds_limit); e != hipSuccess) return e;
    const int grid = (groups + groups_per_wg - 1) / groups_per_wg;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(waves * 64), lds, stream, tg, dots,
                       reinterpret_cast<const int4*>(pre.q), pre.scale, pre.sum, rows, in_dim, out_dim, slices);
    return hipGetLastError();
}

template <int kType>
hipError_t launch_gemv_type(hipStream_t stream, const GemvTargets& tg, int* dots, const float* input,
                            const GemvActivations& pre, int rows, int in_dim, int out_dim, const GemvTuning& tune) {
    if (pre.q != nullptr) {
        return dots ? launch_rows<kType, true>(stream, tg, dots, pre, rows, in_dim, out_dim, tune)
                    : launch_rows<kType, false>(stream, tg, dots, pre, rows, in_dim, out_dim, tune);
    }
    switch (rows) {  // up to four rows: activations quantized in the kernel's own prologue
#define AFHIP_FUSED_ROWS(R)                                                                          \
    case R:                                                                                          \
        return dots ? launch_fused<kType, R, true>(stream, tg, dots, input, in_dim, out_dim, tune)   \
                    : launch_fused<kType, R, false>(stream, tg, dots, input, in_dim, out_dim, tune);
        AFHIP_FUSED_ROWS(1)
        AFHIP_FUSED_ROWS(2)
        AFHIP_FUSED_ROWS(3)
        AFHIP_FUSED_ROWS(4)
#undef AFHIP_FUSED_ROWS
        default: return hipErrorInvalidValue;  // more rows arrive quantized
    }
}

}  // namespace

// quantized X (int8 + f32 scale + i32 sum per block) plus, for each of up to 16
// wavefronts, one partial-sum slot per (row, column) it owns (at most 4 columns)
size_t gemv_fused_lds_bytes(int rows, int in_dim) {
    const size_t x_blocks = static_cast<size_t>(rows) * (in_dim / 32);
    return static_cast<size_t>(rows) * in_dim + x_blocks * 8 + static_cast<size_t>(16) * (rows < 4 ? 4 : rows) * 4 * 4;
}

int gemv_fused_max_in_dim() { return 16 * kSliceBlocks * 32; }

hipError_t launch_gemv_fused(hipStream_t stream, int tensor_type, float* dst, int* dots, const float* input,
                             const GemvActivations& pre, const uint8_t* weight_prepared, int rows, int in_dim,
                             int out_dim, const GemvTuning& tune, float* dst_b, const uint8_t* weight_b_prepared,
                             const Epilogue& ep, const Epilogue& ep_b) {
    if (in_dim > gemv_fused_max_in_dim()) return hipErrorInvalidValue;
    if (weight_b_prepared != nullptr && dots != nullptr) return hipErrorInvalidValue;  // block dots: one matrix at a time
    const GemvTargets tg{dst, dst_b, weight_prepared, weight_b_prepared, 0, ep, ep_b};
    if (tensor_type == 2) return launch_gemv_type<2>(stream, tg, dots, input, pre, rows, in_dim, out_dim, tune);
    return launch_gemv_type<8>(stream, tg, dots, input, pre, rows, in_dim, out_dim, tune);
}

// Timing diagnostics on the Q4_0 decode kernel for one, two and four rows (compact instantiation: in_dim <= 4096; at
// four rows the one whose quantizing wavefronts request their weights late, which launch_fused picks on a launch of
// 24 MB of weights and more -- the probe's matrix).
namespace {
template <int kRows>
hipError_t launch_gemv_probe_rows(hipStream_t stream, int probe, float* dst, const float* input, const uint8_t* weight_prepared,
                                  int in_dim, int out_dim, uint32_t* stamps, size_t stamps_bytes, int* grid_out, int* waves_out) {
    constexpr int kCols = 4;
    const int groups = (out_dim + kCols - 1) / kCols;
    const int x_blocks = kRows * (in_dim / 32);
    if (in_dim > kSliceBlocks * 32) {
        // the timeline of a row longer than one K slice: launch_fused's shape for one matrix, the kernel's general
        // instantiation (K slices side by side in a workgroup, their sums meeting in LDS)
        if (probe != kProbeTimeline || stamps == nullptr) return hipErrorInvalidValue;
        const int slices = (in_dim / 32 + kSliceBlocks - 1) / kSliceBlocks;
        const int waves = workgroup_waves(1024, 1024, slices, groups, false, (x_blocks + 127) / 128);
        const int groups_per_wg = waves / slices, grid = (groups + groups_per_wg - 1) / groups_per_wg;
        const bool ready_counter = use_ready_counter(kRows, x_blocks, waves);
        const size_t lds = gemv_fused_lds_bytes(kRows, in_dim) + (ready_counter ? ready_counter_lds_bytes(x_blocks) : 0);
        const size_t tile_off = tile_scales_offset(2, static_cast<size_t>(out_dim) * (in_dim / 32));
        if (grid_out) *grid_out = grid;
        if (waves_out) *waves_out = waves;
        if (stamps_bytes < static_cast<size_t>(grid) * waves * 32 || slices > 255 || groups_per_wg > 255) return hipErrorInvalidValue;
        auto kernel = gemv_fused_kernel<2, kRows, kCols, false, false, false, kProbeTimeline>;
        static std::atomic<size_t> long_lds_limit{64 * 1024};
        if (hipError_t e = allow_large_lds(kernel, lds, &long_lds_limit); e != hipSuccess) return e;
        const uint32_t shape = static_cast<uint32_t>(slices) | static_cast<uint32_t>(groups_per_wg) << 8 |
                               (grid <= compute_units() ? 1u << 16 : 0u) | (ready_counter ? kGemvReadyCounter : 0u);
        const GemvExtras extras{reinterpret_cast<int*>(stamps), nullptr, Epilogue{}, Epilogue{}};
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * slices, groups_per_wg), lds, stream, weight_prepared,
                           static_cast<const uint8_t*>(nullptr), input, dst, static_cast<float*>(nullptr),
                           static_cast<uint32_t>(tile_off >> 4), in_dim / 32, out_dim, shape, extras);
        return hipGetLastError();
    }
    const int waves = workgroup_waves(1024, 1024, 1, groups, false, (x_blocks + 127) / 128);
    if (x_blocks > waves * 64) return hipErrorInvalidValue;  // the compact instantiation: one block of X per thread
    const int grid = (groups + waves - 1) / waves;
    const size_t tile_off = tile_scales_offset(2, static_cast<size_t>(out_dim) * (in_dim / 32));
    const bool ready_counter = use_ready_counter(kRows, x_blocks, waves);
    const uint32_t shape = 1u | static_cast<uint32_t>(waves) << 8 | (grid <= compute_units() ? 1u << 16 : 0u) |
                           (ready_counter ? kGemvReadyCounter : 0u);
    if (grid_out) *grid_out = grid;
    if (waves_out) *waves_out = waves;
    if (probe == kProbeTimeline && (stamps == nullptr || stamps_bytes < static_cast<size_t>(grid) * waves * 32)) return hipErrorInvalidValue;
    const GemvExtras extras{reinterpret_cast<int*>(stamps), nullptr, Epilogue{}, Epilogue{}};
    const size_t lds = gemv_fused_lds_bytes(kRows, in_dim) + (ready_counter ? ready_counter_lds_bytes(x_blocks) : 0);
    static std::atomic<size_t> lds_limit[9] = {{64 * 1024}, {64 * 1024}, {64 * 1024}, {64 * 1024},
                                               {64 * 1024}, {64 * 1024}, {64 * 1024}, {64 * 1024}, {64 * 1024}};
#define AFHIP_PROBE(P)                                                                                                  \
    case P: {                                                                                                           \
        auto kernel = gemv_fused_kernel<2, kRows, kCols, false, false, true, P, (kRows >= 4 ? 2 : 0)>;                  \
        if (hipError_t e = allow_large_lds(kernel, lds, &lds_limit[P]); e != hipSuccess) return e;                      \
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(64, waves), lds, stream, weight_prepared,                           \
                           static_cast<const uint8_t*>(nullptr), input, dst, static_cast<float*>(nullptr),              \
                           static_cast<uint32_t>(tile_off >> 4), in_dim / 32, out_dim, shape, extras);                  \
        break;                                                                                                          \
    }
    switch (probe) {
        AFHIP_PROBE(0) AFHIP_PROBE(1) AFHIP_PROBE(2) AFHIP_PROBE(3) AFHIP_PROBE(4) AFHIP_PROBE(5) AFHIP_PROBE(6) AFHIP_PROBE(7) AFHIP_PROBE(8)
    }
#undef AFHIP_PROBE
    return hipGetLastError();
}
}  // namespace

hipError_t launch_gemv_probe(hipStream_t stream, int probe, int rows, float* dst, const float* input,
                             const uint8_t* weight_prepared, int in_dim, int out_dim, uint32_t* stamps, size_t stamps_bytes,
                             int* grid_out, int* waves_out) {
    if (in_dim > gemv_fused_max_in_dim() || probe < 0 || probe > 8) return hipErrorInvalidValue;
    switch (rows) {
        case 1: return launch_gemv_probe_rows<1>(stream, probe, dst, input, weight_prepared, in_dim, out_dim, stamps, stamps_bytes, grid_out, waves_out);
        case 2: return launch_gemv_probe_rows<2>(stream, probe, dst, input, weight_prepared, in_dim, out_dim, stamps, stamps_bytes, grid_out, waves_out);
        case 4: return launch_gemv_probe_rows<4>(stream, probe, dst, input, weight_prepared, in_dim, out_dim, stamps, stamps_bytes, grid_out, waves_out);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_gemv_argmax_keys(hipStream_t stream, int tensor_type, unsigned long long* keys, int* key_count,
                                   const float* input, const uint8_t* weight_prepared, int in_dim, int out_dim,
                                   const GemvTuning& tune) {
    if (in_dim > gemv_fused_max_in_dim() || keys == nullptr || key_count == nullptr) return hipErrorInvalidValue;
    const GemvTargets tg{nullptr, nullptr, weight_prepared, nullptr, 0, Epilogue{}, Epilogue{}};
    if (tensor_type == 2)
        return launch_fused<2, 1, false, true>(stream, tg, nullptr, input, in_dim, out_dim, tune, keys, key_count);
    return launch_fused<8, 1, false, true>(stream, tg, nullptr, input, in_dim, out_dim, tune, keys, key_count);
}

}  // namespace afhip
