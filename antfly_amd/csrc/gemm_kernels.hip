// Prefill GEMM (rows >= 9) on CDNA4 int8 MFMA, activation-quantized route
// (ops/native_compute.zig:13304-13478 for Q8_0, :23427-23775 for Q4_0):
//   dot[m][n][b] = sum_i qx[m][32b+i] * qw[n][32b+i]            (int32, exact)
//   y[m][n]      = sum_b (sx[m][b] * sw[n][b]) * f32(dot[m][n][b])
//
// Per 32x32 output tile and per pair of blocks (b, b+1) a wavefront issues
//   2 x v_mfma_i32_32x32x32_i8     the int32 dots of block b and of block b+1
//   1 x v_mfma_f32_32x32x1_2b_f32  the scale products sx[m][b]*sw[n][b] of both
//                                  blocks (two rank-1 outer products; each entry
//                                  is the correctly rounded f32 product)
// and then one int->float conversion and one fused multiply-add per element and
// block on the vector ALU.  All three results share the 32x32 MFMA register
// layout, so the epilogue is element-wise.  On this chip the vector ALU and the
// matrix pipe of a SIMD do not run these two halves side by side, so a pair costs
// their sum; everything else (global loads, LDS traffic, barriers) is arranged to
// hide behind that.
//
// Workgroup = kWavesM x kWavesN output tiles of 32x32, times kSplit wavefronts per
// tile that share the K loop: a stage holds 2*kSplit blocks and wavefront ks of a
// tile takes pair ks of every stage.  The kSplit partial sums of a tile are added
// in LDS at the end, in ks order (so y is a fixed-order sum of kSplit block-ascending
// partial sums).  Sixteen wavefronts per workgroup put four on every SIMD.
//
// Operands reach LDS without passing through registers: activations and Q8_0 weight
// bytes are fetched with global_load_lds_dwordx4 into a ring of kRing stages (4, or
// 3 for the widest stages), kRing - 1 stages ahead of the one being consumed.  One
// such load moves 64 x 16 bytes: whole 128-byte lines of kRowsPerLoad rows, with
// consecutive lanes on the chunks of one line (one cache-line lookup per eight
// lanes).  LDS holds a stage row-major with the 16-byte chunk index XOR-swizzled by
// the row, so that the MFMA fragment reads (one row per lane, same chunk column) of 16
// consecutive lanes hit 16 different bank groups.  Block scales arrive the same way
// (f32 activation scales as they are, fp16 weight scales zero-extended to 32 bits
// and converted when read).  Q4_0 nibble chunks land in a staging area of the slot
// and are expanded to int8 fragments by the wavefront that fetched them.
//
// MFMA operands: A = activations (row = lane % 32 -> m), B = weights (column =
// lane % 32 -> n); lane / 32 selects bytes [16*(lane/32), +16) of the block.
// Result register v of a lane is row 8*(v/4) + 4*(lane/32) + v%4, column
// lane % 32, so stores are 128 bytes contiguous along n.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdlib>

#include "device_common.h"
#include "gemv_common.h"
#include "qmatmul_launch.h"

namespace afhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int kWavesM, int kWavesN, int kSplit, bool kQ4>
struct GemmShape {
    static constexpr int kTiles = kWavesM * kWavesN;
    static constexpr int kWaves = kTiles * kSplit;
    static constexpr int kThreads = 64 * kWaves;
    static constexpr int kTM = 32 * kWavesM, kTN = 32 * kWavesN;
    static constexpr int kStageBlocks = 2 * kSplit;              // one pair per wavefront and stage
    static constexpr int kChunksPerRow = 2 * kStageBlocks;       // 16-byte chunks of int8 per row and stage
    static constexpr int kRowsPerLoad = 64 / kChunksPerRow;      // rows one 64-lane LDS load covers
    static constexpr int kGroupsA = kTM / kRowsPerLoad, kGroupsB = kTN / kRowsPerLoad;
    static constexpr int kABytes = kTM * kChunksPerRow * 16, kBBytes = kTN * kChunksPerRow * 16;
    // LDS keeps a stage of an operand row-major, [row][chunk], with the chunk index
    // XOR-swizzled by the row so that 16 consecutive rows reading the same chunk
    // column hit 16 different 16-byte bank groups (a row is 16 * kChunksPerRow bytes,
    // the banks wrap every 256 bytes).
    static constexpr int kRowsPerWrap = 16 / kChunksPerRow > 0 ? 16 / kChunksPerRow : 1;
    __device__ static constexpr int chunk_pos(int row, int chunk) {
        return row * kChunksPerRow + (chunk ^ ((row / kRowsPerWrap) % kChunksPerRow));
    }
    static_assert(kChunksPerRow == 4 || kChunksPerRow == 8 || kChunksPerRow == 16, "swizzle covers rows of 64..256 bytes");
    static constexpr int kSxBytes = kTM * kStageBlocks * 4, kSwBytes = kTN * kStageBlocks * 4;
    static constexpr int kRawBytes = kQ4 ? kTN * kStageBlocks * 16 : 0;  // Q4_0 nibble chunks as fetched
    static constexpr int kStageBytes = kABytes + kBBytes + kSxBytes + kSwBytes + kRawBytes;
    static constexpr int kReduceBytes = kSplit > 1 ? kSplit * kTM * kTN * 4 : 0;
    // LDS stages: loads run kRing - 1 stages ahead of the consumer
    static constexpr int kRing = 4 * kStageBytes <= 160 * 1024 ? 4 : 3;
    static constexpr int kLdsBytes = kRing * kStageBytes > kReduceBytes ? kRing * kStageBytes : kReduceBytes;
    static_assert(kSplit == 1 || kSplit == 2 || kSplit == 4 || kSplit == 8, "kSplit");
    static_assert(kThreads <= 1024, "workgroup size");
    static_assert(kTM % kRowsPerLoad == 0 && kTN % kRowsPerLoad == 0, "tile rows per load");
    static_assert(kLdsBytes <= 160 * 1024, "LDS");
};

// s_waitcnt for "at most n vector memory operations outstanding" (nothing else waited
// for).  n is wave-uniform; the instruction needs an immediate.
__device__ __forceinline__ void wait_vm_outstanding(int n) {
    // simm16: vmcnt[3:0] | expcnt << 4 | lgkmcnt << 8 | vmcnt[5:4] << 14
#define AFHIP_WAIT_VM(N) __builtin_amdgcn_s_waitcnt(((N) & 15) | (7 << 4) | (15 << 8) | (((N) >> 4) << 14))
    switch (n) {
        case 1: AFHIP_WAIT_VM(1); break;
        case 2: AFHIP_WAIT_VM(2); break;
        case 3: AFHIP_WAIT_VM(3); break;
        case 4: AFHIP_WAIT_VM(4); break;
        case 5: AFHIP_WAIT_VM(5); break;
        case 6: AFHIP_WAIT_VM(6); break;
        case 8: AFHIP_WAIT_VM(8); break;
        case 10: AFHIP_WAIT_VM(10); break;
        case 12: AFHIP_WAIT_VM(12); break;
        default: AFHIP_WAIT_VM(0); break;  // 0, or a count not listed: waiting for everything is always safe
    }
#undef AFHIP_WAIT_VM
}

// One 64-lane load from global memory straight into LDS: lane l's `bytes` at
// base + voff land at lds_addr + l * max(bytes, 4) (a 2-byte element is zero-extended
// to 4).  Issued as inline assembly on purpose: the compiler would otherwise make
// every later LDS read wait for all such loads in flight, which defeats the ring.
// Completion is tracked with wait_vm_outstanding(); base and lds_addr are wave-uniform.
// M0 is declared as clobbered, so the compiler keeps nothing of its own in it across these statements.
__device__ __forceinline__ void lds_load16(const void* base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_load4(const void* base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}
__device__ __forceinline__ void lds_load2(const void* base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_ushort %1, %2" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}

extern __shared__ __align__(16) unsigned char gemm_lds[];

// kShareK: this launch walks only a share of K per workgroup (see below); a template parameter
// so that the ordinary kernel carries none of it.
// kStamps (diagnostic): the kernel computes as usual but, instead of results, every wavefront stores eight
// 32-bit counts over the start of dst, [8 * (workgroup * wavefronts + wavefront)]: shader-clock cycles before
// the K loop, in it, waiting for its own loads, waiting at the workgroup barrier, 100 MHz reference ticks
// spent in the loop (cycles / ticks = the clock the chip held), cycles after the loop, 0, and the HW_ID register.
template <int kType, int kWavesM, int kWavesN, int kSplit, bool kWriteDots, bool kShareK = false, bool kStamps = false>
__device__ __forceinline__ void gemm_i8_body(
    float* __restrict__ dst, int* __restrict__ dots, const int8_t* __restrict__ qx, const float* __restrict__ sx,
    const uint8_t* __restrict__ weight, int rows, int in_dim, int out_dim, int m_tiles, int n_tiles,
    int share_blocks, float* __restrict__ partial, const Epilogue& ep) {
    using S = GemmShape<kWavesM, kWavesN, kSplit, kType == 2>;
    constexpr int kWaves = S::kWaves, kSB = S::kStageBlocks, kRPL = S::kRowsPerLoad, kCPR = S::kChunksPerRow;
    constexpr int kTM = S::kTM, kTN = S::kTN, kRing = S::kRing;
    constexpr int kQuantBytes = kType == 2 ? 16 : 32;
    constexpr bool kQ4 = kType == 2;
    // units of 64 lanes per stage, by kind
    constexpr int kUnitsA = S::kGroupsA;                          // LDS loads of activation bytes
    constexpr int kUnitsB = kQ4 ? kTN * kSB / 64 : S::kGroupsB;   // Q8_0: LDS loads; Q4_0: register loads of 16-byte nibble chunks
    constexpr int kUnitsSx = kTM * kSB / 64, kUnitsSw = kTN * kSB / 64;
    constexpr int kPerA = (kUnitsA + kWaves - 1) / kWaves, kPerB = (kUnitsB + kWaves - 1) / kWaves;
    constexpr int kPerSx = (kUnitsSx + kWaves - 1) / kWaves, kPerSw = (kUnitsSw + kWaves - 1) / kWaves;
    // each kind starts its round-robin over the wavefronts where the previous one stopped
    constexpr int kStartB = kUnitsA % kWaves, kStartSx = (kStartB + kUnitsB) % kWaves, kStartSw = (kStartSx + kUnitsSx) % kWaves;

    // K range of this workgroup: all of it, or (a small grid spread over more compute units)
    // share blockIdx.y of share_blocks blocks, whose sums go to partial[share][rows][out_dim]
    // for splitk_reduce_kernel.  kb_full is the row pitch, kb the blocks walked here.
    const int kb_full = in_dim >> 5;
    const int blk_begin = kShareK ? static_cast<int>(blockIdx.y) * share_blocks : 0;
    const int kb = kShareK ? min(share_blocks, kb_full - blk_begin) : kb_full;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ks = wave / S::kTiles, tile = wave % S::kTiles;
    const int wm = tile / kWavesN, wn = tile % kWavesN;
    const int lj = lane & 31, lh = lane >> 5;

    // Workgroups that share a weight tile (same n tile, different m tiles) sit on
    // the same XCD (consecutive workgroup ids go round-robin over the 8 XCDs), so
    // each L2 reads every weight byte once.
    const int id = blockIdx.x;
    const int xcd = id & 7, slot_id = id >> 3;
    const int m_tile = slot_id % m_tiles;
    const int n_tile = (slot_id / m_tiles) * 8 + xcd;
    if (n_tile >= n_tiles) return;
    const int m0 = m_tile * kTM, n0 = n_tile * kTN;

    const size_t blocks = static_cast<size_t>(out_dim) * kb_full;
    const uint8_t* a_base = reinterpret_cast<const uint8_t*>(qx) + static_cast<size_t>(m0) * in_dim + static_cast<size_t>(blk_begin) * 32;
    const uint8_t* b_base = weight + (static_cast<size_t>(n0) * kb_full + blk_begin) * kQuantBytes;
    const uint8_t* sx_base = reinterpret_cast<const uint8_t*>(sx + static_cast<size_t>(m0) * kb_full + blk_begin);
    const uint8_t* sw_base = weight + blocks * kQuantBytes + (static_cast<size_t>(n0) * kb_full + blk_begin) * 2;

    const int stages = (kb + kSB - 1) / kSB;
    const int last_blocks = kb - (stages - 1) * kSB;  // blocks in the last stage, 1..kSB

    // first unit of each kind this wavefront handles (then every kWaves-th)
    const int ua0 = wave;
    const int ub0 = (wave + kWaves - kStartB) % kWaves;
    const int usx0 = (wave + kWaves - kStartSx) % kWaves;
    const int usw0 = (wave + kWaves - kStartSw) % kWaves;
    int loads_per_stage = 0;
#pragma unroll
    for (int i = 0; i < kPerA; ++i) loads_per_stage += ua0 + i * kWaves < kUnitsA;
#pragma unroll
    for (int i = 0; i < kPerB; ++i) loads_per_stage += ub0 + i * kWaves < kUnitsB;
#pragma unroll
    for (int i = 0; i < kPerSx; ++i) loads_per_stage += usx0 + i * kWaves < kUnitsSx;
#pragma unroll
    for (int i = 0; i < kPerSw; ++i) loads_per_stage += usw0 + i * kWaves < kUnitsSw;

    // Per-lane byte offsets of the loads, for a full stage ([0]) and for the last
    // stage ([1], block indices clamped to the last valid block: nothing is read past
    // a row's end; the scales of the clamped blocks are written as zero).
    // LDS position p = lane of a 64-lane load is chunk slot p % kCPR of row p / kCPR:
    // eight (or more) consecutive lanes read one 128-byte line, in swizzled order.
    const int dma_r = lane / kCPR, dma_slot = lane % kCPR;
    uint32_t off_a[kPerA][2], off_b[kPerB][2], off_sx[kPerSx][2], off_sw[kPerSw][2];
    int lds_b4[kPerB][2];  // Q4_0: LDS chunk positions of the low- and high-nibble halves
    auto dma_chunk_last = [&](int c) { return min(c >> 1, last_blocks - 1) * 2 + (c & 1); };
#pragma unroll
    for (int i = 0; i < kPerA; ++i) {
        const int r = min((ua0 + i * kWaves) * kRPL + dma_r, kTM - 1);
        const int c = dma_slot ^ ((r / S::kRowsPerWrap) % kCPR);
        const uint32_t rowoff = static_cast<uint32_t>(min(m0 + r, rows - 1) - m0) * static_cast<uint32_t>(in_dim);
        off_a[i][0] = rowoff + c * 16;
        off_a[i][1] = rowoff + dma_chunk_last(c) * 16;
    }
#pragma unroll
    for (int i = 0; i < kPerB; ++i) {
        if (kQ4) {
            const int q = min((ub0 + i * kWaves) * 64 + lane, kTN * kSB - 1);
            const int r = q / kSB, blk = q % kSB;
            const uint32_t rowoff = static_cast<uint32_t>(min(n0 + r, out_dim - 1) - n0) * static_cast<uint32_t>(kb_full) * 16u;
            off_b[i][0] = rowoff + blk * 16;
            off_b[i][1] = rowoff + min(blk, last_blocks - 1) * 16;
            lds_b4[i][0] = S::chunk_pos(r, 2 * blk);
            lds_b4[i][1] = S::chunk_pos(r, 2 * blk + 1);
        } else {
            const int r = min((ub0 + i * kWaves) * kRPL + dma_r, kTN - 1);
            const int c = dma_slot ^ ((r / S::kRowsPerWrap) % kCPR);
            const uint32_t rowoff = static_cast<uint32_t>(min(n0 + r, out_dim - 1) - n0) * static_cast<uint32_t>(kb_full) * 32u;
            off_b[i][0] = rowoff + c * 16;
            off_b[i][1] = rowoff + dma_chunk_last(c) * 16;
            lds_b4[i][0] = lds_b4[i][1] = 0;
        }
    }
#pragma unroll
    for (int i = 0; i < kPerSx; ++i) {
        const int q = min((usx0 + i * kWaves) * 64 + lane, kTM * kSB - 1);
        const int r = q / kSB, blk = q % kSB;
        const uint32_t rowoff = static_cast<uint32_t>(min(m0 + r, rows - 1) - m0) * static_cast<uint32_t>(kb_full);
        off_sx[i][0] = (rowoff + blk) * 4;
        off_sx[i][1] = (rowoff + min(blk, last_blocks - 1)) * 4;
    }
#pragma unroll
    for (int i = 0; i < kPerSw; ++i) {
        const int q = min((usw0 + i * kWaves) * 64 + lane, kTN * kSB - 1);
        const int r = q / kSB, blk = q % kSB;
        const uint32_t rowoff = static_cast<uint32_t>(min(n0 + r, out_dim - 1) - n0) * static_cast<uint32_t>(kb_full);
        off_sw[i][0] = (rowoff + blk) * 2;
        off_sw[i][1] = (rowoff + min(blk, last_blocks - 1)) * 2;
    }

    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(gemm_lds)));
    constexpr int kOffB = S::kABytes, kOffSx = kOffB + S::kBBytes, kOffSw = kOffSx + S::kSxBytes, kOffRaw = kOffSw + S::kSwBytes;
    auto stage_ptr = [&](int slot) { return gemm_lds + slot * S::kStageBytes; };

    // Issues every load of stage `st` (clamped to the last stage) towards ring slot `slot`.
    auto issue_loads = [&](int slot, int st) {
        const int se = min(st, stages - 1);
        const int sel = se == stages - 1 ? 1 : 0;
        const uint32_t sp = lds_base + slot * S::kStageBytes;
#pragma unroll
        for (int i = 0; i < kPerA; ++i) {
            const int u = ua0 + i * kWaves;
            if (u < kUnitsA) lds_load16(a_base + static_cast<size_t>(se) * (kSB * 32), off_a[i][sel], sp + u * 1024);
        }
#pragma unroll
        for (int i = 0; i < kPerB; ++i) {
            const int u = ub0 + i * kWaves;
            if (u < kUnitsB)
                lds_load16(b_base + static_cast<size_t>(se) * (kSB * kQuantBytes), off_b[i][sel],
                           sp + (kQ4 ? kOffRaw + u * 1024 : kOffB + u * 1024));
        }
#pragma unroll
        for (int i = 0; i < kPerSx; ++i) {
            const int u = usx0 + i * kWaves;
            if (u < kUnitsSx) lds_load4(sx_base + static_cast<size_t>(se) * (kSB * 4), off_sx[i][sel], sp + kOffSx + u * 256);
        }
#pragma unroll
        for (int i = 0; i < kPerSw; ++i) {
            const int u = usw0 + i * kWaves;
            if (u < kUnitsSw) lds_load2(sw_base + static_cast<size_t>(se) * (kSB * 2), off_sw[i][sel], sp + kOffSw + u * 256);
        }
    };

    // Q4_0: expands the nibble chunks this wavefront fetched for ring slot `slot` into
    // int8 fragments (its own loads have landed: no other wavefront is involved).
    auto expand_q4 = [&](int slot) {
        if (!kQ4) return;
        unsigned char* sp = stage_ptr(slot);
        const int4* raw = reinterpret_cast<const int4*>(sp + kOffRaw);
        int4* bs = reinterpret_cast<int4*>(sp + kOffB);
#pragma unroll
        for (int i = 0; i < kPerB; ++i) {
            const int u = ub0 + i * kWaves;
            if (u < kUnitsB) {
                const int4 r = raw[u * 64 + lane];
                const uint32_t p[4] = {static_cast<uint32_t>(r.x), static_cast<uint32_t>(r.y), static_cast<uint32_t>(r.z), static_cast<uint32_t>(r.w)};
                int v[8];
                unpack_q4(p, v);  // low nibbles = values 0..15 (half 0), high nibbles = 16..31 (half 1)
                bs[lds_b4[i][0]] = make_int4(v[0], v[1], v[2], v[3]);
                bs[lds_b4[i][1]] = make_int4(v[4], v[5], v[6], v[7]);
            }
        }
    };

    // this lane's fragment positions (loop-invariant; only the ring slot changes)
    const int row = wm * 32 + lj;  // activation row (A operand) inside the tile
    const int col = wn * 32 + lj;  // weight column (B operand) inside the tile
    const int b0 = 2 * ks;         // first block of this wavefront's pair inside a stage
    const int frag_a0 = S::chunk_pos(row, 2 * b0 + lh), frag_a1 = S::chunk_pos(row, 2 * b0 + 2 + lh);
    const int frag_b0 = S::chunk_pos(col, 2 * b0 + lh), frag_b1 = S::chunk_pos(col, 2 * b0 + 2 + lh);
    const int frag_sx = row * kSB + b0 + lh;  // lanes 0-31 carry block b0, lanes 32-63 block b0 + 1
    const int frag_sw = col * kSB + b0 + lh;

    v16f acc = {};

    // MFMA operands of one stage as read from LDS (scales still raw)
    struct Frag {
        int4 a0, a1, w0, w1;
        float ta;
        uint32_t tb;  // fp16 bits
    };
    auto read_frag = [&](int slot, Frag& f) {
        const unsigned char* sp = stage_ptr(slot);
        const int4* as = reinterpret_cast<const int4*>(sp);
        const int4* bs = reinterpret_cast<const int4*>(sp + kOffB);
        f.a0 = as[frag_a0];
        f.a1 = as[frag_a1];
        f.w0 = bs[frag_b0];
        f.w1 = bs[frag_b1];
        f.ta = reinterpret_cast<const float*>(sp + kOffSx)[frag_sx];
        f.tb = reinterpret_cast<const uint32_t*>(sp + kOffSw)[frag_sw];
    };
    // One pair of blocks, first block `blk` (absolute index): MFMAs of block blk and of
    // the scale products, vector-ALU work of block blk, then the same for block blk + 1 in
    // the registers block blk's dots have left (the two halves of a wavefront's work do
    // not overlap anyway, and 16 registers fewer are live).  `between` runs after the
    // last MFMA has been issued: the operand registers are free from there on.
    auto pair_step = [&](const Frag& f, int blk, auto&& between) {
        // blocks past the end of K (clamped re-reads of the last block) get scale 0
        const bool live = blk + lh < kb;
        const float ta = live ? f.ta : 0.0f;
        const float tb = live ? half_bits_to_f32(static_cast<uint16_t>(f.tb)) : 0.0f;
        const v4i a0 = {f.a0.x, f.a0.y, f.a0.z, f.a0.w}, a1 = {f.a1.x, f.a1.y, f.a1.z, f.a1.w};
        const v4i w0 = {f.w0.x, f.w0.y, f.w0.z, f.w0.w}, w1 = {f.w1.x, f.w1.y, f.w1.z, f.w1.w};
        const v16i zi = {};
        const v32f zf = {};
        const int n = n0 + col;
        v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, w0, zi, 0, 0, 0);
        v32f t = __builtin_amdgcn_mfma_f32_32x32x1f32(ta, tb, zf, 0, 0, 0);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            if (kWriteDots && blk + h < kb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                    if (m < rows && n < out_dim) dots[(static_cast<size_t>(m) * out_dim + n) * kb_full + blk_begin + blk + h] = c[v];
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[v] = __builtin_fmaf(t[16 * h + v], static_cast<float>(c[v]), acc[v]);
            if (h == 0) {
                // compiler fence (no instruction): block blk is finished before block blk + 1 starts
                asm volatile("" : "+v"(acc), "+v"(t) : : "memory");
                c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, w1, zi, 0, 0, 0);
                between();
            }
        }
    };
    // Program-order fence for the compiler (it emits no instruction): a stage's arithmetic
    // is emitted before it.  Without it the optimizer gathers the MFMAs of several stages
    // in one place and spills their results.
    auto pin_acc = [&]() { asm volatile("" : "+v"(acc) : : "memory"); };

    uint64_t stamp_begin = 0, stamp_loop = 0, stamp_tail = 0, ref_loop = 0, ref_tail = 0, stamp_wait = 0, stamp_barrier = 0;
    if (kStamps) stamp_begin = __builtin_readcyclecounter();
    // ---- prologue: stages 0 .. kRing-2 in flight, stages 0 and 1 landed, stage 0 in registers
    static_assert(kRing == 4, "the loop reads stage st + 1 while stage st + 2 lands and stage st + 3 is issued");
#pragma unroll
    for (int d = 0; d < kRing - 1; ++d) issue_loads(d, d);
    // Loads complete in order: a stage has landed for this wavefront once at most the
    // loads of the stages issued after it are outstanding.
    wait_vm_outstanding(loads_per_stage);
    expand_q4(0);
    expand_q4(1);
    __syncthreads();
    {
        // The next stage's operands are read from LDS while this stage's arithmetic runs.
        Frag frag[2];
        read_frag(0, frag[0]);
        if (kStamps) {
            stamp_loop = __builtin_readcyclecounter();
            ref_loop = __builtin_amdgcn_s_memrealtime();
        }
        for (int st0 = 0; st0 < stages; st0 += kRing) {
#pragma unroll
            for (int d = 0; d < kRing; ++d) {
                const int st = st0 + d;  // may run past `stages` in the last round: zero scales, no effect
                // the slot of stage st - 1 is free (its fragments were read a stage ago): refill it, kRing - 1 stages ahead
                issue_loads((d + kRing - 1) % kRing, st + kRing - 1);
                // the next stage's operands landed before the last barrier
                pair_step(frag[d & 1], st * kSB + b0, [&]() { read_frag((d + 1) % kRing, frag[(d + 1) & 1]); });
                pin_acc();
                // stage st + 2 (issued two stages ago) has to be complete before the barrier:
                // the next stage reads its operands
                uint64_t s0 = 0, s1 = 0;
                if (kStamps) s0 = __builtin_readcyclecounter();
                wait_vm_outstanding(loads_per_stage);
                expand_q4((d + 2) % kRing);
                if (kStamps) s1 = __builtin_readcyclecounter();
                __syncthreads();
                if (kStamps) {
                    stamp_wait += s1 - s0;
                    stamp_barrier += __builtin_readcyclecounter() - s1;
                }
            }
        }
    }
    if (kStamps) {
        stamp_tail = __builtin_readcyclecounter();
        ref_tail = __builtin_amdgcn_s_memrealtime();
    }

    // Loads still in flight target ring slots nobody reads again; they must land before
    // the ring is reused for the reduction (and before the workgroup ends).
    wait_vm_outstanding(0);
    const int n = n0 + col;
    if (kSplit > 1) {
        // ---- the kSplit partial sums of a tile meet in LDS
        __syncthreads();
        float* red = reinterpret_cast<float*>(gemm_lds);  // [ks][tile][v][lane]
#pragma unroll
        for (int v = 0; v < 16; ++v) red[((ks * S::kTiles + tile) * 16 + v) * 64 + lane] = acc[v];
        __syncthreads();
        if (dst == nullptr) return;
        constexpr int kPer = 16 / kSplit;
#pragma unroll
        for (int j = 0; j < kPer; ++j) {
            const int v = ks * kPer + j;
            float sum = red[(tile * 16 + v) * 64 + lane];
#pragma unroll
            for (int k2 = 1; k2 < kSplit; ++k2) sum += red[((k2 * S::kTiles + tile) * 16 + v) * 64 + lane];
            const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (kStamps) {
                asm volatile("" : : "v"(sum));  // the sum is formed, not stored
            } else if (m < rows && n < out_dim) {
                const size_t at = static_cast<size_t>(m) * out_dim + n;
                if (kShareK) partial[static_cast<size_t>(blockIdx.y) * rows * out_dim + at] = sum;
                else dst[at] = finish_output(ep, n, at, sum);
            }
        }
        if (kStamps && lane == 0) {
            const uint64_t stamp_end = __builtin_readcyclecounter();
            int* out = reinterpret_cast<int*>(dst) + 8 * (static_cast<size_t>(blockIdx.x) * kWaves + wave);
            out[0] = static_cast<int>(stamp_loop - stamp_begin);
            out[1] = static_cast<int>(stamp_tail - stamp_loop);
            out[2] = static_cast<int>(stamp_wait);
            out[3] = static_cast<int>(stamp_barrier);
            out[4] = static_cast<int>(ref_tail - ref_loop);
            out[5] = static_cast<int>(stamp_end - stamp_tail);
            out[6] = 0;
            out[7] = static_cast<int>(__builtin_amdgcn_s_getreg((31 << 11) | 4));
        }
    } else {
        if (dst == nullptr) return;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (m < rows && n < out_dim) {
                const size_t at = static_cast<size_t>(m) * out_dim + n;
                if (kShareK) partial[static_cast<size_t>(blockIdx.y) * rows * out_dim + at] = acc[v];
                else dst[at] = finish_output(ep, n, at, acc[v]);
            }
        }
    }
}

template <int kType, int kWavesM, int kWavesN, int kSplit, bool kWriteDots, bool kShareK = false, bool kStamps = false>
__global__ __launch_bounds__(64 * kWavesM * kWavesN * kSplit) void gemm_i8_kernel(
    float* __restrict__ dst, int* __restrict__ dots, const int8_t* __restrict__ qx, const float* __restrict__ sx,
    const uint8_t* __restrict__ weight, int rows, int in_dim, int out_dim, int m_tiles, int n_tiles,
    int share_blocks, float* __restrict__ partial, Epilogue ep) {
    gemm_i8_body<kType, kWavesM, kWavesN, kSplit, kWriteDots, kShareK, kStamps>(dst, dots, qx, sx, weight, rows, in_dim, out_dim,
                                                                                 m_tiles, n_tiles, share_blocks, partial, ep);
}

namespace {

template <int kType, int kWavesM, int kWavesN, int kSplit>
hipError_t launch_tile(hipStream_t stream, float* dst, int* dots, const int8_t* qx, const float* sx,
                       const uint8_t* weight, int rows, int in_dim, int out_dim, const Epilogue& ep, float* partial) {
    using S = GemmShape<kWavesM, kWavesN, kSplit, kType == 2>;
    const int m_tiles = (rows + S::kTM - 1) / S::kTM;
    const int n_tiles = (out_dim + S::kTN - 1) / S::kTN;
    const int n_groups = (n_tiles + 7) / 8;
    const long long grid = static_cast<long long>(n_groups) * m_tiles * 8;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    // per-lane load offsets are 32-bit, relative to the workgroup's first row
    if (static_cast<long long>(S::kTM > S::kTN ? S::kTM : S::kTN) * in_dim > 0x7fffffffLL) return hipErrorInvalidValue;
    // K shares: only with room for their partial sums, never for the block-dot output
    const int kb = in_dim / 32;
    const int splits = partial != nullptr && dots == nullptr ? gemm_i8_splits(rows, in_dim, out_dim) : 1;
    const int share_blocks = (kb + splits - 1) / splits;
    const int shares = (kb + share_blocks - 1) / share_blocks;  // no empty share
    float* sums = shares > 1 ? partial : nullptr;
    dim3 g(static_cast<unsigned>(grid), static_cast<unsigned>(shares)), b(S::kThreads);
    auto kernel_f32 = gemm_i8_kernel<kType, kWavesM, kWavesN, kSplit, false>;
    auto kernel_shares = gemm_i8_kernel<kType, kWavesM, kWavesN, kSplit, false, true>;
    auto kernel_dots = gemm_i8_kernel<kType, kWavesM, kWavesN, kSplit, true>;
    // more than 64 KB of LDS has to be asked for once per kernel
    static std::atomic<bool> attr_done{false};
    const hipError_t attr = attr_done.load(std::memory_order_acquire) ? hipSuccess : [&]() {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel_f32),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, S::kLdsBytes);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel_shares), hipFuncAttributeMaxDynamicSharedMemorySize,
                                S::kLdsBytes);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel_dots), hipFuncAttributeMaxDynamicSharedMemorySize,
                                S::kLdsBytes);
        if (e == hipSuccess) attr_done.store(true, std::memory_order_release);  // a failure is not remembered: the next call tries again
        return e;
    }();
    if (attr != hipSuccess) return attr;
    if (dots)
        hipLaunchKernelGGL(kernel_dots, g, b, S::kLdsBytes, stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim,
                           m_tiles, n_tiles, share_blocks, sums, ep);
    else if (shares > 1)
        hipLaunchKernelGGL(kernel_shares, g, b, S::kLdsBytes, stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim,
                           m_tiles, n_tiles, share_blocks, sums, ep);
    else
        hipLaunchKernelGGL(kernel_f32, g, b, S::kLdsBytes, stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim,
                           m_tiles, n_tiles, share_blocks, sums, ep);
    if (hipError_t e = hipGetLastError(); e != hipSuccess || shares == 1) return e;
    return launch_splitk_reduce(stream, dst, sums, static_cast<size_t>(rows) * out_dim, out_dim, shares, ep);
}

template <int kType>
hipError_t launch_type(hipStream_t stream, float* dst, int* dots, const int8_t* qx, const float* sx,
                       const uint8_t* weight, int rows, int in_dim, int out_dim, const Epilogue& ep, float* partial) {
    // 64 x 128 tiles while they still give every CU a workgroup, 32 x 64 with a deeper K split otherwise
    const long long big = static_cast<long long>((rows + 63) / 64) * ((out_dim + 127) / 128);
    static const char* force = std::getenv("AFHIP_GEMM_TILE");  // tuning: "L" = 64x128, "S" = 32x64
    const bool use_big = force ? force[0] != 'S' : big >= 256;
    if (use_big) return launch_tile<kType, 2, 4, 2>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim, ep, partial);
    return launch_tile<kType, 1, 2, 4>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim, ep, partial);
}

}  // namespace

// K shares of a GEMM launch: one when its 32 x 64 tiles fill the compute units anyway, else as
// many (a power of two, at most eight, at least 16 blocks = two stages each) as spread it over them.
int gemm_i8_splits(int rows, int in_dim, int out_dim) {
    const long workgroups = static_cast<long>((rows + 31) / 32) * ((out_dim + 63) / 64);
    const int kb = in_dim / 32;
    const int units = gemv_compute_units();
    int splits = 1;
    while (splits < 8 && workgroups * splits * 2 <= units && kb / (splits * 2) >= 16) splits *= 2;
    return splits;
}

size_t gemm_i8_partial_bytes(size_t rows, size_t in_dim, size_t out_dim) {
    if (rows == 0 || rows > 0x7fffffff || in_dim > 0x7fffffff || out_dim > 0x7fffffff) return 0;
    const int splits = gemm_i8_splits(static_cast<int>(rows), static_cast<int>(in_dim), static_cast<int>(out_dim));
    return splits > 1 ? static_cast<size_t>(splits) * rows * out_dim * 4 : 0;
}

// dst = epilogue(sum over the K shares, in order): second kernel of a split-K launch.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(float* __restrict__ dst, const float* __restrict__ partial,
                                                            size_t count, int out_dim, int splits, Epilogue ep) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < count;
         i += static_cast<size_t>(gridDim.x) * blockDim.x) {
        float total = 0.0f;
        for (int z = 0; z < splits; ++z) total += partial[static_cast<size_t>(z) * count + i];
        dst[i] = finish_output(ep, static_cast<int>(i % out_dim), i, total);
    }
}

hipError_t launch_splitk_reduce(hipStream_t stream, float* dst, const float* partial, size_t count, int out_dim, int shares,
                                const Epilogue& ep) {
    size_t grid = (count + 255) / 256;
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, dst, partial, count, out_dim,
                       shares, ep);
    return hipGetLastError();
}

// Diagnostic: the Q8_0 64 x 128 tile kernel with its clock readings in place of results (see kStamps); dst has to
// hold 8 ints per wavefront of the grid, which it does whenever it holds the rows x out_dim results.
hipError_t launch_gemm_i8_stamps(hipStream_t stream, float* dst, const int8_t* qx, const float* sx, const uint8_t* weight,
                                 int rows, int in_dim, int out_dim) {
    using S = GemmShape<2, 4, 2, false>;
    const int m_tiles = (rows + S::kTM - 1) / S::kTM, n_tiles = (out_dim + S::kTN - 1) / S::kTN;
    const long long grid = static_cast<long long>((n_tiles + 7) / 8) * m_tiles * 8;
    if (grid > 0x7fffffffLL || static_cast<long long>(S::kTN) * in_dim > 0x7fffffffLL) return hipErrorInvalidValue;
    if (static_cast<long long>(rows) * out_dim < grid * S::kWaves * 8) return hipErrorInvalidValue;
    auto kernel = gemm_i8_kernel<8, 2, 4, 2, false, false, true>;
    if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           S::kLdsBytes);
        e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(S::kThreads), S::kLdsBytes, stream, dst, nullptr, qx, sx,
                       weight, rows, in_dim, out_dim, m_tiles, n_tiles, in_dim / 32, nullptr, Epilogue{});
    return hipGetLastError();
}

hipError_t launch_gemm_i8(hipStream_t stream, int tensor_type, float* dst, int* dots, const int8_t* qx, const float* sx,
                          const uint8_t* weight_prepared, int rows, int in_dim, int out_dim, const Epilogue& ep, float* partial) {
    if (tensor_type == 2) return launch_type<2>(stream, dst, dots, qx, sx, weight_prepared, rows, in_dim, out_dim, ep, partial);
    return launch_type<8>(stream, dst, dots, qx, sx, weight_prepared, rows, in_dim, out_dim, ep, partial);
}

}  // namespace afhip
