// Batched decode (a few to 128 rows) on CDNA4 int8 MFMA, activation-quantized route
// (ops/native_compute.zig:13304-13478 for Q8_0, :23427-23775 for Q4_0):
//   dot[m][n][b] = sum_i qx[m][32b+i] * qw[n][32b+i]            (int32, exact)
//   y[m][n]      = sum_b (sx[m][b] * sw[n][b]) * f32(dot[m][n][b])
//
// With so few rows the weights are read once and nothing is reused across workgroups, so the
// kernel is built like the decode GEMV, not like the prefill GEMM: single shot, no ring, no
// barrier inside the K loop.
//   * A workgroup of eight wavefronts owns 32 output columns and one share of K of at most
//     8 * kWaveBlocks blocks; wavefront w owns kWaveBlocks consecutive blocks of it (16 Q4_0 /
//     8 Q8_0: 8 KB of quant bytes).  It requests ALL its weight bytes at once with eight
//     global_load_lds_dwordx4 into its own 8 KB of LDS -- whole 128-byte lines, eight lanes per
//     line, chunk slots XOR-swizzled by the column so that the later fragment reads of 16
//     consecutive columns hit 16 different bank groups.  The LDS region is private to the
//     wavefront: no barrier before it is read.
//   * The activations were quantized beforehand into MFMA operand order
//     (quantize_fragments_kernel): the A fragment of 32 rows and one block is 1 KB contiguous,
//     lane l holding bytes [16 * (l / 32), +16) of row l % 32, so a wavefront takes it with one
//     coalesced 16-byte load per lane, straight into registers.  Rows past `rows` are zeros.
//   * Per block: v_mfma_i32_32x32x32_i8 gives the 32 x 32 int32 dots.  Q4_0 nibbles never become
//     separate bytes: with bit 3 flipped and placed in the high half of a byte a nibble n reads as
//     the int8 16 * (n - 8) (three operations per dword), so the MFMA yields 16 * dot exactly and
//     the weight scale is taken times 1/16 (a power of two: exact).  The scale products
//     sx[m][b] * sw[n][b] of two blocks come from one v_mfma_f32_32x32x1_2b_f32 (two rank-1
//     products, each entry the correctly rounded f32 product), then one convert and one fused
//     multiply-add per live result register and block.  Only the registers of rows that exist
//     are touched (kLive of 16: 4 for up to 8 rows, 8 for up to 16, ...).
//   * The eight wavefronts' sums meet in LDS in wavefront order (y is a fixed-order sum of eight
//     block-ascending partial sums); K shares of a long K go to partial[share][rows][out_dim]
//     and splitk_reduce_kernel adds them in share order.
//   * Up to eight rows (Q8_0: sixteen, as two groups of eight) on a K of whole 256-value runs take
//     batch8_mfma_kernel (further down): the 16x16x64 MFMA on two blocks at once, tiles of 8 .. 64
//     columns, weights requested two stages ahead instead of all at once, a long K in at most two
//     shares where that is possible.
//   * Nine to 64 rows whose 64-column tiles times K shares make a grid of five eighths to all of
//     the compute units take batch32_mfma_kernel (further down): this kernel's arithmetic, staged
//     weight requests, one workgroup per compute unit.
#include <hip/hip_runtime.h>

#include <atomic>

#include <cstdlib>
#include <type_traits>

#include "device_common.h"
#include "gemv_common.h"
#include "qmatmul_launch.h"

namespace afhip {

namespace {

typedef int bm_v4i __attribute__((ext_vector_type(4)));
typedef int bm_v16i __attribute__((ext_vector_type(16)));
typedef float bm_v32f __attribute__((ext_vector_type(32)));

constexpr int kBmWaves = 8;
constexpr int kBmThreads = 64 * kBmWaves;
constexpr int kBmWaveBytes = 8192;  // quant bytes one wavefront owns: 32 columns x kWaveBlocks blocks
constexpr int kBmLdsBytes = kBmWaves * kBmWaveBytes;

template <int kType>
struct BmFormat {
    static constexpr int kQuantBytes = kType == 2 ? 16 : 32;
    static constexpr int kWaveBlocks = kBmWaveBytes / (32 * kQuantBytes);  // 16 (Q4_0) / 8 (Q8_0)
    static constexpr int kShareBlocks = kBmWaves * kWaveBlocks;            // 128 / 64
};

// One 64-lane load from global memory straight into LDS: lane l's 16 bytes at base + voff land
// at lds_addr + 16 * l.  Inline assembly: the compiler does not track these loads, which is why
// the kernel waits for them by hand before anything reads the LDS region.
__device__ __forceinline__ void bm_lds_load16(const void* base, uint32_t voff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" : : "s"(lds_addr), "v"(voff), "s"(base) : "memory", "m0");
}

extern __shared__ __align__(16) unsigned char bm_lds[];

// the second matrix of a pair launch (grid.z == 2)
struct BmSecond {
    float* dst;
    const uint8_t* weight;
    Epilogue ep;
};

// Program-order fence for the compiler (no instruction): what was computed into `a` so far is
// finished before anything behind the fence starts.  Keeps the scheduler from running the MFMAs of
// several blocks ahead and holding all their results in registers.
__device__ __forceinline__ void fence_registers(float (&a)[4]) {
    asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]));
}
__device__ __forceinline__ void fence_registers(float (&a)[8]) {
    asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
}
__device__ __forceinline__ void fence_registers(float (&a)[12]) {
    asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(a[8]),
                 "+v"(a[9]), "+v"(a[10]), "+v"(a[11]));
}
__device__ __forceinline__ void fence_registers(float (&a)[16]) {
    asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(a[8]),
                 "+v"(a[9]), "+v"(a[10]), "+v"(a[11]), "+v"(a[12]), "+v"(a[13]), "+v"(a[14]), "+v"(a[15]));
}

}  // namespace

// X f32 [rows][in_dim] -> qa: [row tile][block][64 lanes][16 bytes] (lane = 32 * half + row % 32:
// bytes [16 * half, +16) of the block's 32 int8), sa: f32 [block][32 * row_tiles].  Rows past
// `rows` get zeros and scale 0.  Eight lanes per block as in quantize_activations_kernel
// (ops/native_compute.zig:11998-12028): same scale, reciprocal and rounding, bit for bit.
// kByteOrder (Q4_0 operands of batch32_mfma_kernel): within a block the lane half h holds the dwords
// x[8h..8h+3], x[16+8h..+3], x[8h+4..8h+7], x[16+8h+4..+7] instead of x[16h..16h+15] -- the values whose
// nibbles share the bytes [8 h, 8 h + 8) of the weight block, so that a lane unpacks whole bytes.
// zero_a (and zero_b): result arrays of zero_count floats that the matmul launch behind this one adds its two K shares'
// sums to; cleared here, by the launch that has to run first anyway.
template <bool kByteOrder>
__global__ __launch_bounds__(256) void quantize_fragments_kernel(const float* __restrict__ x, int rows, int in_dim, int row_tiles,
                                                                  uint32_t* __restrict__ qa, float* __restrict__ sa,
                                                                  float* __restrict__ zero_a, float* __restrict__ zero_b, size_t zero_count) {
    const int units_per_row = in_dim >> 2, kb = in_dim >> 5, padded = row_tiles * 32;
    const size_t units = static_cast<size_t>(padded) * units_per_row;
    if (zero_a != nullptr) {
        for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < zero_count; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
            zero_a[i] = 0.0f;
            if (zero_b != nullptr) zero_b[i] = 0.0f;
        }
    }
    for (size_t u = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; u < units;
         u += static_cast<size_t>(gridDim.x) * blockDim.x) {
        const int r = static_cast<int>(u / units_per_row), c4 = static_cast<int>(u % units_per_row);
        const int b = c4 >> 3, j = c4 & 7;
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (r < rows) v = reinterpret_cast<const float4*>(x)[static_cast<size_t>(r) * units_per_row + c4];
        float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        m = max_over_8(m);
        const float s = act_scale(m);
        const float inv = m == 0.0f ? 0.0f : 1.0f / s;
        const int q0 = act_quant(v.x, inv), q1 = act_quant(v.y, inv);
        const int q2 = act_quant(v.z, inv), q3 = act_quant(v.w, inv);
        const int half = kByteOrder ? (j >> 1) & 1 : j >> 2, dw = kByteOrder ? 2 * (j & 1) + (j >> 2) : j & 3;
        const size_t lane_entry = (static_cast<size_t>(r >> 5) * kb + b) * 64 + half * 32 + (r & 31);
        qa[lane_entry * 4 + dw] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
        if (j == 0) sa[static_cast<size_t>(b) * padded + r] = r < rows ? s : 0.0f;
    }
}

template <int kType, int kRowTiles, int kLive>
__global__ __launch_bounds__(kBmThreads, kRowTiles == 1 ? 4 : 2) void batch_mfma_kernel(float* __restrict__ dst_a, float* __restrict__ partial_a,
                                                                  const uint32_t* __restrict__ qa, const float* __restrict__ sa,
                                                                  const uint8_t* __restrict__ weight_a, int rows, int in_dim,
                                                                  int out_dim, int share_blocks, Epilogue ep_a, BmSecond second, int accumulate) {
    using F = BmFormat<kType>;
    // blockIdx.z == 1: the second matrix of a pair (same X, same shape)
    const bool is_b = blockIdx.z != 0;
    float* dst = is_b ? second.dst : dst_a;
    const uint8_t* weight = is_b ? second.weight : weight_a;
    const Epilogue ep = is_b ? second.ep : ep_a;
    float* partial = partial_a == nullptr ? nullptr : partial_a + (is_b ? static_cast<size_t>(gridDim.y) * rows * out_dim : 0);
    constexpr int kQB = F::kQuantBytes, kWB = F::kWaveBlocks, kPairs = kWB / 2;
    constexpr int kAhead = kRowTiles == 1 ? 8 : (kRowTiles == 2 ? 4 : 2);  // A fragments in registers per row tile
    static_assert(kWB % kAhead == 0 && kAhead % 2 == 0, "fragment ring");
    const int kb_full = in_dim >> 5;
    const int padded = kRowTiles * 32;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lj = lane & 31, lh = lane >> 5;
    const int n0 = blockIdx.x * 32;
    // blocks of this wavefront: [blk0, blk0 + nb), nb in 0..kWB; indices past the end are clamped
    // to the last valid block for every load and their scale products are forced to zero
    const int share_begin = static_cast<int>(blockIdx.y) * share_blocks;
    const int share_end = min(share_begin + share_blocks, kb_full);
    const int blk0 = share_begin + wave * kWB;
    const int nb = max(0, min(kWB, share_end - blk0));
    const int last = blk0 + max(nb, 1) - 1 < kb_full ? blk0 + max(nb, 1) - 1 : kb_full - 1;  // a valid block whatever nb is
    auto clamp_blk = [&](int j) { return min(blk0 + j, last); };

    const size_t blocks_total = static_cast<size_t>(out_dim) * kb_full;
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(bm_lds))) + wave * kBmWaveBytes;

    // ---- 1. loads.  Order matters: a wavefront's loads complete in the order they were issued,
    // and every wavefront of the grid issues at once, so memory serves all first halves before all
    // second halves.  First half of the weights (LDS-direct, four 1 KB loads), then what the first
    // half of the K loop needs (A fragments, scales), then values only the second half needs, then
    // the second half of the weights.  The compiler counts only its own loads when it waits for
    // one: with at least four of its loads issued behind everything the first half needs, its
    // wait lets exactly the four youngest loads -- the second half of the weights -- stay in flight
    // while the first half is computed.  (Its count can only be too strict, never too lax: loads
    // it does not know of only add to the number outstanding.)
    auto issue_weights = [&](int hb) {
        const uint8_t* wbase = weight + static_cast<size_t>(n0) * kb_full * kQB;
        const int c8 = lane >> 3, slot = lane & 7;
#pragma unroll
        for (int cg = 0; cg < 4; ++cg) {
            const int c = 8 * cg + c8;
            const int chunk = slot ^ ((c >> 1) & 7);
            const int cc = min(n0 + c, out_dim - 1) - n0;
            uint32_t off;
            if (kType == 2) {
                off = (static_cast<uint32_t>(cc) * kb_full + clamp_blk(8 * hb + chunk)) * 16u;
            } else {
                off = (static_cast<uint32_t>(cc) * kb_full + clamp_blk(4 * hb + (chunk >> 1))) * 32u + (chunk & 1) * 16u;
            }
            bm_lds_load16(wbase, off, lds_wave + (hb * 4 + cg) * 1024);
        }
    };
    issue_weights(0);

    // Rows that exist live in the first 2 * kLive lanes of each half of a fragment.  The other
    // lanes' values only reach result rows nobody reads, so they repeat a live lane's address
    // instead of fetching their own zeros: a fragment load then touches 2 * kLive * 32 bytes.
    const int lr = lj % (2 * kLive);
    const int alane = lh * 32 + lr;
    // The fragment and scale loads below have to be issued BEHIND the weight requests above (the wait for the first
    // fragment is what says that the first half of the weights has landed).  Their addresses are taken from pointers
    // that pass through a statement ordered after those requests, so no scheduling can lift them above.
    const uint32_t* qa_behind = qa;
    const float* sa_behind = sa;
    asm volatile("" : "+s"(qa_behind), "+s"(sa_behind) : : "memory");
    const bm_v4i* qa4 = reinterpret_cast<const bm_v4i*>(qa_behind);
    auto load_a = [&](int rt, int j) { return qa4[(static_cast<size_t>(rt) * kb_full + clamp_blk(j)) * 64 + alane]; };
    auto load_ta = [&](int rt, int p) { return sa_behind[static_cast<size_t>(clamp_blk(2 * p + lh)) * padded + rt * 32 + lr]; };
    bm_v4i afrag[kRowTiles][kAhead];
    float ta[kRowTiles][kPairs];  // activation scale of row lj, block 2p + lh
    constexpr int kHalfBlocks = kWB / 2, kHalfPairs = kPairs / 2;
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt)
#pragma unroll
        for (int j = 0; j < kAhead; ++j)
            if (j < kHalfBlocks) afrag[rt][j] = load_a(rt, j);
    // Weight scales, fp16 in block order: pair p needs block 2p + lh = half lh of dword p of the
    // wavefront's run of scales.  With rows of whole 16-byte runs (in_dim a multiple of 256) that is
    // one or two 16-byte loads per lane; otherwise one 2-byte load per pair.
    uint32_t tb_word[kPairs];
    {
        const int cc = min(n0 + lj, out_dim - 1);
        const uint16_t* sw = reinterpret_cast<const uint16_t*>(weight + blocks_total * kQB) + static_cast<size_t>(cc) * kb_full;
        if ((kb_full & 7) == 0) {
            // (reads past the wavefront's last valid block stay inside the scale regions; those pairs count for nothing)
            const uint4* run = reinterpret_cast<const uint4*>(sw + min(blk0, kb_full - 8));
#pragma unroll
            for (int q = 0; q < kPairs / 4; ++q) {
                const uint4 v = run[q];
                tb_word[4 * q] = v.x;
                tb_word[4 * q + 1] = v.y;
                tb_word[4 * q + 2] = v.z;
                tb_word[4 * q + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int p = 0; p < kPairs; ++p) tb_word[p] = static_cast<uint32_t>(sw[clamp_blk(2 * p + lh)]) * 0x10001u;
        }
    }
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt)
#pragma unroll
        for (int p = 0; p < kHalfPairs; ++p) ta[rt][p] = load_ta(rt, p);
    // ... and what only the second half needs (at least four loads)
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt)
#pragma unroll
        for (int j = kHalfBlocks; j < kAhead; ++j) afrag[rt][j] = load_a(rt, j);
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt)
#pragma unroll
        for (int p = kHalfPairs; p < kPairs; ++p) ta[rt][p] = load_ta(rt, p);
    // With a fragment ring shorter than half the blocks, fragments of the first half are still
    // requested inside the loop.  Loads complete in order: requested behind the second half of the
    // weights they would arrive behind it and the first half would be computed only after the
    // whole stream.  There the second half of the weights is requested from inside the loop, right
    // after the loads that complete the first half's fragments and the first ones of the second half's
    // (which are the loads the compiler's wait may retire early instead of the weights).
    constexpr int kIssuePair = kAhead >= kHalfBlocks ? -1 : (kHalfBlocks - kAhead) / 2;
    static_assert(kIssuePair >= 0 || kRowTiles * ((kAhead > kHalfBlocks ? kAhead - kHalfBlocks : 0) + kPairs - kHalfPairs) >= 4 || kType == 8,
                  "cover loads");
    if (kIssuePair < 0) issue_weights(1);

    // The first A fragment was requested behind the first half of the weights: once it is here, so
    // are they.  (The statement makes the compiler wait for that fragment and keeps the LDS reads
    // below it.)
    asm volatile("" : "+v"(afrag[0][0]) : : "memory");

    // this lane's fragment position inside a 1 KB load unit: column lj, chunk slot swizzled by the column
    const int frag_unit = lj >> 3;  // cg
    const int frag_row = (lj & 7) * 8, frag_swz = (lj >> 1) & 7;
    const uint4* wlds = reinterpret_cast<const uint4*>(bm_lds + wave * kBmWaveBytes);
    auto read_b = [&](int j) {
        int li, chunk;
        if (kType == 2) {
            li = (j >> 3) * 4 + frag_unit;
            chunk = j & 7;
        } else {
            li = (j >> 2) * 4 + frag_unit;
            chunk = (j & 3) * 2 + lh;
        }
        const uint4 w = wlds[li * 64 + frag_row + (chunk ^ frag_swz)];
        bm_v4i b;
        if (kType == 2) {
            // A nibble n stands for n - 8.  As the HIGH nibble of a byte, n ^ 8 reads as the int8
            // 16 * (n - 8): flip bit 3 of every nibble, move the wanted nibbles (low = values 0..15
            // = k half 0, high = values 16..31) to the high positions and clear the others.  The
            // dots come out multiplied by 16, which the weight scale takes back (exactly).
            const uint32_t sh = 4u * (1 - lh);
            b = bm_v4i{static_cast<int>(((w.x ^ 0x88888888u) << sh) & 0xF0F0F0F0u), static_cast<int>(((w.y ^ 0x88888888u) << sh) & 0xF0F0F0F0u),
                       static_cast<int>(((w.z ^ 0x88888888u) << sh) & 0xF0F0F0F0u), static_cast<int>(((w.w ^ 0x88888888u) << sh) & 0xF0F0F0F0u)};
        } else {
            b = bm_v4i{static_cast<int>(w.x), static_cast<int>(w.y), static_cast<int>(w.z), static_cast<int>(w.w)};
        }
        return b;
    };

    float acc[kRowTiles][kLive];
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt)
#pragma unroll
        for (int v = 0; v < kLive; ++v) acc[rt][v] = 0.0f;

    // ---- 3. the K loop of this wavefront: pairs of blocks, no barrier
    if (nb > 0) {
        const bm_v16i zi = {};
        const bm_v32f zf = {};
#pragma unroll
        for (int p = 0; p < kPairs; ++p) {
            // the second half of the weights (and every fragment requested so far) has to be here
            if (p == kHalfPairs) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            const bool live_blk = 2 * p + lh < nb;  // a clamped re-read of the last block counts for nothing
            const float tb = live_blk ? half_bits_to_f32(static_cast<uint16_t>(tb_word[p] >> (16 * lh))) * (kType == 2 ? 0.0625f : 1.0f) : 0.0f;
#pragma unroll
            for (int rt = 0; rt < kRowTiles; ++rt) {
                const bm_v4i a0 = afrag[rt][(2 * p) % kAhead], a1 = afrag[rt][(2 * p + 1) % kAhead];
                const bm_v32f t = __builtin_amdgcn_mfma_f32_32x32x1f32(live_blk ? ta[rt][p] : 0.0f, tb, zf, 0, 0, 0);
                // one block after the other: the second block's dots take the registers the first one's have left
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const bm_v4i a = h == 0 ? a0 : a1, b = read_b(2 * p + h);
                    bm_v16i c = zi;
                    c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < kLive; ++v) acc[rt][v] = __builtin_fmaf(t[16 * h + v], static_cast<float>(c[v]), acc[rt][v]);
                    fence_registers(acc[rt]);
                }
                // the fragments of blocks 2p, 2p + 1 are consumed: fetch the ones kAhead blocks on
                if (2 * p + kAhead < kWB) {
                    afrag[rt][(2 * p) % kAhead] = load_a(rt, 2 * p + kAhead);
                    afrag[rt][(2 * p + 1) % kAhead] = load_a(rt, 2 * p + 1 + kAhead);
                }
            }
            if (p == kIssuePair) issue_weights(1);
        }
    } else {
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // its weight loads still write LDS, which the sums are about to reuse
    }

    // ---- 4. the wavefronts' sums meet in LDS, one row tile at a time (the weight regions are dead
    // after the first barrier; 8 wavefronts x 16 registers x 64 lanes of floats are half the LDS)
    float* red = reinterpret_cast<float*>(bm_lds);  // [wave][v][lane]
    constexpr int kItems = kLive * 64;
#pragma unroll
    for (int rt = 0; rt < kRowTiles; ++rt) {
        __syncthreads();
#pragma unroll
        for (int v = 0; v < kLive; ++v) red[(wave * kLive + v) * 64 + lane] = acc[rt][v];
        __syncthreads();
        for (int i = tid; i < kItems; i += kBmThreads) {
            // the first four wavefronts' sums, the last four's, then both: what two K shares of four wavefronts each
            // add up to (launch_batch_mfma splits a single share there where that is faster, to the same bits)
            float half[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                half[h] = red[(kBmWaves / 2) * h * kItems + i];
#pragma unroll
                for (int w = 1; w < kBmWaves / 2; ++w) half[h] += red[((kBmWaves / 2) * h + w) * kItems + i];
            }
            const float sum = half[0] + half[1];
            const int l = i & 63, v = i >> 6;
            const int m = rt * 32 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3);
            const int n = n0 + (l & 31);
            if (m < rows && n < out_dim) {
                const size_t at = static_cast<size_t>(m) * out_dim + n;
                if (partial != nullptr) partial[static_cast<size_t>(blockIdx.y) * rows * out_dim + at] = sum;
                else if (accumulate) unsafeAtomicAdd(dst + at, sum);  // (two K shares, no epilogue, the result cleared beforehand: see batch8_mfma_kernel)
                else dst[at] = finish_output(ep, n, at, sum);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Up to eight rows: v_mfma_i32_16x16x64_i8 on two blocks at once.
//
// The instruction multiplies 16 rows x 64 k by 64 k x 16 columns, twice the k of one block, and two
// blocks cannot share an int32 sum (their scales differ).  With at most eight rows the A operand has
// room to keep them apart: A row 8 * s + r (s = 0, 1) is row r of X with the bytes of block 2P + s
// in its k half s and ZEROS in the other half, the B operand is the weights of block 2P in k half 0
// and of block 2P + 1 in k half 1.  Result row 8 * s + r is then exactly the dot of row r with block
// 2P + s: one instruction of a quarter of the 32x32x32 one's work gives the dots of two blocks for
// 16 columns, and all four of its result registers are live (lane l: column l % 16, lane group
// g = l / 16: block 2P + g / 2, rows 4 * (g % 2) + v).
//
// The scale products sx[row][block] * sw[column][block] come in the same register layout from one
// v_mfma_f32_16x16x4_f32: A row 8 * s + r carries sx of (r, block 2P + s) at k = s and zeros
// elsewhere, B row k carries sw of block 2P + k (k < 2): every entry is one product plus zeros,
// the correctly rounded f32 product.  What is left for the vector unit per MFMA is the nibble
// unpacking, four conversions and four fused multiply-adds; the LDS sees one read.  (Fetching the
// row scales per result register through the lane-exchange crossbar instead made the LDS pipe, one
// per compute unit, the bottleneck.)
//
// The smaller column granule also makes four load stages of a wavefront's eight 1 KB units instead
// of two: (blocks first half, columns 0..15), (first half, 16..31), (second half, 0..15), (second
// half, 16..31), each waited for by itself, so that a quarter of the arithmetic, not half, is left
// when the last byte arrives.

// X f32 [rows <= 8][in_dim] -> qa8: [pair P][32 entries][16 bytes], sa8: f32 [pair][16].
// Entry 16 * s + 8 * h + r holds sixteen int8 of row r, block 2P + s, k half h, in the k order of the
// weight operand (below): what lane 16 * (2 s + h) + 8 * s + r of the A operand needs; the other lanes
// of the operand are zeros and are not stored.  Slot 8 * s + r of sa8 is the block's scale.  Rows
// past `rows` and a block past the last one are zeros with scale 0.  Same scale, reciprocal and
// rounding as quantize_fragments_kernel.
// k order, lane half h = g % 2:  Q8_0: values [16 h, 16 h + 16).  Q4_0: dwords x[8h..8h+3],
// x[16+8h..+3], x[8h+4..8h+7], x[16+8h+4..+7] -- the low and the high nibbles of bytes [8 h, 8 h + 8) of
// the block, dword by dword, so that one lane unpacks whole bytes.
// zero_a (and zero_b): result arrays of zero_count floats that the matmul launch behind this one adds its two K shares'
// sums to; cleared here, by the launch that has to run first anyway.
template <int kType>
__global__ __launch_bounds__(256) void quantize_fragments8_kernel(const float* __restrict__ x, int rows, int in_dim,
                                                                   uint32_t* __restrict__ qa8, float* __restrict__ sa8,
                                                                   float* __restrict__ zero_a, float* __restrict__ zero_b, int zero_count) {
    const int kb = in_dim >> 5, slots = ((kb + 1) >> 1) * 2;  // block slots: whole pairs
    const int units = 8 * slots * 8;                           // (row, block slot, eight lanes)
    // blockIdx.y: the group of eight rows (rows 8 .. 15 of X make a second set of fragments and scales behind the first)
    const int group = blockIdx.y;
    x += static_cast<size_t>(group) * 8 * in_dim;
    rows -= 8 * group;
    qa8 += static_cast<size_t>(group) * (slots / 2) * 128;
    sa8 += static_cast<size_t>(group) * (slots / 2) * 16;
    if (zero_a != nullptr && group == 0) {
        for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < zero_count; i += gridDim.x * blockDim.x) {
            zero_a[i] = 0.0f;
            if (zero_b != nullptr) zero_b[i] = 0.0f;
        }
    }
    for (int u = blockIdx.x * blockDim.x + threadIdx.x; u < units; u += gridDim.x * blockDim.x) {
        const int j = u & 7, bs = (u >> 3) % slots, r = (u >> 3) / slots;
        const bool real = r < rows && bs < kb;
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (real) v = reinterpret_cast<const float4*>(x)[(static_cast<size_t>(r) * in_dim >> 2) + bs * 8 + j];
        float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        m = max_over_8(m);
        const float s = act_scale(m);
        const float inv = m == 0.0f ? 0.0f : 1.0f / s;
        const int q0 = act_quant(v.x, inv), q1 = act_quant(v.y, inv);
        const int q2 = act_quant(v.z, inv), q3 = act_quant(v.w, inv);
        const int pair = bs >> 1, hs = bs & 1, i = hs * 8 + r;
        // values [4 j, 4 j + 4) of the block: which 16-byte half, which dword of it
        const int h2 = kType == 2 ? (j >> 1) & 1 : j >> 2;
        const int dw = kType == 2 ? 2 * (j & 1) + (j >> 2) : j & 3;
        // entry 16 * s + 8 * h2 + r of the pair: sixteen bytes
        qa8[static_cast<size_t>(pair) * 128 + (16 * hs + 8 * h2 + r) * 4 + dw] = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
        if (j == 0) sa8[pair * 16 + i] = real ? s : 0.0f;
    }
}

// kStamps (bench.py --probe timeline8): the same code, but instead of results every wavefront stores eight readings of the
// 100 MHz clock at dst_a[8 * (8 * workgroup + wavefront)]: [0] entry, [1] .. [4] the first four stages' bytes there, [5] the last
// stage's, [6] K loop done, [7] after the workgroup's reduction.
// kFullCols: a workgroup takes all 16 kCG columns (`cols` is not looked at).
// accumulate: the launch has exactly two K shares and no epilogue; the result array has been cleared (by the quantizer's
// launch) and each share adds its sums with a float atomic -- no partial sums in scratch, no reduce launch behind.
// kHalves: stage rounds of a wavefront -- it owns kHalves runs of eight (Q4_0; four Q8_0) consecutive blocks, and a K share
// is 8 * kHalves of them: a longer K makes fewer shares (K = 14336 of Q4_0: two of 224 blocks at kHalves = 4 instead of
// four of 112), and two shares need no reduce launch.
// kGroups: groups of eight rows (one or two: nine to sixteen rows run every step's two MFMAs once per group on the same
// weight operand; the second group's fragments and row scales lie behind the first's).
template <int kType, int kCG, bool kStamps = false, bool kFullCols = false, int kHalves = 2, int kGroups = 1>
__global__ __launch_bounds__(kBmThreads, kGroups > 1 ? 2 : 4) void batch8_mfma_kernel(float* __restrict__ dst_a, float* __restrict__ partial_a,
                                                                     const uint32_t* __restrict__ qa8, const float* __restrict__ sa8,
                                                                     const uint8_t* __restrict__ weight_a, int rows, int in_dim, int out_dim,
                                                                     int share_blocks, int cols_arg, int accumulate, Epilogue ep_a, BmSecond second) {
    uint32_t stamp[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (kStamps) stamp[0] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
    using F = BmFormat<kType>;
    const bool is_b = blockIdx.z != 0;
    float* dst = is_b ? second.dst : dst_a;
    const uint8_t* weight = is_b ? second.weight : weight_a;
    const Epilogue ep = is_b ? second.ep : ep_a;
    float* partial = partial_a == nullptr ? nullptr : partial_a + (is_b ? static_cast<size_t>(gridDim.y) * rows * out_dim : 0);
    constexpr int kQB = F::kQuantBytes, kStageBlocks = F::kWaveBlocks / 2, kWB = kHalves * kStageBlocks;
    constexpr int kPairs = kWB / 2, kHalfPairs = kStageBlocks / 2;  // pairs of blocks: of the wavefront, of a stage
    constexpr int kCols = 16 * kCG, kStages = kHalves * kCG, kSteps = kStages * kHalfPairs;
    const int kb_full = in_dim >> 5, pairs_total = (kb_full + 1) >> 1;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, g = lane >> 4, par = g >> 1, kh = g & 1;  // column, lane group, block parity, k half
    // a workgroup's columns: `cols` of them, a multiple of 8 in (16 kCG - 16, 16 kCG] (the host picks what spreads the matrix
    // evenly over the compute units); the arithmetic runs on all 16 kCG, the last ones on a copy of column cols - 1
    const int cols = kFullCols ? 16 * kCG : cols_arg;
    const int n0 = blockIdx.x * cols;
    const int share_begin = static_cast<int>(blockIdx.y) * share_blocks;  // a multiple of kWB: even
    const int share_end = min(share_begin + share_blocks, kb_full);
    const int blk0 = share_begin + wave * kWB;
    const int nb = max(0, min(kWB, share_end - blk0));
    const int last = blk0 + max(nb, 1) - 1 < kb_full ? blk0 + max(nb, 1) - 1 : kb_full - 1;
    auto clamp_blk = [&](int j) { return min(blk0 + j, last); };
    const size_t blocks_total = static_cast<size_t>(out_dim) * kb_full;
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(bm_lds))) + wave * kBmWaveBytes;

    // ---- 1. loads.  Stage s = (half hb = s / kCG of the wavefront's blocks, column group cg =
    // s % kCG) is two 1 KB units of weights (8 columns x 8 chunks each), written to slot s % 4 of
    // the wavefront's 8 KB of LDS.  What a compute unit can keep in flight is a small part of what
    // its wavefronts want, and a wavefront that cannot issue a load cannot compute either, so a
    // wavefront requests two stages ahead of the one it works on, not everything at once.
    // Order of the requests (a compute unit has one address unit, all its wavefronts queue there and are
    // served in order): what the quantizer's launch left in the L2 -- the operand fragments in their compact form
    // (two pairs a load) and one or two 4-byte loads for the row scales of the wavefront's pairs -- for the whole
    // workgroup, a barrier, then the first stage, an 8-byte load per column group for the weight scales, two
    // spares; then the second stage.
    // A wavefront's loads complete in the order issued, so "all but the youngest n have completed"
    // says that a stage is there.  The compiler counts only its own loads when it waits for one of
    // them, which can only be too strict: it retires as many more of the oldest younger loads as
    // there are loads it does not know of (two at that point: the second stage).  The two spare
    // loads are those (they are looked at once, after the loop).
    auto issue_stage = [&](int st) {
        const int hb = st / kCG, cg = st % kCG;
        const uint8_t* wbase = weight + static_cast<size_t>(n0) * kb_full * kQB;
        const int c8 = lane >> 3, slot = lane & 7;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int c = 16 * cg + 8 * u + c8;
            const int chunk = slot ^ ((c >> 1) & 7);
            const int cc = min(n0 + min(c, cols - 1), out_dim - 1) - n0;
            uint32_t off;
            if (kType == 2) {
                off = (static_cast<uint32_t>(cc) * kb_full + clamp_blk(8 * hb + chunk)) * 16u;
            } else {
                off = (static_cast<uint32_t>(cc) * kb_full + clamp_blk(4 * hb + (chunk >> 1))) * 32u + (chunk & 1) * 16u;
            }
            bm_lds_load16(wbase, off, lds_wave + ((st & 3) * 2 + u) * 1024);
        }
    };
    const int pair0 = blk0 >> 1;
    // What comes from the L2 goes first, for the whole workgroup: the operand fragments and row scales (written by the
    // quantizer's launch, read by every workgroup) come back in a fraction of the time a weight byte takes, but a compute
    // unit serves its requests in the order issued -- behind the first weight requests they would wait for HBM.  One
    // barrier, reached within a few instructions, keeps every wavefront's weight requests behind all of these.
    // row scales: 64 bytes a pair; lane L of load q takes slot L % 16 of pair 4 q + L / 16
    // operand fragments, compact: 512 bytes a pair, two pairs a load; lane L of load q holds entry
    // L % 32 of pair 2 q + L / 32
    // (Inline assembly: the compiler may move its own loads from read-only memory across the barrier; waited for by
    // hand before the first stage is used.)
    constexpr int kScaleLoads = (kPairs + 3) / 4;
    float sx_part[kGroups][kScaleLoads];
    bm_v4i packed[kGroups][kPairs / 2];
    {
        uint32_t frag_off[kPairs / 2], scale_off[kScaleLoads];
#pragma unroll
        for (int q = 0; q < kPairs / 2; ++q) frag_off[q] = static_cast<uint32_t>(min(pair0 + 2 * q + (lane >> 5), pairs_total - 1) * 32 + (lane & 31)) * 16u;
#pragma unroll
        for (int q = 0; q < kScaleLoads; ++q) scale_off[q] = static_cast<uint32_t>(min(pair0 + 4 * q + g, pairs_total - 1) * 16 + l16) * 4u;
#pragma unroll
        for (int q = 0; q < kPairs / 2; ++q) asm volatile("" : "+v"(frag_off[q]));
#pragma unroll
        for (int q = 0; q < kScaleLoads; ++q) asm volatile("" : "+v"(scale_off[q]));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int grp = 0; grp < kGroups; ++grp) {
            const uint32_t* qa_g = qa8 + static_cast<size_t>(grp) * pairs_total * 128;
            const float* sa_g = sa8 + static_cast<size_t>(grp) * pairs_total * 16;
#pragma unroll
            for (int q = 0; q < kPairs / 2; ++q) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(packed[grp][q]) : "v"(frag_off[q]), "s"(qa_g) : "memory");
#pragma unroll
            for (int q = 0; q < kScaleLoads; ++q) asm volatile("global_load_dword %0, %1, %2" : "=v"(sx_part[grp][q]) : "v"(scale_off[q]), "s"(sa_g) : "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    // Weight scales, fp16 in block order (rows of whole 16-byte runs: the host sends no other shape here): word p of a
    // column's run holds blocks 2p and 2p + 1.
    // Tiles of three column groups and more: the workgroup's scales of this K share -- up to 64 columns x 256 bytes (Q4_0;
    // 128 for Q8_0) -- go through LDS.  Thread t fetches sixteen bytes (eight blocks) per round, sixteen (eight) threads a
    // column: whole 128-byte lines, each asked for once per workgroup and ahead of the first weight stage.  (A wavefront
    // fetching the scales of its own blocks of every column asks for 64 pieces of 32 (16) bytes; with the eight
    // wavefronts' 512 requests per compute unit a Q4_0 launch on 14336 columns took 0.4 us longer, a pair of them 0.9,
    // Q8_0 0.6.)  In LDS a column's chunks are stored at chunk ^ (column % chunks): the sixteen columns a step reads one
    // word of then sit in different banks.  Smaller tiles keep the register form (Q4_0, 16 columns on 4096: 7.14
    // against 7.26 us; Q8_0, 32 columns in 2.7 rounds on 11008: 15.6 against 16.1; Q4_0 24 columns on 6144: no difference).
    constexpr bool kScalesInLds = kCG >= 3 || kHalves > 2;
    constexpr int kChunks = kBmWaves * kWB / 8;
    constexpr int kScaleRounds = (16 * kCG * kChunks + kBmThreads - 1) / kBmThreads;  // rounds of the workgroup's threads over the tile's columns
    constexpr int kAheadStages = 2;  // requested beyond the stage being worked on (the ring has four slots)
    unsigned char* lds_scales = bm_lds + kBmLdsBytes;
    bm_v4i scale_run[kScaleRounds];
    if (kScalesInLds) {
        const uint8_t* sbase = weight + blocks_total * kQB + static_cast<size_t>(n0) * kb_full * 2;
        uint32_t run_off[kScaleRounds];
#pragma unroll
        for (int r = 0; r < kScaleRounds; ++r) {
            const int c = tid / kChunks + r * (kBmThreads / kChunks), chunk = tid % kChunks;
            const int cc = min(n0 + min(c, cols - 1), out_dim - 1) - n0;
            run_off[r] = static_cast<uint32_t>(cc * kb_full + min(share_begin + 8 * chunk, kb_full - 8)) * 2u;
            asm volatile("" : "+v"(run_off[r]));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < kScaleRounds; ++r) {
            scale_run[r] = bm_v4i{0, 0, 0, 0};
            if (tid / kChunks + r * (kBmThreads / kChunks) < 16 * kCG)
                asm volatile("global_load_dwordx4 %0, %1, %2" : "+v"(scale_run[r]) : "v"(run_off[r]), "s"(sbase) : "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    issue_stage(0);
    if (kScalesInLds) {
        // the scale runs are there when at most the first stage's two requests are in flight; the workgroup meets once they
        // are in LDS (the first stage is waited for behind that, with nothing else of the wavefront outstanding: behind
        // the second stage's requests the wait would also have to see those accepted by the memory pipeline, which for
        // the last wavefronts of a unit is well into the stream)
        asm volatile("s_waitcnt vmcnt(2)" : : : "memory");
#pragma unroll
        for (int r = 0; r < kScaleRounds; ++r) {
            asm volatile("" : "+v"(scale_run[r]));
            const int c = tid / kChunks + r * (kBmThreads / kChunks), chunk = tid % kChunks;
            if (c < 16 * kCG) *reinterpret_cast<bm_v4i*>(lds_scales + c * (kChunks * 16) + ((chunk ^ (c & (kChunks - 1))) << 4)) = scale_run[r];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
    // Q8_0: lane group g takes words [g * kWpl, +kWpl) of its wavefront's blocks and the lane exchange hands word p
    // out when its stage comes
    constexpr int kWpl = kPairs / 4;
    uint32_t tb_part[kCG][kWpl];
#pragma unroll
    for (int cg = 0; cg < (kScalesInLds ? 0 : kCG); ++cg) {
        const int cc = min(n0 + min(16 * cg + l16, cols - 1), out_dim - 1);
        const uint16_t* sw = reinterpret_cast<const uint16_t*>(weight + blocks_total * kQB) + static_cast<size_t>(cc) * kb_full;
        const uint32_t* run = reinterpret_cast<const uint32_t*>(sw + min(blk0, kb_full - 8)) + g * kWpl;
        if constexpr (kWpl == 2) {
            const uint2 v = *reinterpret_cast<const uint2*>(run);
            tb_part[cg][0] = v.x;
            tb_part[cg][1] = v.y;
        } else {
            tb_part[cg][0] = run[0];
        }
    }
    constexpr int kSpares = 2;
    uint32_t spare[kSpares] = {0, 0};
    if (!kScalesInLds) {  // (Q4_0 has no load of the compiler's left: nothing to keep its waits from)
#pragma unroll
        for (int k = 0; k < kSpares; ++k) spare[k] = __builtin_nontemporal_load(qa8 + k * 32 + (lane & 31));  // inside the first pair's entries
    }
    // Q4_0 asks for the second stage only when the first one and the register loads are there (below); Q8_0, whose
    // stages are half as many blocks, measured better with the second stage requested up front.
    constexpr bool kStartupAlone = kType == 2;
    if (!kStartupAlone) {
#pragma unroll
        for (int st = 1; st < kAheadStages; ++st) issue_stage(st);
    }

    // this lane's B operand: column 16 * cg + l16, block 2p + par, k half kh.  Q8_0: bytes
    // [16 kh, +16) of the block.  Q4_0: bytes [8 kh, +8), low nibbles and high nibbles dword by
    // dword; a nibble n stands for n - 8: with bit 3 flipped and in the high half of a byte it reads as
    // the int8 16 * (n - 8).  Its address inside a stage's slot (the column group does not enter:
    // 16 columns are two whole units and the swizzle repeats every 16 columns).
    uint32_t baddr[kHalfPairs];
#pragma unroll
    for (int q = 0; q < kHalfPairs; ++q) {
        const int j = 2 * q + par;
        const int unit = l16 >> 3, row = (l16 & 7) * 8, swz = (l16 >> 1) & 7;
        const int chunk = kType == 2 ? j : j * 2 + kh;
        baddr[q] = lds_wave + (unit * 64 + row + (chunk ^ swz)) * 16 + (kType == 2 ? 8 * kh : 0);
    }

    float acc[kGroups][kCG][4];
#pragma unroll
    for (int grp = 0; grp < kGroups; ++grp)
#pragma unroll
        for (int cg = 0; cg < kCG; ++cg)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[grp][cg][v] = 0.0f;

    // ---- 2. the stages, software-pipelined by hand over the steps (one step = a pair of blocks,
    // sixteen columns: one int8 MFMA and one scale-product MFMA).  A step's weight bytes are
    // requested from LDS one step ahead and its results are scaled one step behind, after the next
    // MFMAs have been issued: no step waits for the LDS or for the matrix unit's latency.  (The
    // weight bytes of a stage's first step cannot be requested before the stage is there.)  The
    // scheduling barriers keep the compiler from undoing that order.
    if (nb > 0) {
        typedef unsigned bm_v2u __attribute__((ext_vector_type(2)));
        typedef unsigned bm_v4u __attribute__((ext_vector_type(4)));
        typedef typename std::conditional<kType == 2, bm_v2u, bm_v4u>::type Raw;
        typedef float bm_v4f __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) const Raw LdsRaw;
        Raw raw[2];
        bm_v4i afrag[kGroups][kHalfPairs];
        float sxm[kGroups][kHalfPairs], tbm[kHalfPairs];
        bm_v4i cres[kGroups][2];
        bm_v4f tres[kGroups][2];
        auto stage_of = [&](int it) { return it / kHalfPairs; };
        auto fetch_weights = [&](int it) { raw[it & 1] = *reinterpret_cast<LdsRaw*>(baddr[it % kHalfPairs] + (stage_of(it) & 3) * 2048); };
        auto scale = [&](int it) {
            const int cg = stage_of(it) % kCG;
#pragma unroll
            for (int grp = 0; grp < kGroups; ++grp)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    acc[grp][cg][v] = __builtin_fmaf(tres[grp][it & 1][v], static_cast<float>(cres[grp][it & 1][v]), acc[grp][cg][v]);
        };
#pragma unroll
        for (int it = 0; it < kSteps; ++it) {
            if (it % kHalfPairs == 0) {
                const int st = stage_of(it), hb = st / kCG, cg = st % kCG;
                if (st == 0) {
                    if (kStartupAlone) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
                    else asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * (kAheadStages - 1)) : "memory");
#pragma unroll
                    for (int grp = 0; grp < kGroups; ++grp) {
#pragma unroll
                        for (int q = 0; q < kPairs / 2; ++q) asm volatile("" : "+v"(packed[grp][q]));
#pragma unroll
                        for (int q = 0; q < kScaleLoads; ++q) asm volatile("" : "+v"(sx_part[grp][q]));  // (one operand a statement: never the same register twice)
                    }
#pragma unroll
                    for (int c = 0; c < (kScalesInLds ? 0 : kCG); ++c)
#pragma unroll
                        for (int q = 0; q < kWpl; ++q) asm volatile("" : "+v"(tb_part[c][q]));
                }
                if (kStartupAlone && st == 0) {
#pragma unroll
                    for (int ahead = 1; ahead < kAheadStages; ++ahead) issue_stage(ahead);
                }
                if (st + kAheadStages < kStages) issue_stage(st + kAheadStages);
                // operands of this stage's scale products (in the shadow of the wait below).
                // A: lane (slot i = l16, k = g) carries sx of slot i if k is the slot's block (i / 8), else 0
                // B: lane (column l16, k = g) carries sw of block 2p + k for k < 2 (zero if that block is not
                //    this wavefront's: a clamped re-read of the last block counts for nothing), else 0;
                //    Q4_0: times 1/16, the nibbles enter the dots as 16 * (n - 8)
#pragma unroll
                for (int q = 0; q < kHalfPairs; ++q) {
                    const int p = hb * kHalfPairs + q;
                    uint32_t word;
                    if (kScalesInLds) {
                        const int c = 16 * cg + l16, pw = wave * kPairs + p;  // column of the tile, pair of the share
                        word = *reinterpret_cast<const uint32_t*>(lds_scales + c * (kChunks * 16) + (((pw >> 2) ^ (c & (kChunks - 1))) << 4) + ((pw & 3) << 2));
                    } else {
                        word = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(4 * (16 * (p / kWpl) + l16), static_cast<int>(tb_part[cg][p % kWpl])));
                    }
                    const float sw = half_bits_to_f32(static_cast<uint16_t>(word >> (16 * kh))) * (kType == 2 ? 0.0625f : 1.0f);
                    tbm[q] = (g < 2 && 2 * p + g < nb) ? sw : 0.0f;
                }
                if (cg == 0) {
                    // first stage of a half: the half's row scales and A operands.  Lane (g, slot i) takes
                    // entry 8 g + i % 8 of its pair through the lane exchange if the slot's block is the lane
                    // group's, else zeros
#pragma unroll
                    for (int grp = 0; grp < kGroups; ++grp)
#pragma unroll
                        for (int q = 0; q < kHalfPairs; ++q) {
                            const int p = hb * kHalfPairs + q;
                            const float sx = __int_as_float(__builtin_amdgcn_ds_bpermute(4 * (16 * (p & 3) + l16), __float_as_int(sx_part[grp][p >> 2])));
                            sxm[grp][q] = g == (l16 >> 3) ? sx : 0.0f;
                            const int from = 4 * (32 * (p & 1) + 8 * g + (l16 & 7));
#pragma unroll
                            for (int d = 0; d < 4; ++d) {
                                const int got = __builtin_amdgcn_ds_bpermute(from, packed[grp][p >> 1][d]);
                                afrag[grp][q][d] = (l16 >> 3) == par ? got : 0;
                            }
                        }
                }
                // this stage is there when at most the stages requested behind it are in flight
                {
                    const int younger = 2 * ((kStages - 1 - st) < kAheadStages ? (kStages - 1 - st) : kAheadStages);
                    if (younger == 6) asm volatile("s_waitcnt vmcnt(6)" : : : "memory");
                    else if (younger == 4) asm volatile("s_waitcnt vmcnt(4)" : : : "memory");
                    else if (younger == 2) asm volatile("s_waitcnt vmcnt(2)" : : : "memory");
                    else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
                }
                fetch_weights(it);
                if (kStamps && st < 4) stamp[1 + st] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
                if (kStamps && st == kStages - 1) stamp[5] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
            }
            __builtin_amdgcn_sched_barrier(0);
            if (it + 1 < kSteps && (it + 1) % kHalfPairs != 0) fetch_weights(it + 1);
            bm_v4i b;
            {
                const Raw w = raw[it & 1];
                if constexpr (kType == 2) {
                    const uint32_t x = w[0] ^ 0x88888888u, y = w[1] ^ 0x88888888u;
                    b = bm_v4i{static_cast<int>((x << 4) & 0xF0F0F0F0u), static_cast<int>(x & 0xF0F0F0F0u), static_cast<int>((y << 4) & 0xF0F0F0F0u),
                               static_cast<int>(y & 0xF0F0F0F0u)};
                } else {
                    b = bm_v4i{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[kType == 2 ? 0 : 2]), static_cast<int>(w[kType == 2 ? 1 : 3])};
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            const int q = it % kHalfPairs;
#pragma unroll
            for (int grp = 0; grp < kGroups; ++grp) {
                cres[grp][it & 1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afrag[grp][q], b, bm_v4i{0, 0, 0, 0}, 0, 0, 0);
                tres[grp][it & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(sxm[grp][q], tbm[q], bm_v4f{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (it > 0) scale(it - 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        scale(kSteps - 1);
        if (kStamps) stamp[6] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
    } else {
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // nothing may still be writing LDS when the region is reused
    }
    asm volatile("" : : "v"(spare[0]), "v"(spare[1]));

    // ---- 3. the wavefronts' sums (and the two block parities) meet in LDS
    float* red = reinterpret_cast<float*>(bm_lds);  // [wave][cg * 4 + v][lane], one group of rows at a time
#pragma unroll
    for (int grp = 0; grp < kGroups; ++grp) {
        __syncthreads();
#pragma unroll
        for (int cg = 0; cg < kCG; ++cg)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[(wave * kCG * 4 + cg * 4 + v) * 64 + lane] = acc[grp][cg][v];
        __syncthreads();
        if (tid < 8 * kCols) {
            const int m8 = tid / kCols, c = tid % kCols, m = 8 * grp + m8;
            const int item = ((c >> 4) * 4 + (m8 & 3)) * 64 + 16 * (m8 >> 2) + (c & 15);
            float sum = 0.0f;
#pragma unroll
            for (int w = 0; w < kBmWaves; ++w) sum += red[w * kCG * 256 + item] + red[w * kCG * 256 + item + 32];
            const int n = n0 + c;
            if (kStamps) {
                asm volatile("" : : "v"(sum));  // (keeps the arithmetic alive)
            } else if (m < rows && c < cols && n < out_dim) {
                const size_t at = static_cast<size_t>(m) * out_dim + n;
                if (partial != nullptr) partial[static_cast<size_t>(blockIdx.y) * rows * out_dim + at] = sum;
                // two K shares, no epilogue: both add to the zeroed result; 0 + a + b = 0 + b + a to the bit, whoever comes first
                else if (accumulate) unsafeAtomicAdd(dst + at, sum);
                else dst[at] = finish_output(ep, n, at, sum);
            }
        }
    }
    if (kStamps) {
        __syncthreads();
        stamp[7] = static_cast<uint32_t>(__builtin_amdgcn_s_memrealtime());
        if (lane == 0) {
            uint32_t* o = reinterpret_cast<uint32_t*>(dst_a) + (static_cast<size_t>(blockIdx.x) * kBmWaves + wave) * 8;
#pragma unroll
            for (int q = 0; q < 8; ++q) o[q] = stamp[q];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Nine to 64 rows (one or two row tiles) on a matrix wide enough for 64-column tiles: batch_mfma_kernel's arithmetic
// (v_mfma_i32_32x32x32_i8 per block, scale products of a pair of blocks from one
// v_mfma_f32_32x32x1_2b_f32, one convert and one multiply-add per live result register) with what
// the eight-row kernel showed to matter:
//   * 64 columns per workgroup (two groups of 32): the A fragments -- 16 KB per wavefront, as much
//     as the weights per 32 columns -- are read once for both groups, and there is one workgroup
//     per compute unit with the whole register file (no second workgroup to leave room for);
//   * weights staged: stage (half hb of the wavefront's blocks, column group cg) is four 1 KB
//     units in one of two 4 KB slots; a stage is requested when the stage two before it has been
//     computed, so one stage travels while one is worked on (requesting all at once leaves a
//     wavefront stuck issuing loads while the data it could work on is already there);
//   * the A fragments of the second half of the blocks are requested block by block during the
//     last stage that uses the first half's (behind the weight requests already out, in front of
//     the last one);
//   * a lane unpacks whole bytes of Q4_0 nibbles (low and high: 8 operations per block instead of
//     12; the fragments' k order follows, quantize_fragments_kernel<true>);
//   * the arithmetic of a pair of blocks is ordered by hand: both int8 MFMAs and the scale MFMA
//     first, then the conversions and multiply-adds of both blocks, with the next pair's LDS reads
//     in flight meanwhile.
template <int kType, int kRT, int kLive>
__global__ __launch_bounds__(kBmThreads, 2) void batch32_mfma_kernel(float* __restrict__ dst_a, float* __restrict__ partial_a,
                                                                      const uint32_t* __restrict__ qa, const float* __restrict__ sa,
                                                                      const uint8_t* __restrict__ weight_a, int rows, int in_dim, int out_dim,
                                                                      int share_blocks, Epilogue ep_a, BmSecond second, int accumulate) {
    using F = BmFormat<kType>;
    const bool is_b = blockIdx.z != 0;
    float* dst = is_b ? second.dst : dst_a;
    const uint8_t* weight = is_b ? second.weight : weight_a;
    const Epilogue ep = is_b ? second.ep : ep_a;
    float* partial = partial_a == nullptr ? nullptr : partial_a + (is_b ? static_cast<size_t>(gridDim.y) * rows * out_dim : 0);
    constexpr int kQB = F::kQuantBytes, kWB = F::kWaveBlocks, kHB = kWB / 2, kPairs = kWB / 2, kHalfPairs = kPairs / 2;
    const int kb_full = in_dim >> 5;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lj = lane & 31, lh = lane >> 5;
    const int n0 = blockIdx.x * 64;
    const int share_begin = static_cast<int>(blockIdx.y) * share_blocks;
    const int share_end = min(share_begin + share_blocks, kb_full);
    const int blk0 = share_begin + wave * kWB;
    const int nb = max(0, min(kWB, share_end - blk0));
    const int last = blk0 + max(nb, 1) - 1 < kb_full ? blk0 + max(nb, 1) - 1 : kb_full - 1;
    auto clamp_blk = [&](int j) { return min(blk0 + j, last); };
    const size_t blocks_total = static_cast<size_t>(out_dim) * kb_full;
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(bm_lds))) + wave * kBmWaveBytes;

    // stage st = 2 * hb + cg -> slot st % 2
    auto issue_stage = [&](int st) {
        const int hb = st >> 1, cg = st & 1;
        const uint8_t* wbase = weight + static_cast<size_t>(n0) * kb_full * kQB;
        const int c8 = lane >> 3, slot = lane & 7;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = 32 * cg + 8 * u + c8;
            const int chunk = slot ^ ((c >> 1) & 7);
            const int cc = min(n0 + c, out_dim - 1) - n0;
            uint32_t off;
            if (kType == 2) {
                off = (static_cast<uint32_t>(cc) * kb_full + clamp_blk(8 * hb + chunk)) * 16u;
            } else {
                off = (static_cast<uint32_t>(cc) * kb_full + clamp_blk(4 * hb + (chunk >> 1))) * 32u + (chunk & 1) * 16u;
            }
            bm_lds_load16(wbase, off, lds_wave + ((st & 1) * 4 + u) * 1024);
        }
    };
    issue_stage(0);
    // weight scales of both column groups (fp16, block order; rows of whole 16-byte runs): word p of a
    // column's run holds blocks 2p and 2p + 1
    uint32_t tb_word[2][kPairs];
#pragma unroll
    for (int cg = 0; cg < 2; ++cg) {
        const int cc = min(n0 + 32 * cg + lj, out_dim - 1);
        const uint16_t* sw = reinterpret_cast<const uint16_t*>(weight + blocks_total * kQB) + static_cast<size_t>(cc) * kb_full;
        const uint4* run = reinterpret_cast<const uint4*>(sw + min(blk0, kb_full - 8));
#pragma unroll
        for (int q = 0; q < kPairs / 4; ++q) {
            const uint4 v = run[q];
            tb_word[cg][4 * q] = v.x;
            tb_word[cg][4 * q + 1] = v.y;
            tb_word[cg][4 * q + 2] = v.z;
            tb_word[cg][4 * q + 3] = v.w;
        }
    }
    // A fragments and row scales of the first half of the blocks.  Rows that exist live in the first
    // 2 * kLive lanes of each half of a fragment; the other lanes repeat a live lane's address.
    const int lr = lj % (2 * kLive);
    const int alane = lh * 32 + lr;
    const bm_v4i* qa4 = reinterpret_cast<const bm_v4i*>(qa);
    auto load_a = [&](int rt, int j) { return qa4[(static_cast<size_t>(rt) * kb_full + clamp_blk(j)) * 64 + (rt + 1 < kRT ? lane : alane)]; };
    auto load_ta = [&](int rt, int p) { return sa[static_cast<size_t>(clamp_blk(2 * p + lh)) * (32 * kRT) + rt * 32 + (rt + 1 < kRT ? lj : lr)]; };
    bm_v4i afrag[kRT][kHB];
    float ta[kRT][kHalfPairs];
#pragma unroll
    for (int rt = 0; rt < kRT; ++rt) {
#pragma unroll
        for (int j = 0; j < kHB; ++j) afrag[rt][j] = load_a(rt, j);
#pragma unroll
        for (int p = 0; p < kHalfPairs; ++p) ta[rt][p] = load_ta(rt, p);
    }
    issue_stage(1);

    // this lane's B operand inside a slot: column lj of the group, block j of the half, k half lh
    uint32_t baddr[kHB];
#pragma unroll
    for (int j = 0; j < kHB; ++j) {
        const int unit = lj >> 3, row = (lj & 7) * 8, swz = (lj >> 1) & 7;
        const int chunk = kType == 2 ? j : 2 * j + lh;
        baddr[j] = lds_wave + (unit * 64 + row + (chunk ^ swz)) * 16 + (kType == 2 ? 8 * lh : 0);
    }
#pragma unroll
    for (int j = 0; j < kHB; ++j) asm volatile("" : "+v"(baddr[j]));

    // (a full row tile has all 16 result registers live; kLive counts those of the last one)
    float acc[2][kRT][16];
#pragma unroll
    for (int cg = 0; cg < 2; ++cg)
#pragma unroll
        for (int rt = 0; rt < kRT; ++rt)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[cg][rt][v] = 0.0f;

    if (nb > 0) {
        typedef unsigned bm_v2u __attribute__((ext_vector_type(2)));
        typedef unsigned bm_v4u __attribute__((ext_vector_type(4)));
        typedef typename std::conditional<kType == 2, bm_v2u, bm_v4u>::type Raw;
        typedef __attribute__((address_space(3))) const Raw LdsRaw;
        auto unpack = [&](const Raw& w) {
            bm_v4i b;
            if constexpr (kType == 2) {
                const uint32_t x = w[0] ^ 0x88888888u, y = w[1] ^ 0x88888888u;
                b = bm_v4i{static_cast<int>((x << 4) & 0xF0F0F0F0u), static_cast<int>(x & 0xF0F0F0F0u), static_cast<int>((y << 4) & 0xF0F0F0F0u),
                           static_cast<int>(y & 0xF0F0F0F0u)};
            } else {
                b = bm_v4i{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[kType == 2 ? 0 : 2]), static_cast<int>(w[kType == 2 ? 1 : 3])};
            }
            return b;
        };
        const bm_v16i zi = {};
        const bm_v32f zf = {};
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int hb = st >> 1, cg = st & 1;
            // this stage is there when at most the stage requested behind it is in flight
            if (st < 3) asm volatile("s_waitcnt vmcnt(4)" : : : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
            Raw raw0 = *reinterpret_cast<LdsRaw*>(baddr[0] + (st & 1) * 4096);
            Raw raw1 = *reinterpret_cast<LdsRaw*>(baddr[1] + (st & 1) * 4096);
            bm_v4i b0 = unpack(raw0), b1 = unpack(raw1);
            if (kHalfPairs > 1) {
                raw0 = *reinterpret_cast<LdsRaw*>(baddr[2] + (st & 1) * 4096);
                raw1 = *reinterpret_cast<LdsRaw*>(baddr[3] + (st & 1) * 4096);
            }
#pragma unroll
            for (int q = 0; q < kHalfPairs; ++q) {
                const int p = hb * kHalfPairs + q;
                const bool live_blk = 2 * p + lh < nb;  // a clamped re-read of the last block counts for nothing
                const float tb = live_blk ? half_bits_to_f32(static_cast<uint16_t>(tb_word[cg][p] >> (16 * lh))) * (kType == 2 ? 0.0625f : 1.0f) : 0.0f;
#pragma unroll
                for (int rt = 0; rt < kRT; ++rt) {
                    constexpr int kFull = 16;
                    const int live_regs = rt + 1 < kRT ? kFull : kLive;
                    __builtin_amdgcn_sched_barrier(0);
                    const bm_v32f t = __builtin_amdgcn_mfma_f32_32x32x1f32(live_blk ? ta[rt][q] : 0.0f, tb, zf, 0, 0, 0);
                    const bm_v16i c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(afrag[rt][2 * q], b0, zi, 0, 0, 0);
                    const bm_v16i c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(afrag[rt][2 * q + 1], b1, zi, 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (cg == 1 && hb == 0) {
                        // last use of the first half's fragments of this pair: the second half's take their place
                        afrag[rt][2 * q] = load_a(rt, kHB + 2 * q);
                        afrag[rt][2 * q + 1] = load_a(rt, kHB + 2 * q + 1);
                        ta[rt][q] = load_ta(rt, kHalfPairs + q);
                    }
                    // while the matrix unit works (last row tile: its operands are no longer needed): the next
                    // pair's weights out of their nibbles, the pair after that out of LDS
                    if (rt == kRT - 1 && q + 1 < kHalfPairs) {
                        b0 = unpack(raw0);
                        b1 = unpack(raw1);
                        if (q + 2 < kHalfPairs) {
                            raw0 = *reinterpret_cast<LdsRaw*>(baddr[(2 * q + 4) % kHB] + (st & 1) * 4096);
                            raw1 = *reinterpret_cast<LdsRaw*>(baddr[(2 * q + 5) % kHB] + (st & 1) * 4096);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int v = 0; v < kFull; ++v)
                        if (v < live_regs) acc[cg][rt][v] = __builtin_fmaf(t[v], static_cast<float>(c0[v]), acc[cg][rt][v]);
#pragma unroll
                    for (int v = 0; v < kFull; ++v)
                        if (v < live_regs) acc[cg][rt][v] = __builtin_fmaf(t[16 + v], static_cast<float>(c1[v]), acc[cg][rt][v]);
                    fence_registers(acc[cg][rt]);
                }
            }
            // the slot is free: the stage two on takes it
            if (st + 2 < 4) issue_stage(st + 2);
        }
    } else {
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // nothing may still be writing LDS when the region is reused
    }

    // ---- the wavefronts' sums meet in LDS, one row tile at a time: [wave][cg][v][lane] (8 x 2 x 16 x 64 floats = the whole 64 KB)
    float* red = reinterpret_cast<float*>(bm_lds);
    constexpr int kItems = 2 * 16 * 64;
#pragma unroll
    for (int rt = 0; rt < kRT; ++rt) {
        __syncthreads();
#pragma unroll
        for (int cg = 0; cg < 2; ++cg)
#pragma unroll
            for (int v = 0; v < 16; ++v) red[((wave * 2 + cg) * 16 + v) * 64 + lane] = acc[cg][rt][v];
        __syncthreads();
        for (int i = tid; i < kItems; i += kBmThreads) {
            const int l = i & 63, v = (i >> 6) & 15, cg = i >> 10;
            const int m = rt * 32 + 8 * (v >> 2) + 4 * (l >> 5) + (v & 3);
            const int n = n0 + 32 * cg + (l & 31);
            if (m < rows && n < out_dim) {
                float sum = red[i];
#pragma unroll
                for (int w = 1; w < kBmWaves; ++w) sum += red[w * kItems + i];
                const size_t at = static_cast<size_t>(m) * out_dim + n;
                if (partial != nullptr) partial[static_cast<size_t>(blockIdx.y) * rows * out_dim + at] = sum;
                else if (accumulate) unsafeAtomicAdd(dst + at, sum);  // (two K shares, no epilogue, the result cleared beforehand: see batch8_mfma_kernel)
                else dst[at] = finish_output(ep, n, at, sum);
            }
        }
    }
}

namespace {

template <int kType, int kRowTiles, int kLive>
hipError_t bm_launch(hipStream_t stream, float* dst, float* partial, const uint32_t* qa, const float* sa, const uint8_t* weight,
                     int rows, int in_dim, int out_dim, int shares, int share_blocks, const Epilogue& ep, const BmSecond& second, bool accumulate) {
    const dim3 grid(static_cast<unsigned>((out_dim + 31) / 32), static_cast<unsigned>(shares), second.weight ? 2u : 1u), block(kBmThreads);
    hipLaunchKernelGGL((batch_mfma_kernel<kType, kRowTiles, kLive>), grid, block, kBmLdsBytes, stream, dst,
                       shares > 1 && !accumulate ? partial : nullptr, qa, sa, weight, rows, in_dim, out_dim, share_blocks, ep, second, accumulate ? 1 : 0);
    return hipGetLastError();
}

template <int kType>
hipError_t bm_launch_rows(hipStream_t stream, float* dst, float* partial, const uint32_t* qa, const float* sa, const uint8_t* weight,
                          int rows, int in_dim, int out_dim, int shares, int share_blocks, const Epilogue& ep, const BmSecond& second, bool accumulate) {
#define AFHIP_BM(TILES, LIVE) \
    return bm_launch<kType, TILES, LIVE>(stream, dst, partial, qa, sa, weight, rows, in_dim, out_dim, shares, share_blocks, ep, second, accumulate)
    if (rows <= 8) AFHIP_BM(1, 4);
    if (rows <= 16) AFHIP_BM(1, 8);
    if (rows <= 24) AFHIP_BM(1, 12);
    if (rows <= 32) AFHIP_BM(1, 16);
    if (rows <= 64) AFHIP_BM(2, 16);
    if (rows <= 96) AFHIP_BM(3, 16);
    AFHIP_BM(4, 16);
#undef AFHIP_BM
}

// LDS of an eight-row launch: the wavefronts' rings, and for Q4_0 the workgroup's weight scales of one K share
static size_t bm8_lds_bytes(int tensor_type, int column_groups, int halves = 2) {
    const int share_blocks = (tensor_type == 2 ? BmFormat<2>::kShareBlocks : BmFormat<8>::kShareBlocks) / 2 * halves;
    return kBmLdsBytes + (column_groups >= 3 || halves > 2 ? 16 * column_groups * (share_blocks / 8) * 16 : 0);
}
// (raising a kernel's limit is sticky: once per instantiation)
template <typename Kernel>
static hipError_t bm_allow_large_lds(Kernel kernel, size_t lds, std::atomic<size_t>* limit) {
    if (lds <= limit->load(std::memory_order_acquire)) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e == hipSuccess) limit->store(160 * 1024, std::memory_order_release);
    return e;
}

template <int kType, int kCG, int kHalves, int kGroups>
hipError_t bm_launch8(hipStream_t stream, float* dst, float* partial, const uint32_t* qa, const float* sa, const uint8_t* weight, int rows,
                      int in_dim, int out_dim, int shares, int share_blocks, int cols, bool accumulate, const Epilogue& ep, const BmSecond& second) {
    const dim3 grid(static_cast<unsigned>((out_dim + cols - 1) / cols), static_cast<unsigned>(shares), second.weight ? 2u : 1u), block(kBmThreads);
    if (accumulate || shares == 1) partial = nullptr;
    const size_t lds = bm8_lds_bytes(kType, kCG, kHalves);
    static std::atomic<size_t> lds_limit[2] = {{64 * 1024}, {64 * 1024}};
    if (cols == 16 * kCG) {
        auto kernel = batch8_mfma_kernel<kType, kCG, false, true, kHalves, kGroups>;
        if (hipError_t e = bm_allow_large_lds(kernel, lds, &lds_limit[0]); e != hipSuccess) return e;
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, dst, partial, qa, sa, weight, rows, in_dim, out_dim, share_blocks, cols,
                           accumulate ? 1 : 0, ep, second);
    } else {
        auto kernel = batch8_mfma_kernel<kType, kCG, false, false, kHalves, kGroups>;
        if (hipError_t e = bm_allow_large_lds(kernel, lds, &lds_limit[1]); e != hipSuccess) return e;
        hipLaunchKernelGGL(kernel, grid, block, lds, stream, dst, partial, qa, sa, weight, rows, in_dim, out_dim, share_blocks, cols,
                           accumulate ? 1 : 0, ep, second);
    }
    return hipGetLastError();
}


// Column groups of sixteen a workgroup takes: four (64 columns: the activations' share of a
// workgroup's traffic and a wavefront's set-up halve) where that still gives most compute units a
// workgroup, else two.
int bm8_column_groups(int out_dim) { return (out_dim + 63) / 64 >= gemv_compute_units() * 3 / 4 ? 4 : 2; }

int bm_shares(int tensor_type, int in_dim) {
    const int share_max = tensor_type == 2 ? BmFormat<2>::kShareBlocks : BmFormat<8>::kShareBlocks;
    return (in_dim / 32 + share_max - 1) / share_max;
}

// The eight-row kernel's stage rounds per wavefront (its kHalves: 2 or 4, Q8_0 also 8) and the K shares that makes.
// The fewest rounds that leave at most two shares (two add to the result themselves, more need a reduce launch; with
// fewer, longer shares a workgroup takes fewer columns and fetches more operand fragments for them), else the most.
// One share instead of two where the two shares' grid of 64-column tiles would not fit the compute units in one round
// while a single share's may.  (A pair counts as one of its matrices and an epilogue does not enter: each half of a
// pair stays bit-identical to the single op, and an op with a bias to the plain op plus the bias.)
// Measured, five rows, against two rounds everywhere (us): Q4_0 K = 14336 x 4096 columns 11.7 against 13.8 (two shares
// instead of four), 11008 x 4096 11.4 against 13.4, 8192 x 28672 29.3 against 31.2, 28672 x 4096 19.3 against 22.4;
// Q8_0 4096 x 14336 (eight rows) 14.0 against 15.5 (one share in one round), 4096 x 11008 11.8 against 14.0,
// 8192 x 8192 15.1 against 22.3 (16.0 as one share), 14336 x 4096 14.4 against 19.3 (16.7 at four rounds).  Where two
// shares fit one round they stay: Q4_0 8192 x 8192 11.7 (12.6 as one share), 6144 x 4096 8.5 (9.4).
int bm8_halves(int tensor_type, int in_dim, int out_dim) {
    const long kb = in_dim / 32, base = (tensor_type == 2 ? BmFormat<2>::kShareBlocks : BmFormat<8>::kShareBlocks) / 2;
    const int most = tensor_type == 2 ? 4 : 8;
    const long tiles = (out_dim + 63) / 64;
    for (int h = 2; h <= most; h *= 2) {
        const long shares = (kb + h * base - 1) / (h * base);
        if (shares > 2) continue;
        if (shares == 2 && h < most && 2 * tiles > gemv_compute_units()) continue;
        return h;
    }
    return most;
}
int bm8_shares(int tensor_type, int in_dim, int halves) {
    const int share_max = (tensor_type == 2 ? BmFormat<2>::kShareBlocks : BmFormat<8>::kShareBlocks) / 2 * halves;
    return (in_dim / 32 + share_max - 1) / share_max;
}

// A single group of sixteen columns a workgroup: for a matrix whose 32-column tiles (times K shares) leave compute
// units idle while its 16-column tiles fill them in one round -- 4096 columns at K = 4096: 7.9 against 9.0 us on
// batch_mfma_kernel; with a second, partial round (6144 columns: 9.7 against 9.4) it does not pay.
bool bm8_one_column_group(size_t shares, size_t out_dim) {
    const size_t units = static_cast<size_t>(gemv_compute_units());
    const size_t narrow = (out_dim + 15) / 16 * shares;
    return (out_dim + 31) / 32 * shares < units && narrow >= units && narrow <= units + units / 8;
}

// Columns a workgroup of the eight-row kernel takes (a multiple of 8 up to 64).  Where some column count gives a grid of
// no more workgroups than compute units, the smallest such count: every unit gets one workgroup, or nearly every
// one, and none two.  Measured at five and eight rows against the rule below: 11008 columns (K = 4096) 10.6 us on 230
// workgroups of 48 columns against 12.2 on 344 of 32 (172 of 64: 11.6); K = 14336 x 4096 columns 14.7 on 64 x 4 K
// shares against 15.6 on 128 x 4; K = 8192 x 8192 columns 14.4 on 128 x 2 against 15.3 on 256 x 2; Q8_0 6144 columns
// 11.5 on 128 x 2 of 48 against 12.2 on 192 x 2; 14336 columns 12.1 .. 12.3 on 256 of 56 against 12.4 on 224 of 64.
// (A column count that is not a multiple of 16 leaves part of a workgroup's last column group idle.)
// Else the grid takes several rounds whatever the tile, and fewer, larger workgroups fetch the operand fragments less
// often: 64 columns from 12288 columns on, 16 where that is one round and a bit, else 32 (Q8_0, 14336 columns, two
// K shares: 18.0 us on 448 workgroups of 64 against 18.9 on 598 of 48; a pair of those 30.2 against 32.2).
int bm8_columns(long shares, int out_dim, bool pair) {
    const long units = gemv_compute_units();
    for (long cols = 8; cols <= 64; cols += 8)
        if ((out_dim + cols - 1) / cols * shares * (pair ? 2 : 1) <= units) return static_cast<int>(cols);
    if (bm8_column_groups(out_dim) == 4) return 64;
    return bm8_one_column_group(static_cast<size_t>(shares), static_cast<size_t>(out_dim)) ? 16 : 32;
}

template <int kType>
hipError_t bm_launch32(hipStream_t stream, float* dst, float* partial, const uint32_t* qa, const float* sa, const uint8_t* weight, int rows,
                       int in_dim, int out_dim, int shares, int share_blocks, const Epilogue& ep, const BmSecond& second, bool accumulate) {
    const dim3 grid(static_cast<unsigned>((out_dim + 63) / 64), static_cast<unsigned>(shares), second.weight ? 2u : 1u), block(kBmThreads);
#define AFHIP_BM32(RT, LIVE)                                                                                                                 \
    hipLaunchKernelGGL((batch32_mfma_kernel<kType, RT, LIVE>), grid, block, kBmLdsBytes, stream, dst, shares > 1 && !accumulate ? partial : nullptr, \
                       qa, sa, weight, rows, in_dim, out_dim, share_blocks, ep, second, accumulate ? 1 : 0)
    if (rows <= 16) AFHIP_BM32(1, 8);
    else if (rows <= 24) AFHIP_BM32(1, 12);
    else if (rows <= 32) AFHIP_BM32(1, 16);
    else AFHIP_BM32(2, 16);
#undef AFHIP_BM32
    return hipGetLastError();
}

}  // namespace

bool batch_mfma_supports(int tensor_type, size_t rows, size_t in_dim, size_t out_dim) {
    if (tensor_type != 2 && tensor_type != 8) return false;
    if (rows < 1 || rows > 128 || in_dim == 0 || in_dim % 32 != 0 || out_dim == 0) return false;
    // 32-bit lane offsets relative to a column tile, grid.y
    if (in_dim > (1u << 22) || out_dim > 0x7fffffff) return false;
    return true;
}

// The eight-row kernel: at most eight rows -- Q8_0 sixteen, as two groups of eight -- and rows of whole 16-byte runs of
// weight scales.  Nine and sixteen rows against the 32-row kernels (us): Q8_0 K = 4096 x 14336 columns 18.7 -> 15.4,
// 28672 columns 34.7 -> 26.4, K = 14336 x 4096 21.0 -> 16.1, K = N = 8192 23.5 -> 17.1, a pair of 14336 columns
// 35.0 -> 27.1, 4096 x 4096 8.7 -> 8.9, K = 2048 x 8192 columns 8.3 -> 8.8.  Q4_0, whose 32-row kernels are better (half
// the bytes per block, the same MFMA time), loses with two groups -- 14336 columns 13.3 -> 14.6, K = N = 8192
// 13.8 -> 14.7, 128256 columns 74 -> 84; 4096 columns 9.8 -> 9.2 and K = 14336 x 4096 16.8 -> 15.8 are the only gains --
// and keeps one there: a step's MFMAs of two groups (2 x (16 + 32) cycles a SIMD) take as long as its bytes.  On a K
// beyond 8192 and up to 8192 columns Q4_0 takes two groups too -- there the other kernels need three and more K shares
// and a reduce launch, this one two shares that add to the result themselves: sixteen rows, K = 14336 x 4096 columns
// 17.0 -> 15.9 us, 6144 columns 22.7 -> 19.3, 8192 columns 26.5 -> 22.7, a pair of 4096 columns 29.1 -> 22.8, K = 11008
// x 4096 15.9 -> 15.4, K = 28672 x 4096 27.2 -> 26.2 (14336 x 14336 columns loses: 39.3 -> 41.0).
// (It used to be kept to grids
// of at least a workgroup per compute unit; with its tiles sized to the matrix and its first requests in order it also
// wins below that: five rows, K = 4096, against batch_mfma_kernel: 6144 columns 8.5 against 9.6 us, 3072 6.8 against
// 9.0, 1024 6.6 against 8.7.)
bool batch_mfma_eight_rows(int tensor_type, size_t rows, size_t in_dim, size_t out_dim) {
    if (!batch_mfma_supports(tensor_type, rows, in_dim, out_dim)) return false;
    const bool sixteen = tensor_type == 8 || (in_dim > 8192 && out_dim <= 8192);
    return rows <= (sixteen ? 16u : 8u) && (in_dim / 32) % 8 == 0;
}

// Workspace: [qa: 32 * row_tiles * in_dim bytes][sa: (in_dim / 32) * 32 * row_tiles floats][partial sums of K shares, for two matrices]
size_t batch_mfma_workspace_bytes(int tensor_type, size_t rows, size_t in_dim, size_t out_dim) {
    if (!batch_mfma_supports(tensor_type, rows, in_dim, out_dim)) return 0;
    const size_t padded = (rows + 31) / 32 * 32;
    const size_t shares = static_cast<size_t>(bm_shares(tensor_type, static_cast<int>(in_dim)));
    const size_t front = padded * in_dim + (in_dim / 32) * padded * 4;
    return (front + 255) / 256 * 256 + (shares > 1 ? 2 * shares * rows * out_dim * 4 : 0);  // (twice: a pair of matrices)
}

// Largest grid the 32-row kernel is chosen for; negative: one workgroup per compute unit.
static std::atomic<long> batch32_bound{-1};
void set_batch32_max_workgroups(long bound) { batch32_bound.store(bound, std::memory_order_relaxed); }

hipError_t launch_batch_mfma(hipStream_t stream, int tensor_type, float* dst, const float* input, const uint8_t* weight_prepared,
                             int rows, int in_dim, int out_dim, uint8_t* workspace, float* dst_b,
                             const uint8_t* weight_b_prepared, const Epilogue& ep, const Epilogue& ep_b, void* quantizer_done) {
    if (!batch_mfma_supports(tensor_type, rows, in_dim, out_dim) || workspace == nullptr) return hipErrorInvalidValue;
    const int row_tiles = (rows + 31) / 32, padded = row_tiles * 32, kb = in_dim / 32;
    uint32_t* qa = reinterpret_cast<uint32_t*>(workspace);
    float* sa = reinterpret_cast<float*>(workspace + static_cast<size_t>(padded) * in_dim);
    const size_t front = static_cast<size_t>(padded) * in_dim + static_cast<size_t>(kb) * padded * 4;
    float* partial = reinterpret_cast<float*>(workspace + (front + 255) / 256 * 256);
    const bool eight = batch_mfma_eight_rows(tensor_type, rows, in_dim, out_dim);
    auto plain = [](const Epilogue& e) { return e.bias == nullptr && e.residual == nullptr && e.activation == kActNone; };
    const bool both_plain = plain(ep) && (weight_b_prepared == nullptr || plain(ep_b));
    const int halves = eight ? bm8_halves(tensor_type, in_dim, out_dim) : 2;
    const int shares = eight ? bm8_shares(tensor_type, in_dim, halves) : bm_shares(tensor_type, in_dim);
    // equal shares, whole wavefront slices: a multiple of the blocks one wavefront owns
    const int wave_blocks = (tensor_type == 2 ? BmFormat<2>::kWaveBlocks : BmFormat<8>::kWaveBlocks) / 2 * halves;
    int share_blocks = (kb + shares - 1) / shares;
    share_blocks = (share_blocks + wave_blocks - 1) / wave_blocks * wave_blocks;
    int real_shares = (kb + share_blocks - 1) / share_blocks;
    // Nine to 64 rows (rows of whole 16-byte runs of scales) where the 64-column tiles times the K shares (times two
    // for a pair) make a grid of five eighths of the compute units up to all of them: batch32_mfma_kernel holds one
    // workgroup per unit, and a second round of them costs more than batch_mfma_kernel's two resident workgroups per
    // unit (N = 20480: 21.1 against 18.5 us).  The grid counts, not the width: a long K on few columns qualifies through
    // its shares (sixteen rows, against batch_mfma_kernel: Q4_0 K = 14336 x 4096 columns 17.9 -> 17.0 us, 64 rows
    // 31.8 -> 27.6, K = N = 8192 15.7 -> 14.0, K = 8192 x 6144 columns 14.3 -> 13.0; Q8_0 K = 4096 x 8192 columns
    // 12.7 -> 11.1, K = 8192 x 4096 columns 15.4 -> 14.4).  Below: 160 and 172 workgroups (K = 4096, 10240 and 11008
    // columns) 13.8 -> 12.7 and 13.9 -> 12.8, Q8_0 160 (5120 columns) 11.0 -> 9.9; 128 workgroups lose (8192 columns
    // 10.6 -> 12.5).  set_batch32_max_workgroups overrides the bound (tests
    // reach the kernel's K shares and pair launches that way; 0 switches the kernel off).
    const long bound_set = batch32_bound.load(std::memory_order_relaxed);
    const long bound = bound_set >= 0 ? bound_set : gemv_compute_units();
    const long groups32 = static_cast<long>((out_dim + 63) / 64) * real_shares * (weight_b_prepared ? 2 : 1);
    const bool thirty_two = !eight && rows <= 64 && kb % 8 == 0 && groups32 >= gemv_compute_units() * 5 / 8 && groups32 <= bound;
    // batch_mfma_kernel on a K of one share that more than four of its wavefronts work on, few column tiles (at most
    // half the compute units' worth, one matrix counted) and no epilogue: two shares of four wavefronts each.  The
    // kernel adds its wavefronts' sums as (first four) + (last four), so the two shares' sums are exactly those halves
    // and the result has the same bits as the single share's (which a call with an epilogue keeps: no reduce launch
    // for it).  Four wavefronts a workgroup on twice the workgroups, sixteen rows: 4096 x 4096 columns 9.8 -> 8.8 us,
    // 2048 columns 9.3 -> 8.2, 48 rows 14.5 -> 12.8.  (Beyond one workgroup per compute unit it loses: 6144 columns
    // 10.1 -> 11.8, 8192 columns at 64 rows 15.7 -> 22.4.)
    if (!eight && !thirty_two && real_shares == 1 && both_plain && kb > (kBmWaves / 2) * wave_blocks &&
        2 * static_cast<long>((out_dim + 31) / 32) <= gemv_compute_units()) {
        share_blocks = (kBmWaves / 2) * wave_blocks;
        real_shares = 2;
    }
    // Two K shares and nothing to do to the sums but add them: the kernel's shares add to the result themselves
    // (cleared by the quantizer's launch), which saves the reduce launch -- two of them for a pair.
    const bool accumulate = real_shares == 2 && both_plain;
    const int groups = rows > 8 ? 2 : 1;  // (eight-row kernel) groups of eight rows
    if (eight) {  // its own operand layout: 512 + 64 bytes per pair of blocks and group of eight rows, inside the same region
        const int pairs = (kb + 1) / 2;
        sa = reinterpret_cast<float*>(workspace + static_cast<size_t>(groups) * pairs * 512);
        const int units = 8 * (2 * pairs) * 8;
        const dim3 qgrid(static_cast<unsigned>((units + 255) / 256), static_cast<unsigned>(groups));
        float* zero_a = accumulate ? dst : nullptr;
        float* zero_b = accumulate && weight_b_prepared ? dst_b : nullptr;
        const int zero_count = rows * out_dim;
        if (tensor_type == 2)
            hipLaunchKernelGGL(quantize_fragments8_kernel<2>, qgrid, dim3(256), 0, stream, input, rows, in_dim, qa, sa, zero_a, zero_b, zero_count);
        else
            hipLaunchKernelGGL(quantize_fragments8_kernel<8>, qgrid, dim3(256), 0, stream, input, rows, in_dim, qa, sa, zero_a, zero_b, zero_count);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    } else {
        const size_t units = static_cast<size_t>(padded) * (in_dim / 4);
        size_t grid = (units + 255) / 256;
        if (grid > 4096) grid = 4096;
        float* zero_a = accumulate ? dst : nullptr;
        float* zero_b = accumulate && weight_b_prepared ? dst_b : nullptr;
        const size_t zero_count = static_cast<size_t>(rows) * out_dim;
        if (thirty_two && tensor_type == 2)
            hipLaunchKernelGGL(quantize_fragments_kernel<true>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, input, rows, in_dim,
                               row_tiles, qa, sa, zero_a, zero_b, zero_count);
        else
            hipLaunchKernelGGL(quantize_fragments_kernel<false>, dim3(static_cast<unsigned>(grid)), dim3(256), 0, stream, input, rows, in_dim,
                               row_tiles, qa, sa, zero_a, zero_b, zero_count);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    }
    // (an op that is being timed: its activation-quantizer phase ends here)
    if (quantizer_done != nullptr) (void)hipEventRecord(static_cast<hipEvent_t>(quantizer_done), stream);
    const size_t count = static_cast<size_t>(rows) * out_dim;
    // a pair is one launch over both matrices (grid.z)
    const BmSecond second{dst_b, weight_b_prepared, ep_b};
    hipError_t e;
    if (eight) {
        const int cols = bm8_columns(real_shares, out_dim, weight_b_prepared != nullptr), cg = (cols + 15) / 16;
#define AFHIP_BM8(T, CG, H, G) bm_launch8<T, CG, H, G>(stream, dst, partial, qa, sa, weight_prepared, rows, in_dim, out_dim, real_shares, share_blocks, cols, accumulate, ep, second)
#define AFHIP_BM8_CG(T, H, G) (cg == 4 ? AFHIP_BM8(T, 4, H, G) : (cg == 3 ? AFHIP_BM8(T, 3, H, G) : (cg == 2 ? AFHIP_BM8(T, 2, H, G) : AFHIP_BM8(T, 1, H, G))))
#define AFHIP_BM8_G(T, H) (groups == 2 ? AFHIP_BM8_CG(T, H, 2) : AFHIP_BM8_CG(T, H, 1))
        // (Q4_0: two groups of rows only on a long K, which runs four stage rounds)
        if (tensor_type == 2) e = halves == 4 ? AFHIP_BM8_G(2, 4) : AFHIP_BM8_CG(2, 2, 1);
        else e = halves == 8 ? AFHIP_BM8_G(8, 8) : (halves == 4 ? AFHIP_BM8_G(8, 4) : AFHIP_BM8_G(8, 2));
#undef AFHIP_BM8_G
#undef AFHIP_BM8_CG
#undef AFHIP_BM8
    }
    else if (thirty_two)
        e = tensor_type == 2 ? bm_launch32<2>(stream, dst, partial, qa, sa, weight_prepared, rows, in_dim, out_dim, real_shares, share_blocks, ep, second, accumulate)
                             : bm_launch32<8>(stream, dst, partial, qa, sa, weight_prepared, rows, in_dim, out_dim, real_shares, share_blocks, ep, second, accumulate);
    else
        e = tensor_type == 2
                       ? bm_launch_rows<2>(stream, dst, partial, qa, sa, weight_prepared, rows, in_dim, out_dim, real_shares, share_blocks, ep, second, accumulate)
                       : bm_launch_rows<8>(stream, dst, partial, qa, sa, weight_prepared, rows, in_dim, out_dim, real_shares, share_blocks, ep, second, accumulate);
    if (e != hipSuccess) return e;
    if (real_shares > 1 && !accumulate) {
        e = launch_splitk_reduce(stream, dst, partial, count, out_dim, real_shares, ep);
        if (e != hipSuccess) return e;
        if (weight_b_prepared) {
            e = launch_splitk_reduce(stream, dst_b, partial + static_cast<size_t>(real_shares) * count, count, out_dim, real_shares, ep_b);
            if (e != hipSuccess) return e;
        }
    }
    return hipSuccess;
}

// The eight-row kernel's own timeline (Q4_0, one K share, a matrix the kernel takes in tiles of 49 .. 64 columns): the
// compact-fragment quantizer, then the kernel template with its stamps flag, which stores clock readings (32 bytes per
// wavefront, eight wavefronts a workgroup) into `stamps` instead of results.
hipError_t launch_batch8_timeline(hipStream_t stream, uint32_t* stamps, size_t stamps_bytes, const float* input,
                                  const uint8_t* weight_prepared, int rows, int in_dim, int out_dim, uint8_t* workspace, int* workgroups,
                                  int* columns) {
    const int kb = in_dim / 32;
    if (rows < 1 || rows > 8 || in_dim % 256 != 0 || kb > BmFormat<2>::kShareBlocks || workspace == nullptr || stamps == nullptr) return hipErrorInvalidValue;
    if (!batch_mfma_supports(2, rows, in_dim, out_dim)) return hipErrorInvalidValue;
    const int cols = bm8_columns(1, out_dim, false);
    if (cols <= 48) return hipErrorInvalidValue;
    const int groups = (out_dim + cols - 1) / cols;
    if (workgroups) *workgroups = groups;
    if (columns) *columns = cols;
    if (stamps_bytes < static_cast<size_t>(groups) * kBmWaves * 32) return hipErrorInvalidValue;
    uint32_t* qa = reinterpret_cast<uint32_t*>(workspace);
    const int pairs = (kb + 1) / 2;
    float* sa = reinterpret_cast<float*>(workspace + static_cast<size_t>(pairs) * 512);
    const int units = 8 * (2 * pairs) * 8;
    hipLaunchKernelGGL(quantize_fragments8_kernel<2>, dim3(static_cast<unsigned>((units + 255) / 256)), dim3(256), 0, stream, input, rows, in_dim, qa, sa,
                       static_cast<float*>(nullptr), static_cast<float*>(nullptr), 0);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    int share_blocks = (kb + BmFormat<2>::kWaveBlocks - 1) / BmFormat<2>::kWaveBlocks * BmFormat<2>::kWaveBlocks;
    static std::atomic<size_t> lds_limit{64 * 1024};
    if (hipError_t e = bm_allow_large_lds(batch8_mfma_kernel<2, 4, true>, bm8_lds_bytes(2, 4), &lds_limit); e != hipSuccess) return e;
    hipLaunchKernelGGL((batch8_mfma_kernel<2, 4, true>), dim3(static_cast<unsigned>(groups), 1, 1), dim3(kBmThreads), bm8_lds_bytes(2, 4), stream,
                       reinterpret_cast<float*>(stamps), static_cast<float*>(nullptr), qa, sa, weight_prepared, rows, in_dim, out_dim, share_blocks,
                       cols, 0, Epilogue{}, BmSecond{nullptr, nullptr, Epilogue{}});
    return hipGetLastError();
}

}  // namespace afhip
