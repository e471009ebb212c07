// Prefill GEMM (rows >= 9) on CDNA4 int8 MFMA, activation-quantized route
// (ops/native_compute.zig:13304-13478 for Q8_0, :23427-23775 for Q4_0):
//   dot[m][n][b] = sum_i qx[m][32b+i] * qw[n][32b+i]            (int32, exact)
//   y[m][n]      = sum_b (sx[m][b] * sw[n][b]) * f32(dot[m][n][b]), b ascending
//
// Per 32x32 output tile and per pair of blocks (b, b+1) a wavefront issues
//   2 x v_mfma_i32_32x32x32_i8     the int32 dots of block b and of block b+1
//   1 x v_mfma_f32_32x32x1_2b_f32  the scale products sx[m][b]*sw[n][b] of both
//                                  blocks (two rank-1 outer products; each entry
//                                  is the correctly rounded f32 product)
// and then one int->float conversion and one fused multiply-add per element and
// block on the vector ALU.  All three results share the 32x32 MFMA register
// layout, so the epilogue is element-wise.  The vector ALU work (2 operations per
// (m, n, block)) is what bounds this kernel, not the MFMA pipe.
//
// Workgroup tile = (32*kWavesM) rows x (32*kWavesN) columns, one 32x32 tile per
// wavefront.  The K loop moves in stages of four blocks (128 values): while one
// stage is consumed from LDS the next is in flight from global memory to
// registers (double-buffered LDS, one barrier per stage).  LDS keeps operands in
// MFMA fragment order -- [block][half][row][16 bytes] -- so fragment reads are
// unit-stride 128-bit reads; Q4_0 nibbles are expanded to int8 once, on the way
// into LDS.
//
// MFMA operands: A = activations (row = lane % 32 -> m), B = weights (column =
// lane % 32 -> n); lane / 32 selects bytes [16*(lane/32), +16) of the block.
// Result register v of a lane is row 8*(v/4) + 4*(lane/32) + v%4, column
// lane % 32, so stores are 128 bytes contiguous along n.
#include <hip/hip_runtime.h>

#include <cstdlib>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v32f __attribute__((ext_vector_type(32)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kStageBlocks = 4;  // 128 K-values per LDS stage
constexpr int kPrefetch = 2;     // stages in flight from global memory (even)

// One LDS stage.  Operand planes are [block][half] x rows of 16 bytes; a plane is
// padded by two rows so that the 16 lanes of a 128-bit store phase (2 rows x 8
// planes, or 4 rows x 4 plane pairs for Q4_0) fall into 16 different bank groups.
// Scale planes are padded by 16 floats for the same reason.
template <int kTM, int kTN>
struct GemmLds {
    static constexpr int kPlaneA = kTM + 2, kPlaneB = kTN + 2;
    static constexpr int kScaleA = kTM + 16, kScaleB = kTN + 16;
    int4 a[kStageBlocks * 2 * kPlaneA];
    int4 b[kStageBlocks * 2 * kPlaneB];
    float sx[kStageBlocks * kScaleA];
    float sw[kStageBlocks * kScaleB];
};

template <int kType, int kWavesM, int kWavesN, bool kWriteDots>
__global__ __launch_bounds__(64 * kWavesM * kWavesN) void gemm_i8_kernel(
    float* __restrict__ dst, int* __restrict__ dots, const int8_t* __restrict__ qx, const float* __restrict__ sx,
    const uint8_t* __restrict__ weight, int rows, int in_dim, int out_dim, int m_tiles, int n_tiles) {
    constexpr int kThreads = 64 * kWavesM * kWavesN;
    constexpr int kTM = 32 * kWavesM;
    constexpr int kTN = 32 * kWavesN;
    using Lds = GemmLds<kTM, kTN>;
    constexpr int kQuantBytes = kType == 2 ? 16 : 32;
    constexpr int kAChunks = kTM * 8;                        // 16-byte chunks of activations per stage
    constexpr int kBChunks = kTN * (kType == 2 ? 4 : 8);     // 16-byte chunks of weight bytes per stage
    constexpr int kALoads = (kAChunks + kThreads - 1) / kThreads;
    constexpr int kBLoads = (kBChunks + kThreads - 1) / kThreads;

    __shared__ GemmLds<kTM, kTN> lds[2];

    const int kb = in_dim >> 5;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / kWavesN, wn = wave % kWavesN;
    const int lj = lane & 31, lh = lane >> 5;

    // Workgroups that share a weight tile (same n tile, different m tiles) sit on
    // the same XCD (consecutive workgroup ids go round-robin over the 8 XCDs), so
    // each L2 reads every weight byte once.
    const int id = blockIdx.x;
    const int xcd = id & 7, slot = id >> 3;
    const int m_tile = slot % m_tiles;
    const int n_tile = (slot / m_tiles) * 8 + xcd;
    if (n_tile >= n_tiles) return;
    const int m0 = m_tile * kTM, n0 = n_tile * kTN;

    const size_t blocks = static_cast<size_t>(out_dim) * kb;
    const uint8_t* wq = weight;
    const uint16_t* wd = reinterpret_cast<const uint16_t*>(weight + blocks * kQuantBytes);

    // ---- staging registers
    constexpr int kSxLoads = (kStageBlocks * kTM + kThreads - 1) / kThreads;
    constexpr int kSwLoads = (kStageBlocks * kTN + kThreads - 1) / kThreads;
    // kPrefetch stages are in flight from global memory at any time (the latency of
    // one stage's loads is several stages of compute); nothing may consume a staged
    // value before store_stage.
    u32x4 ra[kPrefetch][kALoads], rb[kPrefetch][kBLoads];
    float rsx[kPrefetch][kSxLoads];
    uint16_t rsw[kPrefetch][kSwLoads];  // raw fp16 bits

    auto load_stage = [&](int set, int kb0) {
#pragma unroll
        for (int i = 0; i < kALoads; ++i) {
            const int q = tid + i * kThreads;
            if (kAChunks % kThreads == 0 || q < kAChunks) {
                const int r = q >> 3, c = q & 7;
                const int m = min(m0 + r, rows - 1);
                const int blk = min(kb0 + (c >> 1), kb - 1);
                ra[set][i] = *reinterpret_cast<const u32x4*>(qx + static_cast<size_t>(m) * in_dim + blk * 32 + (c & 1) * 16);
            }
        }
#pragma unroll
        for (int i = 0; i < kBLoads; ++i) {
            const int q = tid + i * kThreads;
            if (kBChunks % kThreads == 0 || q < kBChunks) {
                if (kType == 2) {
                    const int r = q >> 2, c = q & 3;
                    const int n = min(n0 + r, out_dim - 1);
                    const int blk = min(kb0 + c, kb - 1);
                    rb[set][i] = *reinterpret_cast<const u32x4*>(wq + (static_cast<size_t>(n) * kb + blk) * 16);
                } else {
                    const int r = q >> 3, c = q & 7;
                    const int n = min(n0 + r, out_dim - 1);
                    const int blk = min(kb0 + (c >> 1), kb - 1);
                    rb[set][i] = *reinterpret_cast<const u32x4*>(wq + (static_cast<size_t>(n) * kb + blk) * 32 + (c & 1) * 16);
                }
            }
        }
        // block scales, one (row, block) per load (clamped addresses; blocks past the
        // end are zeroed when the stage is written to LDS)
#pragma unroll
        for (int i = 0; i < kSxLoads; ++i) {
            const int t = min(tid + i * kThreads, kStageBlocks * kTM - 1);
            const int m = min(m0 + (t >> 2), rows - 1);
            rsx[set][i] = sx[static_cast<size_t>(m) * kb + min(kb0 + (t & 3), kb - 1)];
        }
#pragma unroll
        for (int i = 0; i < kSwLoads; ++i) {
            const int t = min(tid + i * kThreads, kStageBlocks * kTN - 1);
            const int n = min(n0 + (t >> 2), out_dim - 1);
            rsw[set][i] = wd[static_cast<size_t>(n) * kb + min(kb0 + (t & 3), kb - 1)];
        }
    };

    auto store_stage = [&](int set, int stage_kb0, GemmLds<kTM, kTN>& s) {
#pragma unroll
        for (int i = 0; i < kALoads; ++i) {
            const int q = tid + i * kThreads;
            if (kAChunks % kThreads == 0 || q < kAChunks) {
                const int r = q >> 3, c = q & 7;
                s.a[c * Lds::kPlaneA + r] = make_int4(ra[set][i].x, ra[set][i].y, ra[set][i].z, ra[set][i].w);
            }
        }
#pragma unroll
        for (int i = 0; i < kBLoads; ++i) {
            const int q = tid + i * kThreads;
            if (kBChunks % kThreads == 0 || q < kBChunks) {
                if (kType == 2) {
                    const int r = q >> 2, c = q & 3;
                    const uint32_t p[4] = {rb[set][i].x, rb[set][i].y, rb[set][i].z, rb[set][i].w};
                    int v[8];
                    unpack_q4(p, v);  // low nibbles = values 0..15 (half 0), high nibbles = 16..31 (half 1)
                    s.b[(c * 2 + 0) * Lds::kPlaneB + r] = make_int4(v[0], v[1], v[2], v[3]);
                    s.b[(c * 2 + 1) * Lds::kPlaneB + r] = make_int4(v[4], v[5], v[6], v[7]);
                } else {
                    const int r = q >> 3, c = q & 7;
                    s.b[c * Lds::kPlaneB + r] = make_int4(rb[set][i].x, rb[set][i].y, rb[set][i].z, rb[set][i].w);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kSxLoads; ++i) {
            const int t = tid + i * kThreads;
            if (t < kStageBlocks * kTM) s.sx[(t & 3) * Lds::kScaleA + (t >> 2)] = stage_kb0 + (t & 3) < kb ? rsx[set][i] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < kSwLoads; ++i) {
            const int t = tid + i * kThreads;
            if (t < kStageBlocks * kTN)
                s.sw[(t & 3) * Lds::kScaleB + (t >> 2)] = stage_kb0 + (t & 3) < kb ? half_bits_to_f32(rsw[set][i]) : 0.0f;
        }
    };

    float acc[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

    const int stages = (kb + kStageBlocks - 1) / kStageBlocks;
    // Loads are never predicated: past the last stage they re-read clamped addresses
    // and their scales are written as zero, so the loop body is straight-line code and
    // the compiler can wait for exactly the one stage it is about to store.
#pragma unroll
    for (int d = 0; d < kPrefetch; ++d) load_stage(d, d * kStageBlocks);
    store_stage(0, 0, lds[0]);
    __syncthreads();

    const int row = wm * 32 + lj;  // this lane's activation row (A operand) inside the tile
    const int col = wn * 32 + lj;  // this lane's weight column (B operand) inside the tile
    for (int st0 = 0; st0 < stages; st0 += kPrefetch) {
#pragma unroll
        for (int d = 0; d < kPrefetch; ++d) {
            const int st = st0 + d;  // may run past `stages` in the last round: zero scales, no effect
            const GemmLds<kTM, kTN>& cur = lds[d & 1];  // kPrefetch is even: stage st sits in buffer st & 1 == d & 1
            // register set d has just been written to LDS: refill it with the stage kPrefetch ahead
            load_stage(d, (st + kPrefetch) * kStageBlocks);
            __builtin_amdgcn_sched_barrier(0);

            // a real loop: one pair's MFMA results live at a time
#pragma unroll 1
            for (int pair = 0; pair < kStageBlocks / 2; ++pair) {
                const int b0 = 2 * pair, b1 = b0 + 1;
                const int4 a0v = cur.a[(b0 * 2 + lh) * Lds::kPlaneA + row], a1v = cur.a[(b1 * 2 + lh) * Lds::kPlaneA + row];
                const int4 w0v = cur.b[(b0 * 2 + lh) * Lds::kPlaneB + col], w1v = cur.b[(b1 * 2 + lh) * Lds::kPlaneB + col];
                // scale operands: lanes 0-31 carry block b0, lanes 32-63 block b1
                const float ta = cur.sx[(b0 + lh) * Lds::kScaleA + row];
                const float tb = cur.sw[(b0 + lh) * Lds::kScaleB + col];
                const v4i a0 = {a0v.x, a0v.y, a0v.z, a0v.w}, a1 = {a1v.x, a1v.y, a1v.z, a1v.w};
                const v4i w0 = {w0v.x, w0v.y, w0v.z, w0v.w}, w1 = {w1v.x, w1v.y, w1v.z, w1v.w};
                v16i c0 = {}, c1 = {};
                v32f t = {};
                c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, w0, c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, w1, c1, 0, 0, 0);
                t = __builtin_amdgcn_mfma_f32_32x32x1f32(ta, tb, t, 0, 0, 0);
                if (kWriteDots) {
                    const int blk = st * kStageBlocks + b0;
                    const int n = n0 + col;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                        if (m < rows && n < out_dim) {
                            int* dp = dots + (static_cast<size_t>(m) * out_dim + n) * kb;
                            if (blk < kb) dp[blk] = c0[v];
                            if (blk + 1 < kb) dp[blk + 1] = c1[v];
                        }
                    }
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = __builtin_fmaf(t[v], static_cast<float>(c0[v]), acc[v]);
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[v] = __builtin_fmaf(t[16 + v], static_cast<float>(c1[v]), acc[v]);
            }

            store_stage((d + 1) % kPrefetch, (st + 1) * kStageBlocks, lds[(d + 1) & 1]);
            __syncthreads();
        }
    }

    if (dst == nullptr) return;
    const int n = n0 + col;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
        if (m < rows && n < out_dim) dst[static_cast<size_t>(m) * out_dim + n] = acc[v];
    }
}

namespace {

template <int kType, int kWavesM, int kWavesN>
hipError_t launch_tile(hipStream_t stream, float* dst, int* dots, const int8_t* qx, const float* sx,
                       const uint8_t* weight, int rows, int in_dim, int out_dim) {
    constexpr int kTM = 32 * kWavesM, kTN = 32 * kWavesN;
    const int m_tiles = (rows + kTM - 1) / kTM;
    const int n_tiles = (out_dim + kTN - 1) / kTN;
    const int n_groups = (n_tiles + 7) / 8;
    const long long grid = static_cast<long long>(n_groups) * m_tiles * 8;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 g(static_cast<unsigned>(grid)), b(64 * kWavesM * kWavesN);
    if (dots)
        hipLaunchKernelGGL((gemm_i8_kernel<kType, kWavesM, kWavesN, true>), g, b, 0, stream, dst, dots, qx, sx, weight,
                           rows, in_dim, out_dim, m_tiles, n_tiles);
    else
        hipLaunchKernelGGL((gemm_i8_kernel<kType, kWavesM, kWavesN, false>), g, b, 0, stream, dst, dots, qx, sx, weight,
                           rows, in_dim, out_dim, m_tiles, n_tiles);
    return hipGetLastError();
}

template <int kType>
hipError_t launch_type(hipStream_t stream, float* dst, int* dots, const int8_t* qx, const float* sx,
                       const uint8_t* weight, int rows, int in_dim, int out_dim) {
    // 64 x 128 tiles (8 wavefronts) when they still give every CU a workgroup, 32 x 128 otherwise
    const long long big = static_cast<long long>((rows + 63) / 64) * ((out_dim + 127) / 128);
    static const char* force = std::getenv("AFHIP_GEMM_TILE");  // tuning: "L" = 64x128, "S" = 32x128
    const bool use_big = force ? force[0] == 'L' : big >= 256;
    if (force && force[0] == 'M') return launch_tile<kType, 2, 2>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim);
    if (force && force[0] == 'N') return launch_tile<kType, 1, 2>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim);
    if (use_big) return launch_tile<kType, 2, 4>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim);
    return launch_tile<kType, 1, 4>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim);
}

}  // namespace

hipError_t launch_gemm_i8(hipStream_t stream, int tensor_type, float* dst, int* dots, const int8_t* qx, const float* sx,
                          const uint8_t* weight_prepared, int rows, int in_dim, int out_dim) {
    if (tensor_type == 2) return launch_type<2>(stream, dst, dots, qx, sx, weight_prepared, rows, in_dim, out_dim);
    return launch_type<8>(stream, dst, dots, qx, sx, weight_prepared, rows, in_dim, out_dim);
}

}  // namespace afhip
