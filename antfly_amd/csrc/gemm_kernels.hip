// Prefill GEMM (rows >= 9) on CDNA4 int8 MFMA, activation-quantized route
// (ops/native_compute.zig:13304-13478 for Q8_0, :23427-23775 for Q4_0):
//   dot[m][n][b] = sum_i qx[m][32b+i] * qw[n][32b+i]            (int32, exact)
//   y[m][n]      = sum_b (sx[m][b] * sw[n][b]) * f32(dot[m][n][b]), b ascending
// One v_mfma_i32_32x32x32_i8 forms the 32x32 dots of one 32-value block, so each
// accumulator element takes one int->float conversion, one multiply for the
// scale product and one fused multiply-add per block.
//
// Workgroup tile = (32*kWavesM) rows x (32*kFragsN*kWavesN) columns; every
// wavefront owns 32 rows x 32*kFragsN columns.  The K loop moves in stages of
// four blocks (128 values): while one stage is consumed from LDS the next one is
// in flight from global memory to registers (double-buffered LDS, one barrier
// per stage).  LDS keeps operands in MFMA fragment order -- [block][half][row]
// [16 bytes] -- so fragment reads are unit-stride 128-bit reads, and Q4_0
// nibbles are expanded to int8 once, on the way into LDS.
//
// MFMA operands: A = activations (row = lane % 32 -> m), B = weights (column =
// lane % 32 -> n); both lanes of a pair hold bytes [16*(lane/32), +16) of the
// block.  Result register v of a lane is row 8*(v/4) + 4*(lane/32) + v%4,
// column lane % 32, so stores are 128 bytes contiguous along n.
#include <hip/hip_runtime.h>

#include "device_common.h"
#include "qmatmul_launch.h"

namespace afhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kStageBlocks = 4;  // 128 K-values per LDS stage

template <int kTM, int kTN>
struct GemmLds {
    // fragment-ordered operands and block scales of one stage
    int4 a[kStageBlocks * 2 * kTM];
    int4 b[kStageBlocks * 2 * kTN];
    float sx[kStageBlocks * kTM];
    float sw[kStageBlocks * kTN];
};

template <int kType, int kWavesM, int kWavesN, int kFragsN, bool kWriteDots>
__global__ __launch_bounds__(64 * kWavesM * kWavesN) void gemm_i8_kernel(
    float* __restrict__ dst, int* __restrict__ dots, const int8_t* __restrict__ qx, const float* __restrict__ sx,
    const uint8_t* __restrict__ weight, int rows, int in_dim, int out_dim, int m_tiles, int n_tiles) {
    constexpr int kThreads = 64 * kWavesM * kWavesN;
    constexpr int kTM = 32 * kWavesM;
    constexpr int kTN = 32 * kFragsN * kWavesN;
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
    u32x4 ra[kALoads], rb[kBLoads];
    float rsx[kSxLoads], rsw[kSwLoads];

    auto load_stage = [&](int kb0) {
#pragma unroll
        for (int i = 0; i < kALoads; ++i) {
            const int q = tid + i * kThreads;
            if (kAChunks % kThreads == 0 || q < kAChunks) {
                const int r = q >> 3, c = q & 7;
                const int m = min(m0 + r, rows - 1);
                const int blk = min(kb0 + (c >> 1), kb - 1);
                ra[i] = *reinterpret_cast<const u32x4*>(qx + static_cast<size_t>(m) * in_dim + blk * 32 + (c & 1) * 16);
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
                    rb[i] = *reinterpret_cast<const u32x4*>(wq + (static_cast<size_t>(n) * kb + blk) * 16);
                } else {
                    const int r = q >> 3, c = q & 7;
                    const int n = min(n0 + r, out_dim - 1);
                    const int blk = min(kb0 + (c >> 1), kb - 1);
                    rb[i] = *reinterpret_cast<const u32x4*>(wq + (static_cast<size_t>(n) * kb + blk) * 32 + (c & 1) * 16);
                }
            }
        }
        // block scales, one (row, block) per load; blocks past the end get scale 0
#pragma unroll
        for (int i = 0; i < kSxLoads; ++i) {
            const int t = tid + i * kThreads;
            const int r = t >> 2, c = t & 3;
            const int m = min(m0 + r, rows - 1);
            rsx[i] = (t < kStageBlocks * kTM && kb0 + c < kb) ? sx[static_cast<size_t>(m) * kb + kb0 + c] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < kSwLoads; ++i) {
            const int t = tid + i * kThreads;
            const int r = t >> 2, c = t & 3;
            const int n = min(n0 + r, out_dim - 1);
            rsw[i] = (t < kStageBlocks * kTN && kb0 + c < kb)
                         ? half_bits_to_f32(wd[static_cast<size_t>(n) * kb + kb0 + c]) : 0.0f;
        }
    };

    auto store_stage = [&](GemmLds<kTM, kTN>& s) {
#pragma unroll
        for (int i = 0; i < kALoads; ++i) {
            const int q = tid + i * kThreads;
            if (kAChunks % kThreads == 0 || q < kAChunks) {
                const int r = q >> 3, c = q & 7;
                s.a[((c >> 1) * 2 + (c & 1)) * kTM + r] = make_int4(ra[i].x, ra[i].y, ra[i].z, ra[i].w);
            }
        }
#pragma unroll
        for (int i = 0; i < kBLoads; ++i) {
            const int q = tid + i * kThreads;
            if (kBChunks % kThreads == 0 || q < kBChunks) {
                if (kType == 2) {
                    const int r = q >> 2, c = q & 3;
                    const uint32_t p[4] = {rb[i].x, rb[i].y, rb[i].z, rb[i].w};
                    int v[8];
                    unpack_q4(p, v);  // low nibbles = values 0..15 (half 0), high nibbles = 16..31 (half 1)
                    s.b[(c * 2 + 0) * kTN + r] = make_int4(v[0], v[1], v[2], v[3]);
                    s.b[(c * 2 + 1) * kTN + r] = make_int4(v[4], v[5], v[6], v[7]);
                } else {
                    const int r = q >> 3, c = q & 7;
                    s.b[((c >> 1) * 2 + (c & 1)) * kTN + r] = make_int4(rb[i].x, rb[i].y, rb[i].z, rb[i].w);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kSxLoads; ++i) {
            const int t = tid + i * kThreads;
            if (t < kStageBlocks * kTM) s.sx[(t & 3) * kTM + (t >> 2)] = rsx[i];
        }
#pragma unroll
        for (int i = 0; i < kSwLoads; ++i) {
            const int t = tid + i * kThreads;
            if (t < kStageBlocks * kTN) s.sw[(t & 3) * kTN + (t >> 2)] = rsw[i];
        }
    };

    float acc[kFragsN][16];
#pragma unroll
    for (int f = 0; f < kFragsN; ++f)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[f][v] = 0.0f;

    const int stages = (kb + kStageBlocks - 1) / kStageBlocks;
    load_stage(0);
    store_stage(lds[0]);
    __syncthreads();

    for (int st = 0; st < stages; ++st) {
        const GemmLds<kTM, kTN>& cur = lds[st & 1];
        if (st + 1 < stages) load_stage((st + 1) * kStageBlocks);

#pragma unroll
        for (int bb = 0; bb < kStageBlocks; ++bb) {
            const int4 av = cur.a[(bb * 2 + lh) * kTM + wm * 32 + lj];
            const v4i a = {av.x, av.y, av.z, av.w};
            float sxv[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 t = *reinterpret_cast<const float4*>(&cur.sx[bb * kTM + wm * 32 + 8 * q + 4 * lh]);
                sxv[4 * q + 0] = t.x; sxv[4 * q + 1] = t.y; sxv[4 * q + 2] = t.z; sxv[4 * q + 3] = t.w;
            }
#pragma unroll
            for (int f = 0; f < kFragsN; ++f) {
                const int col = (wn * kFragsN + f) * 32 + lj;
                const int4 bv = cur.b[(bb * 2 + lh) * kTN + col];
                const v4i b = {bv.x, bv.y, bv.z, bv.w};
                const float swl = cur.sw[bb * kTN + col];
                v16i c = {};
                c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
                if (kWriteDots) {
                    const int blk = st * kStageBlocks + bb;
                    const int n = n0 + col;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                        if (blk < kb && m < rows && n < out_dim)
                            dots[(static_cast<size_t>(m) * out_dim + n) * kb + blk] = c[v];
                    }
                }
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    acc[f][v] = __builtin_fmaf(sxv[v] * swl, static_cast<float>(c[v]), acc[f][v]);
            }
        }

        if (st + 1 < stages) store_stage(lds[(st + 1) & 1]);
        __syncthreads();
    }

    if (dst == nullptr) return;
#pragma unroll
    for (int f = 0; f < kFragsN; ++f) {
        const int n = n0 + (wn * kFragsN + f) * 32 + lj;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int m = m0 + wm * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (m < rows && n < out_dim) dst[static_cast<size_t>(m) * out_dim + n] = acc[f][v];
        }
    }
}

namespace {

template <int kType, int kWavesM, int kWavesN, int kFragsN>
hipError_t launch_tile(hipStream_t stream, float* dst, int* dots, const int8_t* qx, const float* sx,
                       const uint8_t* weight, int rows, int in_dim, int out_dim) {
    constexpr int kTM = 32 * kWavesM, kTN = 32 * kFragsN * kWavesN;
    const int m_tiles = (rows + kTM - 1) / kTM;
    const int n_tiles = (out_dim + kTN - 1) / kTN;
    const int n_groups = (n_tiles + 7) / 8;
    const long long grid = static_cast<long long>(n_groups) * m_tiles * 8;
    if (grid > 0x7fffffffLL) return hipErrorInvalidValue;
    dim3 g(static_cast<unsigned>(grid)), b(64 * kWavesM * kWavesN);
    if (dots)
        hipLaunchKernelGGL((gemm_i8_kernel<kType, kWavesM, kWavesN, kFragsN, true>), g, b, 0, stream, dst, dots, qx, sx,
                           weight, rows, in_dim, out_dim, m_tiles, n_tiles);
    else
        hipLaunchKernelGGL((gemm_i8_kernel<kType, kWavesM, kWavesN, kFragsN, false>), g, b, 0, stream, dst, dots, qx, sx,
                           weight, rows, in_dim, out_dim, m_tiles, n_tiles);
    return hipGetLastError();
}

template <int kType>
hipError_t launch_type(hipStream_t stream, float* dst, int* dots, const int8_t* qx, const float* sx,
                       const uint8_t* weight, int rows, int in_dim, int out_dim) {
    // 64 x 128 tiles when they still give every CU a workgroup, 32 x 128 otherwise
    const long long big = static_cast<long long>((rows + 63) / 64) * ((out_dim + 127) / 128);
    if (big >= 256) return launch_tile<kType, 2, 2, 2>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim);
    return launch_tile<kType, 1, 4, 1>(stream, dst, dots, qx, sx, weight, rows, in_dim, out_dim);
}

}  // namespace

hipError_t launch_gemm_i8(hipStream_t stream, int tensor_type, float* dst, int* dots, const int8_t* qx, const float* sx,
                          const uint8_t* weight_prepared, int rows, int in_dim, int out_dim) {
    if (tensor_type == 2) return launch_type<2>(stream, dst, dots, qx, sx, weight_prepared, rows, in_dim, out_dim);
    return launch_type<8>(stream, dst, dots, qx, sx, weight_prepared, rows, in_dim, out_dim);
}

}  // namespace afhip
